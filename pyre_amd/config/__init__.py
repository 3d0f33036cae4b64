from pyre_amd.config.durelix import DurelixConfig
from pyre_amd.config.engine import EngineConfig
from pyre_amd.config.mafurax import MafuraxConfig
from pyre_amd.config.nurasun import NurasunConfig
from pyre_amd.config.model import ConfigError, ModelConfig, Qwen2Config
from pyre_amd.config.presets import PRESETS, preset
from pyre_amd.config.zorulix import ZorulixConfig

__all__ = ["ConfigError", "DurelixConfig", "EngineConfig", "MafuraxConfig", "ModelConfig", "NurasunConfig", "Qwen2Config", "PRESETS", "preset", "ZorulixConfig"]
