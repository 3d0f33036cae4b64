"""Configuration of the Durelix design, read from its own ``config.json`` layout.

``architecture`` names the design; ``vocab``, ``width`` and ``norm.eps`` are the model's, ``embedding.bigram`` the
constants of the second embedding table (absent: the model has none); ``layers`` lists the layers in their order, each
with its ``type`` (which mixer it has), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, null
for none). Every size and constant that can differ between two models of the design is a field here; what a
configuration does not mention is not there (no ``conv``: no convolution; no ``rot``: no rotation; no ``mask``: plain
causal attention; no ``groups``: one group; no ``identity``: no identity experts).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from pyre_amd.config.mafurax import _get, _positive_int
from pyre_amd.config.model import ConfigError, ModelConfig


def _rot(raw, dim: int, where: str) -> tuple[float, int]:
    """(base, turned elements) of a mixer's ``rot`` entry; (0, 0) if it has none."""
    rot = raw.get("rot")
    if not rot:
        return 0.0, 0
    base, dims = float(_get(rot, "base", f"{where}.rot")), _positive_int(rot, "dims", f"{where}.rot")
    if dims % 2 or dims > dim or not (base > 0):
        raise ConfigError(f"config.json: {where}.rot.dims ({dims}) must be even and within dim ({dim}), the base positive")
    return base, dims


def _rot_dict(base: float, dims: int) -> dict:
    return {"rot": {"base": base, "dims": dims}} if dims else {}


@dataclass(frozen=True)
class SinkAttentionConfig:
    """The softmax branch ('left')."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0       #: mask.size; 0: every earlier token is visible
    conv: int = 0         #: taps of the short convolution; 0: none
    rot_base: float = 0.0
    rot_dims: int = 0     #: 0: no rotation

    @classmethod
    def from_dict(cls, raw, where):
        heads, kv = _positive_int(raw, "heads", where), _positive_int(raw, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: {where}.heads ({heads}) is not a multiple of kv_heads ({kv})")
        dim = _positive_int(raw, "dim", where)
        window = int((raw.get("mask") or {}).get("size") or 0)
        conv = int(raw.get("conv") or 0)
        if window < 0 or conv < 0:
            raise ConfigError(f"config.json: {where}.mask.size and conv must not be negative")
        base, dims = _rot(raw, dim, where)
        return cls(heads, kv, dim, _positive_int(raw, "vdim", where), float(_get(raw, "scale", where)), window, conv,
                   base, dims)

    def to_dict(self):
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                               "vdim": self.vdim, **_rot_dict(self.rot_base, self.rot_dims)}
        if self.window:
            out["mask"] = {"size": self.window}
        if self.conv:
            out["conv"] = self.conv
        return out


@dataclass(frozen=True)
class RetentionConfig:
    """The recurrent branch ('right')."""

    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot_base: float = 0.0
    rot_dims: int = 0

    @classmethod
    def from_dict(cls, raw, where):
        heads, dim = _positive_int(raw, "heads", where), _positive_int(raw, "dim", where)
        decay = raw.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or \
                not all(isinstance(d, (int, float)) and not isinstance(d, bool) and 0 < d <= 1 for d in decay):
            raise ConfigError(f"config.json: {where}.decay must list one number in (0, 1] per head ({heads})")
        base, dims = _rot(raw, dim, where)
        return cls(heads, dim, _positive_int(raw, "vdim", where), tuple(float(d) for d in decay), base, dims)

    def to_dict(self):
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim,
                **_rot_dict(self.rot_base, self.rot_dims)}


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: SinkAttentionConfig
    right: RetentionConfig

    @classmethod
    def from_dict(cls, raw, where):
        for k in ("left", "right"):
            if not isinstance(raw.get(k), dict):
                raise ConfigError(f"config.json: {where} has no {k!r}")
        return cls(SinkAttentionConfig.from_dict(raw["left"], f"{where}.left"),
                   RetentionConfig.from_dict(raw["right"], f"{where}.right"))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class DenseConfig:
    ff: int
    kind: ClassVar[str] = "dense"

    @classmethod
    def from_dict(cls, raw, where):
        return cls(_positive_int(raw, "ff", where))

    def to_dict(self):
        return {"ff": self.ff, "kind": self.kind}


@dataclass(frozen=True)
class MixtureConfig:
    experts: int          #: experts with matrices
    top: int
    expert_ff: int
    identity: int = 0     #: experts behind them that hand their input back
    groups: int = 1
    keep_groups: int = 1
    kind: ClassVar[str] = "moe"

    @classmethod
    def from_dict(cls, raw, where):
        router, expert = raw.get("router"), raw.get("expert")
        experts, top = _positive_int(router, "experts", f"{where}.router"), _positive_int(router, "top", f"{where}.router")
        identity = int(router.get("identity") or 0)
        g = router.get("groups") or {}
        groups, keep = int(g.get("count") or 1), int(g.get("keep") or 1)
        total = experts + identity
        if identity < 0 or groups <= 0 or total % groups or not (0 < keep <= groups):
            raise ConfigError(f"config.json: {where}.router: {total} experts do not form {groups} equal groups of which "
                              f"{keep} are kept")
        if top > keep * (total // groups):
            raise ConfigError(f"config.json: {where}.router.top ({top}) exceeds the experts of the kept groups")
        return cls(experts, top, _positive_int(expert, "ff", f"{where}.expert"), identity, groups, keep)

    def to_dict(self):
        router: dict[str, Any] = {"experts": self.experts, "top": self.top}
        if self.identity:
            router["identity"] = self.identity
        if self.groups != 1 or self.keep_groups != 1:
            router["groups"] = {"count": self.groups, "keep": self.keep_groups}
        return {"expert": {"ff": self.expert_ff}, "kind": self.kind, "router": router}


@dataclass(frozen=True)
class BigramConfig:
    buckets: int
    mul_prev: int
    mul_cur: int

    @classmethod
    def from_dict(cls, raw, where):
        out = cls(_positive_int(raw, "buckets", where), _get(raw, "mul_prev", where, int), _get(raw, "mul_cur", where, int))
        if out.mul_prev < 0 or out.mul_cur < 0:
            raise ConfigError(f"config.json: {where}: the multipliers must not be negative")
        return out

    def to_dict(self):
        return {"buckets": self.buckets, "mul_cur": self.mul_cur, "mul_prev": self.mul_prev}


MIXER_CONFIGS = {"parallel": ParallelMixerConfig}
FEED_FORWARD_CONFIGS = {"dense": DenseConfig, "moe": MixtureConfig}


@dataclass(frozen=True)
class DurelixLayerConfig:
    type: str
    mixer: Any
    mlp: Any = None

    @classmethod
    def from_dict(cls, raw, where):
        kind = raw.get("type") if isinstance(raw, dict) else None
        if kind not in MIXER_CONFIGS:
            raise ConfigError(f"config.json: {where}.type is {kind!r}; known: {sorted(MIXER_CONFIGS)}")
        if not isinstance(raw.get("mixer"), dict):
            raise ConfigError(f"config.json: {where} has no 'mixer'")
        mlp = raw.get("mlp")
        if mlp is not None:
            ff_kind = mlp.get("kind") if isinstance(mlp, dict) else None
            if ff_kind not in FEED_FORWARD_CONFIGS:
                raise ConfigError(f"config.json: {where}.mlp.kind is {ff_kind!r}; known: {sorted(FEED_FORWARD_CONFIGS)}")
            mlp = FEED_FORWARD_CONFIGS[ff_kind].from_dict(mlp, f"{where}.mlp")
        return cls(kind, MIXER_CONFIGS[kind].from_dict(raw["mixer"], f"{where}.mixer"), mlp)

    def to_dict(self):
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class DurelixConfig(ModelConfig):
    architecture: ClassVar[str] = "Durelix"

    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    bigram: BigramConfig | None = None

    def __post_init__(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab and width must be positive and there must be a layer")
        if not (self.norm_eps > 0):
            raise ConfigError(f"norm.eps must be positive, got {self.norm_eps!r}")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "DurelixConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json has no 'layers' list")
        bigram = (raw.get("embedding") or {}).get("bigram")
        return cls(vocab=_positive_int(raw, "vocab", "config"), width=_positive_int(raw, "width", "config"),
                   layers=tuple(DurelixLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(layers)),
                   norm_eps=float(_get(raw.get("norm"), "eps", "norm")),
                   bigram=BigramConfig.from_dict(bigram, "embedding.bigram") if bigram else None)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                               "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.bigram is not None:
            out["embedding"] = {"bigram": self.bigram.to_dict()}
        return out
