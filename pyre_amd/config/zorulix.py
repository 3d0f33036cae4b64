"""Configuration of the Zorulix design, read from its own ``config.json`` layout.

``architecture`` names the design; ``vocab``, ``width`` and ``norm.eps`` are the model's, ``embedding.scale`` the factor
on the embedding's rows, ``token_side.dim`` the columns of the second token table that every layer takes (absent: the
layers have no such input); ``layers`` lists the layers in their order, each with its ``type`` (which mixer it has), the
mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, null for none). Every size and constant that can
differ between two models of the design is a field here; what a configuration does not mention is not there (no
``rot``: no rotation; no ``rot.scaling``: plain frequencies; no ``mask``: plain causal attention; no ``shared``: no
shared expert; no ``kv_from``: keys and values of the layer's own).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from pyre_amd.config.mafurax import _get, _positive_int
from pyre_amd.config.model import ConfigError, ModelConfig


@dataclass(frozen=True)
class RotConfig:
    """Rotation of the first ``dims`` elements of a head, element e with e + dims / 2; ``scaling`` = (factor, original,
    fast, slow) stretches the slow frequencies, or None."""

    base: float
    dims: int
    scaling: tuple | None = None

    @classmethod
    def from_dict(cls, raw, dim: int, where: str):
        if not raw:
            return None
        base, dims = float(_get(raw, "base", where)), _positive_int(raw, "dims", where)
        if dims % 2 or dims > dim or not (base > 0) or base == 1.0:
            raise ConfigError(f"config.json: {where}.dims ({dims}) must be even and within dim ({dim}), the base positive "
                              "and not one")
        scaling = None
        sc = raw.get("scaling")
        if sc:
            w = f"{where}.scaling"
            scaling = (float(_get(sc, "factor", w)), float(_get(sc, "original", w)), float(_get(sc, "fast", w)),
                       float(_get(sc, "slow", w)))
            if not all(x > 0 for x in scaling):
                raise ConfigError(f"config.json: {w}: factor, original, fast and slow must be positive")
        return cls(base, dims, scaling)

    def to_dict(self):
        out: dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            factor, original, fast, slow = self.scaling
            out["scaling"] = {"factor": factor, "fast": fast, "original": original, "slow": slow}
        return out


@dataclass(frozen=True)
class AttentionConfig:
    """Grouped softmax attention over a window: the mixer of an 'attention' layer and the left branch of a 'parallel'
    one."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0              #: mask.size; 0: every earlier token is visible
    rot: RotConfig | None = None
    kv_from: int | None = None   #: the layer whose keys and values this one reads instead of making its own

    @classmethod
    def from_dict(cls, raw, where):
        heads, kv = _positive_int(raw, "heads", where), _positive_int(raw, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: {where}.heads ({heads}) is not a multiple of kv_heads ({kv})")
        dim = _positive_int(raw, "dim", where)
        window = int((raw.get("mask") or {}).get("size") or 0)
        if window < 0:
            raise ConfigError(f"config.json: {where}.mask.size must not be negative")
        src = raw.get("kv_from")
        if src is not None and (isinstance(src, bool) or not isinstance(src, int) or src < 0):
            raise ConfigError(f"config.json: {where}.kv_from must be the number of a layer, got {src!r}")
        return cls(heads, kv, dim, _positive_int(raw, "vdim", where), float(_get(raw, "scale", where)), window,
                   RotConfig.from_dict(raw.get("rot"), dim, f"{where}.rot"), src)

    def to_dict(self):
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                               "vdim": self.vdim}
        if self.window:
            out["mask"] = {"size": self.window}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class DeltaRuleConfig:
    """The recurrent branch ('right'): ``heads`` value heads of ``vdim``, ``kv_heads`` query/key heads of ``dim``, a short
    convolution of ``conv`` taps."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, raw, where):
        heads, kv = _positive_int(raw, "heads", where), _positive_int(raw, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: {where}.heads ({heads}) is not a multiple of kv_heads ({kv})")
        return cls(heads, kv, _positive_int(raw, "dim", where), _positive_int(raw, "vdim", where),
                   _positive_int(raw, "conv", where))

    def to_dict(self):
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class ParallelConfig:
    left: AttentionConfig
    right: DeltaRuleConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, raw, where):
        for k in ("left", "right"):
            if not isinstance(raw.get(k), dict):
                raise ConfigError(f"config.json: {where} has no {k!r}")
        left = AttentionConfig.from_dict(raw["left"], f"{where}.left")
        if left.kv_from is not None:
            raise ConfigError(f"config.json: {where}.left: a branch makes its own keys and values")
        return cls(left, DeltaRuleConfig.from_dict(raw["right"], f"{where}.right"),
                   float(_get(raw, "left_scale", where)), float(_get(raw, "right_scale", where)))

    def to_dict(self):
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class MixtureConfig:
    experts: int
    top: int
    expert_ff: int
    shared_ff: int = 0    #: 0: no shared expert
    kind: ClassVar[str] = "moe"

    @classmethod
    def from_dict(cls, raw, where):
        router, expert = raw.get("router"), raw.get("expert")
        experts, top = _positive_int(router, "experts", f"{where}.router"), _positive_int(router, "top", f"{where}.router")
        if top > experts:
            raise ConfigError(f"config.json: {where}.router.top ({top}) exceeds the experts ({experts})")
        shared = raw.get("shared")
        return cls(experts, top, _positive_int(expert, "ff", f"{where}.expert"),
                   _positive_int(shared, "ff", f"{where}.shared") if shared else 0)

    def to_dict(self):
        out: dict[str, Any] = {"expert": {"ff": self.expert_ff}, "kind": self.kind,
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


MIXER_CONFIGS = {"attention": AttentionConfig, "parallel": ParallelConfig}
FEED_FORWARD_CONFIGS = {"moe": MixtureConfig}


@dataclass(frozen=True)
class ZorulixLayerConfig:
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
class ZorulixConfig(ModelConfig):
    architecture: ClassVar[str] = "Zorulix"

    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    embedding_scale: float = 1.0
    side_dim: int = 0     #: columns of the second token table that every layer takes; 0: no such input

    def __post_init__(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab and width must be positive and there must be a layer")
        if not (self.norm_eps > 0):
            raise ConfigError(f"norm.eps must be positive, got {self.norm_eps!r}")
        if self.side_dim < 0:
            raise ConfigError("token_side.dim must not be negative")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            src = getattr(m, "kv_from", None)
            if src is None:
                continue
            other = self.layers[src].mixer if src < i else None
            if not isinstance(other, AttentionConfig) or other.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from names layer {src}, which is no earlier attention layer with "
                                  "keys and values of its own")
            if (other.heads, other.kv_heads, other.dim, other.vdim, other.rot) != (m.heads, m.kv_heads, m.dim, m.vdim, m.rot):
                raise ConfigError(f"layers[{i}].mixer reads the keys and values of layer {src}, whose heads, sizes or "
                                  "rotation differ from its own")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "ZorulixConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json has no 'layers' list")
        emb, side = raw.get("embedding") or {}, raw.get("token_side") or {}
        return cls(vocab=_positive_int(raw, "vocab", "config"), width=_positive_int(raw, "width", "config"),
                   layers=tuple(ZorulixLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(layers)),
                   norm_eps=float(_get(raw.get("norm"), "eps", "norm")),
                   embedding_scale=float(_get(emb, "scale", "embedding")) if "scale" in emb else 1.0,
                   side_dim=_positive_int(side, "dim", "token_side") if side else 0)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                               "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
                               "vocab": self.vocab, "width": self.width}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        return out
