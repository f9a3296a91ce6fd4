"""Configuration of the Mafurax design, read from its own ``config.json`` layout.

``architecture`` names the design; ``vocab``, ``width``, ``logit_scale`` and ``norm.eps`` are the
model's; ``layers`` lists the layers in their order, each with its ``type`` (which mixer it has),
the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, null for none). Every
size and constant that can differ between two models of the design is a field here; sizes that
only a tensor's shape gives (the rows of a distance table, the rank of the decay's product) are
None until the tensors say, unless a configuration made for random weights names them.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from pyre_amd.config.model import ConfigError, ModelConfig


def _get(raw: dict, key: str, where: str, kind=(int, float)):
    if not isinstance(raw, dict) or key not in raw:
        raise ConfigError(f"config.json: {where} has no {key!r}")
    v = raw[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError(f"config.json: {where}.{key} must be a number, got {v!r}")
    return v


def _positive_int(raw: dict, key: str, where: str) -> int:
    v = _get(raw, key, where, int)
    if v <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    return v


@dataclass(frozen=True)
class CappedAttentionConfig:
    """The softmax branch ('left')."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float        #: 0: the scores are not squashed
    bias_max: float
    window: int           #: mask.size; 0: every earlier token is visible
    keep_first: int       #: mask.keep_first
    bias_rows: int | None = None

    @classmethod
    def from_dict(cls, raw, where):
        mask = raw.get("mask") or {}
        heads, kv = _positive_int(raw, "heads", where), _positive_int(raw, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: {where}.heads ({heads}) is not a multiple of kv_heads ({kv})")
        window = int(mask.get("size") or 0)
        keep = int(mask.get("keep_first") or 0)
        if window < 0 or keep < 0:
            raise ConfigError(f"config.json: {where}.mask must not be negative")
        rows = raw.get("bias_rows")
        return cls(heads, kv, _positive_int(raw, "dim", where), _positive_int(raw, "vdim", where),
                   float(_get(raw, "scale", where)), float(raw.get("softcap") or 0.0), float(_get(raw, "bias_max", where)),
                   window, keep, None if rows is None else int(rows))

    def to_dict(self):
        out = {"bias_max": self.bias_max, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
               "mask": {"keep_first": self.keep_first, "size": self.window}, "scale": self.scale,
               "softcap": self.softcap, "vdim": self.vdim}
        if self.bias_rows is not None:
            out["bias_rows"] = self.bias_rows
        return out


@dataclass(frozen=True)
class GatedLinearConfig:
    """The recurrent branch ('right')."""

    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int | None = None

    @classmethod
    def from_dict(cls, raw, where):
        tau = float(_get(raw, "tau", where))
        if not (tau > 0):
            raise ConfigError(f"config.json: {where}.tau must be positive")
        rank = raw.get("rank")
        return cls(_positive_int(raw, "heads", where), _positive_int(raw, "dim", where),
                   _positive_int(raw, "vdim", where), tau, None if rank is None else int(rank))

    def to_dict(self):
        out = {"dim": self.dim, "heads": self.heads, "tau": self.tau, "vdim": self.vdim}
        if self.rank is not None:
            out["rank"] = self.rank
        return out


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: CappedAttentionConfig
    right: GatedLinearConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, raw, where):
        for k in ("left", "right"):
            if not isinstance(raw.get(k), dict):
                raise ConfigError(f"config.json: {where} has no {k!r}")
        return cls(CappedAttentionConfig.from_dict(raw["left"], f"{where}.left"),
                   GatedLinearConfig.from_dict(raw["right"], f"{where}.right"),
                   float(_get(raw, "left_scale", where)), float(_get(raw, "right_scale", where)))

    def to_dict(self):
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class DenseFeedForwardConfig:
    ff: int
    limit: float
    kind: ClassVar[str] = "dense"

    @classmethod
    def from_dict(cls, raw, where):
        return cls(_positive_int(raw, "ff", where), float(_get(raw, "limit", where)))

    def to_dict(self):
        return {"ff": self.ff, "kind": self.kind, "limit": self.limit}


MIXER_CONFIGS = {"parallel": ParallelMixerConfig}
FEED_FORWARD_CONFIGS = {"dense": DenseFeedForwardConfig}


@dataclass(frozen=True)
class MafuraxLayerConfig:
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
class MafuraxConfig(ModelConfig):
    architecture: ClassVar[str] = "Mafurax"

    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    logit_scale: float = 1.0

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
    def from_dict(cls, raw: dict[str, Any]) -> "MafuraxConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json has no 'layers' list")
        return cls(vocab=_positive_int(raw, "vocab", "config"), width=_positive_int(raw, "width", "config"),
                   layers=tuple(MafuraxLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(layers)),
                   norm_eps=float(_get(raw.get("norm"), "eps", "norm")), logit_scale=float(raw.get("logit_scale", 1.0)))

    def to_dict(self) -> dict[str, Any]:
        return {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
