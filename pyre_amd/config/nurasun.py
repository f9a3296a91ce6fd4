"""Configuration of the Nurasun design, read from its own ``config.json`` layout.

``architecture`` names the design; ``vocab``, ``width``, ``residual_mult``, ``logit_softcap`` and ``norm.eps`` are
the model's; ``layers`` lists the layers in their order, each with its ``type`` (which mixer it has), the mixer's
sizes and constants (``mixer``) and its feed-forward (``mlp``, null for none). Every size and constant that can
differ between two models of the design is a field here. What a configuration does not mention is not there: no
``mask`` is plain causal attention, no ``rot`` no rotation, no ``shared`` no shared expert, no ``logit_softcap``
unsquashed logits.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from pyre_amd.config.mafurax import _get, _positive_int
from pyre_amd.config.model import ConfigError, ModelConfig


def _scale(raw, dim: int, where: str) -> float:
    """The factor on the scores: the configuration's, or 1 / sqrt(dim) where it names none."""
    scale = float(_get(raw, "scale", where)) if "scale" in raw else dim ** -0.5
    if not (scale > 0):
        raise ConfigError(f"config.json: {where}.scale must be positive")
    return scale


@dataclass(frozen=True)
class TiedAttentionConfig:
    """'attention': grouped heads, values tied to the keys, rotation of part of a head, runs of positions."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int = 0           #: mask.size; 0: every earlier token is visible
    rot_dims: int = 0        #: rot.dims; 0: no rotation
    rot_base: float = 10000.0

    @classmethod
    def from_dict(cls, raw, where):
        heads = _positive_int(raw, "heads", where)
        kv = _positive_int(raw, "kv_heads", where) if "kv_heads" in raw else heads   # not mentioned: a key head per query head
        if heads % kv:
            raise ConfigError(f"config.json: {where}.heads ({heads}) is not a multiple of kv_heads ({kv})")
        dim = _positive_int(raw, "dim", where)
        vdim = int(raw.get("vdim", dim))
        if vdim != dim:
            raise ConfigError(f"config.json: {where}.vdim ({vdim}) differs from dim ({dim}), but the values are the keys")
        mask, rot = raw.get("mask") or {}, raw.get("rot") or {}
        chunk, dims = int(mask.get("size") or 0), int(rot.get("dims") or 0)
        if chunk < 0 or dims < 0 or dims % 2 or dims > dim:
            raise ConfigError(f"config.json: {where}: mask.size {chunk} / rot.dims {dims} do not fit heads of {dim}")
        base = float(rot.get("base", 10000.0))
        if dims and not (base > 0):
            raise ConfigError(f"config.json: {where}.rot.base must be positive")
        return cls(heads, kv, dim, vdim, _scale(raw, dim, where), chunk, dims, base)

    def to_dict(self):
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                               "vdim": self.vdim}
        if self.chunk:
            out["mask"] = {"size": self.chunk}
        if self.rot_dims:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return out


@dataclass(frozen=True)
class LatentAttentionConfig:
    """'latent_attention': one compressed row per token; ``kv_from`` names the layer whose rows this one reads."""

    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    kv_from: int | None = None

    @classmethod
    def from_dict(cls, raw, where):
        src = raw.get("kv_from")
        if src is not None and (isinstance(src, bool) or not isinstance(src, int) or src < 0):
            raise ConfigError(f"config.json: {where}.kv_from must name a layer, got {src!r}")
        dim = _positive_int(raw, "dim", where)
        return cls(_positive_int(raw, "heads", where), dim, _positive_int(raw, "vdim", where) if "vdim" in raw else dim,
                   _positive_int(raw, "kv_rank", where), _scale(raw, dim, where), src)

    def to_dict(self):
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "scale": self.scale,
                               "vdim": self.vdim}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


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
    experts: int
    top: int
    expert_ff: int
    shared_ff: int = 0       #: 0: no shared expert
    kind: ClassVar[str] = "moe"

    @classmethod
    def from_dict(cls, raw, where):
        router, expert, shared = raw.get("router"), raw.get("expert"), raw.get("shared")
        experts, top = _positive_int(router, "experts", f"{where}.router"), _positive_int(router, "top", f"{where}.router")
        if top > experts:
            raise ConfigError(f"config.json: {where}.router.top ({top}) exceeds experts ({experts})")
        return cls(experts, top, _positive_int(expert, "ff", f"{where}.expert"),
                   _positive_int(shared, "ff", f"{where}.shared") if shared else 0)

    def to_dict(self):
        out: dict[str, Any] = {"expert": {"ff": self.expert_ff}, "kind": self.kind,
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


MIXER_CONFIGS = {"attention": TiedAttentionConfig, "latent_attention": LatentAttentionConfig}
FEED_FORWARD_CONFIGS = {"dense": DenseConfig, "moe": MixtureConfig}


@dataclass(frozen=True)
class NurasunLayerConfig:
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
class NurasunConfig(ModelConfig):
    architecture: ClassVar[str] = "Nurasun"

    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    residual_mult: float = 1.0
    logit_softcap: float = 0.0

    def __post_init__(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab and width must be positive and there must be a layer")
        if not (self.norm_eps > 0):
            raise ConfigError(f"norm.eps must be positive, got {self.norm_eps!r}")
        if self.logit_softcap < 0:
            raise ConfigError("logit_softcap must not be negative")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, LatentAttentionConfig) and m.kv_from is not None:
                src = self.layers[m.kv_from].mixer if m.kv_from < i else None
                if not isinstance(src, LatentAttentionConfig) or src.kv_from is not None or src.kv_rank != m.kv_rank:
                    raise ConfigError(f"layers[{i}].mixer.kv_from = {m.kv_from} must name an earlier latent_attention "
                                      f"layer that makes rows of its own, of rank {m.kv_rank}")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "NurasunConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json has no 'layers' list")
        return cls(vocab=_positive_int(raw, "vocab", "config"), width=_positive_int(raw, "width", "config"),
                   layers=tuple(NurasunLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(layers)),
                   norm_eps=float(_get(raw.get("norm"), "eps", "norm")),
                   residual_mult=float(raw.get("residual_mult", 1.0)), logit_softcap=float(raw.get("logit_softcap") or 0.0))

    def to_dict(self) -> dict[str, Any]:
        return {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                "logit_softcap": self.logit_softcap, "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
                "vocab": self.vocab, "width": self.width}
