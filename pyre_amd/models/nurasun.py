"""The Nurasun design as a list of parts.

Every layer has one norm (tanh(alpha x) gain + shift, no statistics) whose rows both its mixer and its feed-forward
read; their results are added to the residual stream together, times one factor for the whole model. The mixer is
grouped attention whose values are its keys before rotation, over runs of positions ('attention'), or causal
attention over one compressed row per token ('latent_attention'), which may read the rows that an earlier layer
keeps. The feed-forward is a gated unit with the tanh form of GELU, or a mixture of experts with a sigmoid router
and a shared expert, or absent. The logits are squashed. Tensor names: ``embed``, ``head``, ``final.norm``,
``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``; a norm's scalar and shift are ``<name>.alpha`` and ``<name>.b``.
"""

from __future__ import annotations

from pyre_amd.config.nurasun import (DenseConfig, LatentAttentionConfig, MixtureConfig, NurasunConfig,
                                     TiedAttentionConfig)
from pyre_amd.parts.base import (EmbeddingSpec, GeluGLUSpec, LatentAttentionSpec, LayerCall, LMHeadSpec, ModelSpec,
                                 NoPositionSpec, ParallelBlockSpec, RotarySpec, SigmoidMoESpec, TanhNormSpec,
                                 TiedAttentionSpec)
from pyre_amd.registry import register_architecture


def _tied(cfg: NurasunConfig, m: TiedAttentionConfig, prefix: str) -> TiedAttentionSpec:
    position = RotarySpec(m.dim, m.rot_base, 0, rotary_dim=m.rot_dims, exact=True) if m.rot_dims else NoPositionSpec()
    return TiedAttentionSpec(cfg.width, m.heads, m.kv_heads, m.dim, m.scale, position, prefix, chunk=m.chunk, bias=True)


def _latent(cfg: NurasunConfig, m: LatentAttentionConfig, prefix: str) -> LatentAttentionSpec:
    return LatentAttentionSpec(cfg.width, m.heads, m.dim, m.vdim, m.kv_rank, m.scale, cfg.norm_eps, prefix,
                               own_latent=m.kv_from is None)


MIXERS = {TiedAttentionConfig: _tied, LatentAttentionConfig: _latent}


def _dense(cfg: NurasunConfig, f: DenseConfig, prefix: str) -> GeluGLUSpec:
    return GeluGLUSpec(cfg.width, f.ff, prefix)


def _mixture(cfg: NurasunConfig, f: MixtureConfig, prefix: str) -> SigmoidMoESpec:
    return SigmoidMoESpec(cfg.width, f.experts, f.top, f.expert_ff, prefix, shared_size=f.shared_ff)


FEED_FORWARDS = {DenseConfig: _dense, MixtureConfig: _mixture}


def build_nurasun(cfg: NurasunConfig) -> ModelSpec:
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ff = None if layer.mlp is None else FEED_FORWARDS[type(layer.mlp)](cfg, layer.mlp, f"{p}.mlp")
        layers.append(ParallelBlockSpec(mixer=MIXERS[type(layer.mixer)](cfg, layer.mixer, f"{p}.mix"),
                                        norm=TanhNormSpec(cfg.width, f"{p}.norm1"), feed_forward=ff,
                                        scale=cfg.residual_mult))
        schedule.append(LayerCall(i, cache_from=getattr(layer.mixer, "kv_from", None)))
    return ModelSpec(hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=0,
                     embedding=EmbeddingSpec(cfg.vocab, cfg.width, name="embed"), layers=tuple(layers),
                     schedule=tuple(schedule), final_norm=TanhNormSpec(cfg.width, "final.norm"),
                     head=LMHeadSpec(cfg.vocab, cfg.width, name="head", softcap=cfg.logit_softcap))


register_architecture(NurasunConfig.architecture, NurasunConfig, build_nurasun)
