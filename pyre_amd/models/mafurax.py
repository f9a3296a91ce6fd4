"""The Mafurax design as a list of parts.

Every layer norms its sublayers before and after (layer norm with a gain, no bias) and scales the
normed result element by element before it joins the residual stream. The mixer of a 'parallel'
layer is two mixers side by side on the same rows: softmax attention without rotation (unit-norm
queries and keys, capped scores, a learned bias by distance, a window that keeps the sequence's
first tokens, a gate per head) and gated linear attention (a float32 matrix state per head, decayed
per key channel). The feed-forward, where a layer has one, is a gated unit with clipped inputs. The
output head is the embedding table, its logits scaled. Tensor names: ``embed``, ``final.norm``,
``l<i>.norm1 / norm1b / norm2 / norm2b / ls1 / ls2``, ``l<i>.mix.left.*``, ``l<i>.mix.right.*``,
``l<i>.mlp.gate / up / down``.
"""

from __future__ import annotations

from pyre_amd.config.mafurax import DenseFeedForwardConfig, MafuraxConfig, ParallelMixerConfig
from pyre_amd.parts.base import (CappedAttentionSpec, ClippedGLUSpec, EmbeddingSpec, GatedLinearAttentionSpec, LayerCall,
                                 LayerNormSpec, LMHeadSpec, ModelSpec, ParallelMixerSpec, SandwichBlockSpec)
from pyre_amd.registry import register_architecture


def _parallel(cfg: MafuraxConfig, m: ParallelMixerConfig, prefix: str) -> ParallelMixerSpec:
    a, r = m.left, m.right
    left = CappedAttentionSpec(cfg.width, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, f"{prefix}.left", softcap=a.softcap,
                               bias_far=a.bias_max, bias_rows=a.bias_rows, window=a.window, keep_first=a.keep_first,
                               unit_norm=True, norm_eps=cfg.norm_eps, gated=True)
    right = GatedLinearAttentionSpec(cfg.width, r.heads, r.dim, r.vdim, r.tau, f"{prefix}.right", norm_eps=cfg.norm_eps,
                                     rank=r.rank)
    return ParallelMixerSpec(cfg.width, (left, right), (m.left_scale, m.right_scale))


MIXERS = {ParallelMixerConfig: _parallel}


def _dense(cfg: MafuraxConfig, f: DenseFeedForwardConfig, prefix: str) -> ClippedGLUSpec:
    return ClippedGLUSpec(cfg.width, f.ff, f.limit, prefix)


FEED_FORWARDS = {DenseFeedForwardConfig: _dense}


def build_mafurax(cfg: MafuraxConfig) -> ModelSpec:
    def norm(name):
        return LayerNormSpec(cfg.width, cfg.norm_eps, name)

    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        # a layer without a feed-forward: a file may still hold that half's norms and scale; nothing reads them
        ff = dict(unused=(f"{p}.norm2", f"{p}.norm2b", f"{p}.ls2"))
        if layer.mlp is not None:
            ff = dict(feed_forward=FEED_FORWARDS[type(layer.mlp)](cfg, layer.mlp, f"{p}.mlp"), feed_forward_norm=norm(f"{p}.norm2"),
                      feed_forward_post_norm=norm(f"{p}.norm2b"), feed_forward_scale=f"{p}.ls2")
        layers.append(SandwichBlockSpec(mixer=MIXERS[type(layer.mixer)](cfg, layer.mixer, f"{p}.mix"), mixer_norm=norm(f"{p}.norm1"),
                                        mixer_post_norm=norm(f"{p}.norm1b"), mixer_scale=f"{p}.ls1", **ff))
    embedding = EmbeddingSpec(cfg.vocab, cfg.width, name="embed")
    return ModelSpec(hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=0, embedding=embedding,
                     layers=tuple(layers), schedule=tuple(LayerCall(i) for i in range(len(layers))),
                     final_norm=norm("final.norm"),
                     head=LMHeadSpec(cfg.vocab, cfg.width, name=embedding.name, scale=cfg.logit_scale))


register_architecture(MafuraxConfig.architecture, MafuraxConfig, build_mafurax)
