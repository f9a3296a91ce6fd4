"""Causal softmax attention over one compressed row per token, from which every head's keys and values are made."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.attention import STEP_ARRAYS
from pyre_amd.parts.base import LatentAttentionSpec, Mixer, PagedCacheSpec, PagedTensorSpec, TensorSpec, take
from pyre_amd.parts.linear import Linear
from pyre_amd.parts.tied_attention import attend_pages


class LatentAttention(Mixer):
    """c = rms_norm(Wdkv h) gain; head i: k = Wuk_i c, v = Wuv_i c, out_i = softmax(q_i k^T scale) v.

    Only c is kept, and neither keys nor values are ever made: q_i . (Wuk_i c) = (Wuk_i^T q_i) . c, so a head's
    query is carried into the compressed row's space (a product per head), the attention kernels run with c as the
    one shared key and value head, and the weighted sum of rows is carried out again, Wuv_i (sum_j a_j c_j). The
    queries and the compressed row are one input product. A layer without a row of its own (``own_latent`` False)
    reads the pages that another layer of the same rank wrote."""

    def __init__(self, spec: LatentAttentionSpec):
        if not (0 < spec.rank <= ops.ATTN_MAX_HEAD_DIM):
            raise ValueError(f"latent attention: rank {spec.rank} is outside 1..{ops.ATTN_MAX_HEAD_DIM}, the sizes that "
                             "the attention kernels take as a head")
        if max(spec.key_dim, spec.rank) > ops.HEAD_MATMUL_MAX_IN or min(spec.key_dim, spec.value_dim, spec.num_heads) <= 0:
            raise ValueError("latent attention: bad head sizes")
        self.spec = spec
        self.q_dim = spec.num_heads * spec.key_dim
        self.o_dim = spec.num_heads * spec.value_dim
        self.inp = Linear(spec.hidden_size, self.q_dim + (spec.rank if spec.own_latent else 0), "lattn.in")
        self.out = Linear(self.o_dim, spec.hidden_size, "lattn.out")
        self.gain = self.key_up = self.value_up = None

    def cache_spec(self):
        return PagedCacheSpec((PagedTensorSpec("c", (1, self.spec.rank), token_axis=1),))

    def step_arrays(self):
        return list(STEP_ARRAYS)

    def linears(self) -> list:
        return [self.inp, self.out]

    def tensor_specs(self) -> list[TensorSpec]:
        s, p = self.spec, self.spec.prefix
        specs = [TensorSpec(f"{p}.q", (self.q_dim, s.hidden_size))]
        if s.own_latent:
            specs += [TensorSpec(f"{p}.dkv", (s.rank, s.hidden_size)), TensorSpec(f"{p}.dkv.norm", (s.rank,), init="gain")]
        # random weights: the way up from the compressed row drawn wider, so that keys have the scale of queries
        return specs + [TensorSpec(f"{p}.uk", (self.q_dim, s.rank), init="normal:0.1"),
                        TensorSpec(f"{p}.uv", (self.o_dim, s.rank), init="normal:0.1"),
                        TensorSpec(f"{p}.o", (s.hidden_size, self.o_dim))]

    def bind(self, tensors, runtime) -> None:
        s, p = self.spec, self.spec.prefix
        w = take(tensors, f"{p}.q")
        if s.own_latent:
            parts = [w, take(tensors, f"{p}.dkv")]
            w = torch.cat(parts, dim=0)
            del parts
            self.gain = take(tensors, f"{p}.dkv.norm").contiguous()
        self.inp.set(w)
        self.out.set(take(tensors, f"{p}.o"))
        # per head [key_dim, rank] as stored, and [rank, value_dim]: the way up transposed, so that both products
        # walk their matrix row by row
        self.key_up = take(tensors, f"{p}.uk").view(s.num_heads, s.key_dim, s.rank).contiguous()
        self.value_up = take(tensors, f"{p}.uv").view(s.num_heads, s.value_dim, s.rank).transpose(1, 2).contiguous()

    def forward(self, ctx, h, cache):
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        writes = cache.writes and s.own_latent
        proj = self.inp.forward(ctx, h, n)
        q = ws.get("lattn.q", (n, self.q_dim), ctx.dtype)
        rows = cache["c"]
        ops.latent_write(proj, 0, q, rows if writes else None, self.gain, s.norm_eps, cache.slots, n, self.q_dim, s.rank,
                         cache.page_size)
        wide = s.num_heads * s.rank
        q_in = ws.get("lattn.q_in", (n, wide), ctx.dtype)
        ops.head_matmul(q, self.key_up, q_in, n)
        o_in = ws.get("lattn.o_in", (n, wide), ctx.dtype)
        attend_pages(ctx, q_in, o_in, rows, rows, cache, s.num_heads, 1, s.rank, s.rank, s.scale, scratch_name="lattn.spans")
        o = ws.get("lattn.o", (n, self.o_dim), ctx.dtype)
        ops.head_matmul(o_in, self.value_up, o, n)
        return self.out.forward(ctx, o, n)
