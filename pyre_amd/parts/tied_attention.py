"""Grouped softmax attention whose values are its keys as projected, over runs of positions."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.attention import STEP_ARRAYS
from pyre_amd.parts.base import Mixer, PagedCacheSpec, PagedTensorSpec, TensorSpec, TiedAttentionSpec, make_part, take
from pyre_amd.parts.linear import Linear


def attend_pages(ctx, q, o, k_pages, v_pages, cache, nq: int, nkv: int, dk: int, dv: int, scale: float,
                 chunk: int = 0, scratch_name: str = "attn.pages.spans") -> None:
    """Softmax attention of the step's tokens over paged keys ``k_pages [pages, nkv, page, dk]`` and values
    ``v_pages [pages, nkv, page, dv]`` (which may be one and the same tensor), scores and weights in float32 whatever
    the element type: prompt portions in tiles of 32 tokens on the matrix cores, single tokens a block per span of
    128 keys. ``q [n, nq*dk]`` -> ``o [n, nq*dv]``; ``chunk`` > 0: a query sees the keys of its own run of that many
    positions only."""
    s, n, ws = cache, ctx.n_tokens, ctx.workspace
    shape = (nq, nkv, dk, dv, cache.page_size, scale, 0.0, None, 0, 0, 0)
    tiles = ctx.host.arrays["attention.prefill_tiles"]
    singles = ctx.host.arrays["attention.decode_tokens"]
    if len(tiles) and dk > ops.ATTN_BIASED_TILE_MAX_KEY_HEAD:
        # key heads that the tile kernel does not hold: every token on its own
        ops.attn_biased_single(q, o, k_pages, v_pages, None, 1.0, None, n, ctx.positions, ctx.seq_of_token, cache.table,
                               *shape, chunk=chunk)
        return
    if len(tiles):
        ops.attn_biased_tile(q, o, k_pages, v_pages, None, 1.0, ctx.arrays["attention.prefill_tiles"], len(tiles),
                             ctx.positions, ctx.seq_of_token, cache.table, *shape, chunk=chunk)
    if len(singles):
        spans = ops.attn_biased_spans(cache.table.shape[1], cache.page_size, 0, 0, chunk)
        scratch = None
        if spans > 1:
            scratch = ws.get(scratch_name, (len(singles) * nq * spans * (dv + 2),), torch.float32)
        ops.attn_biased_single(q, o, k_pages, v_pages, None, 1.0, ctx.arrays["attention.decode_tokens"], len(singles),
                               ctx.positions, ctx.seq_of_token, cache.table, *shape, scratch=scratch, chunk=chunk)


class TiedAttention(Mixer):
    """q, k = split(h [Wq; Wk]^T + b); v = k; rotate q and k; out = softmax(q k^T scale over the query's run) v; out Wo^T.

    The two projections are one product. A token's page record holds the turned key and, as the value, the key as
    it was before turning: a query head reads both from its group's head. Query head i reads key head
    i // (num_heads / num_kv_heads)."""

    def __init__(self, spec: TiedAttentionSpec):
        if spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError("tied attention: heads must be a multiple of kv_heads")
        if not (0 < spec.head_dim <= ops.ATTN_MAX_HEAD_DIM):
            raise ValueError(f"tied attention: head_dim {spec.head_dim} is outside 1..{ops.ATTN_MAX_HEAD_DIM}")
        if spec.chunk < 0:
            raise ValueError("tied attention: the run of positions must not be negative")
        self.spec = spec
        self.position = make_part("position", spec.position)
        self.q_dim = spec.num_heads * spec.head_dim
        self.kv_dim = spec.num_kv_heads * spec.head_dim
        self.qk = Linear(spec.hidden_size, self.q_dim + self.kv_dim, "tattn.qk")
        self.out = Linear(self.q_dim, spec.hidden_size, "tattn.out")

    def cache_spec(self):
        s = self.spec
        return PagedCacheSpec((PagedTensorSpec("k", (s.num_kv_heads, s.head_dim), token_axis=1),
                               PagedTensorSpec("v", (s.num_kv_heads, s.head_dim), token_axis=1)), chunk=s.chunk)

    def step_arrays(self):
        return list(STEP_ARRAYS)

    def linears(self) -> list:
        return [self.qk, self.out]

    def tensor_specs(self) -> list[TensorSpec]:
        s, p = self.spec, self.spec.prefix
        specs = [TensorSpec(f"{p}.q", (self.q_dim, s.hidden_size)), TensorSpec(f"{p}.k", (self.kv_dim, s.hidden_size)),
                 TensorSpec(f"{p}.o", (s.hidden_size, self.q_dim))]
        if s.bias:
            specs += [TensorSpec(f"{p}.q.b", (self.q_dim,)), TensorSpec(f"{p}.k.b", (self.kv_dim,))]
        return specs

    def bind(self, tensors, runtime) -> None:
        p = self.spec.prefix
        parts = [take(tensors, f"{p}.q"), take(tensors, f"{p}.k")]
        w = torch.cat(parts, dim=0)
        del parts
        b = torch.cat([take(tensors, f"{p}.q.b"), take(tensors, f"{p}.k.b")], dim=0) if self.spec.bias else None
        self.qk.set(w, b)
        self.out.set(take(tensors, f"{p}.o"))

    def forward(self, ctx, h, cache):
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        proj = self.qk.forward(ctx, h, n)
        q = ws.get("tattn.q", (n, self.q_dim), ctx.dtype)
        cos, sin, rot = self.position.rotary(ctx.runtime)
        k_pages, v_pages = cache["k"], cache["v"]
        ops.rope_tied_write(proj, 0, q, k_pages if cache.writes else None, v_pages if cache.writes else None, cos, sin,
                            rot, ctx.positions, cache.slots, n, s.num_heads, s.num_kv_heads, s.head_dim, cache.page_size)
        o = ws.get("tattn.o", (n, self.q_dim), ctx.dtype)
        attend_pages(ctx, q, o, k_pages, v_pages, cache, s.num_heads, s.num_kv_heads, s.head_dim, s.head_dim, s.scale,
                     chunk=s.chunk, scratch_name="tattn.spans")
        return self.out.forward(ctx, o, n)
