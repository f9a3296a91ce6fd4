"""Softmax attention whose positions enter through the scores alone: no rotation, unit-norm queries
and keys, capped scores, a learned bias by distance, a window that keeps the sequence's first tokens,
and a gate per head on the output."""

from __future__ import annotations

import math

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.attention import STEP_ARRAYS
from pyre_amd.parts.base import (CappedAttentionSpec, PagedCacheSpec, PagedTensorSpec, TensorSpec, take)
from pyre_amd.parts.branch import BranchMixer

#: rows of the distance table that the random-weights mode draws when a description leaves them to the file
DEFAULT_BIAS_ROWS = 32


def distance_rows(rows: int, far: float) -> list[int]:
    """Row of a table of ``rows`` rows for every distance 0 .. ceil(far): distance n has its own row while
    n < rows // 2; beyond, the rows are spaced evenly in log(n) between rows // 2 and ``far``, and every
    distance from ``far`` on shares the last row."""
    half = rows // 2
    out = []
    for n in range(int(math.ceil(far)) + 1):
        if n < half or half == 0:
            out.append(min(n, rows - 1))
        elif far <= half:
            out.append(rows - 1)
        else:
            step = math.floor(math.log(n / half) / math.log(far / half) * (rows - half))
            out.append(min(rows - 1, half + int(step)))
    return out


class CappedAttention(BranchMixer):
    role = "cattn"

    def __init__(self, spec: CappedAttentionSpec):
        if spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError("capped attention: heads must be a multiple of kv_heads")
        for name, v in (("key_dim", spec.key_dim), ("value_dim", spec.value_dim)):
            if not (0 < v <= ops.ATTN_MAX_HEAD_DIM):
                raise ValueError(f"capped attention: {name} {v} is outside 1..{ops.ATTN_MAX_HEAD_DIM}")
        if spec.window < 0 or spec.keep_first < 0 or spec.softcap < 0:
            raise ValueError("capped attention: window, keep_first and softcap must not be negative")
        if spec.bias_rows != 0 and not (spec.bias_far > 0):
            raise ValueError("capped attention: a bias by distance needs the distance from which it is constant")
        self.spec = spec
        self.hidden_size = spec.hidden_size
        self.inner = spec.num_heads * spec.value_dim
        self.bias = None   #: float32 [heads, far + 1]: the bias of every distance, made of the table at bind
        self.far = 0

    def cache_spec(self):
        s = self.spec
        return PagedCacheSpec((PagedTensorSpec("k", (s.num_kv_heads, s.key_dim), token_axis=1),
                               PagedTensorSpec("v", (s.num_kv_heads, s.value_dim), token_axis=1)),
                              s.window, s.keep_first if s.window else 0)

    def step_arrays(self):
        return list(STEP_ARRAYS)

    def in_tensors(self):
        s, p = self.spec, self.spec.prefix
        specs = [TensorSpec(f"{p}.q", (s.num_heads * s.key_dim, s.hidden_size)),
                 TensorSpec(f"{p}.k", (s.num_kv_heads * s.key_dim, s.hidden_size)),
                 TensorSpec(f"{p}.v", (s.num_kv_heads * s.value_dim, s.hidden_size))]
        if s.gated:
            specs.append(TensorSpec(f"{p}.g", (s.num_heads, s.hidden_size)))
        return specs

    def out_tensor(self):
        return TensorSpec(f"{self.spec.prefix}.o", (self.spec.hidden_size, self.inner))

    def other_tensors(self):
        s = self.spec
        if s.bias_rows == 0:
            return []
        # random weights: drawn wide, so that the bias of a distance matters beside the scores
        return [TensorSpec(f"{s.prefix}.rel", (s.bias_rows, s.num_heads), init="normal:1.0",
                           random_shape=(s.bias_rows or DEFAULT_BIAS_ROWS, s.num_heads))]

    def bind_others(self, tensors, runtime) -> None:
        s = self.spec
        if s.bias_rows == 0:
            return
        table = take(tensors, f"{s.prefix}.rel").float()               # [rows, heads]
        rows = distance_rows(table.shape[0], s.bias_far)
        self.far = len(rows) - 1
        index = torch.tensor(rows, dtype=torch.long, device=table.device)
        self.bias = table[index].t().contiguous()                       # [heads, far + 1]

    def attend(self, ctx, proj, col0, cache, o, scale) -> None:
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        q = ws.get("cattn.q", (n, s.num_heads * s.key_dim), ctx.dtype)
        gate = ws.get("cattn.gate", (n, s.num_heads), torch.float32) if s.gated else None
        k_pages, v_pages = cache["k"], cache["v"]
        ops.unit_qkv_write(proj, col0, q, k_pages if cache.writes else None, v_pages if cache.writes else None, gate,
                           cache.slots, n, s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, cache.page_size,
                           s.unit_norm, s.norm_eps)
        shape = (s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, cache.page_size, s.scale, s.softcap, self.bias,
                 self.far, s.window, s.keep_first)
        tiles = ctx.host.arrays["attention.prefill_tiles"]
        singles = ctx.host.arrays["attention.decode_tokens"]
        if len(tiles) and s.key_dim > ops.ATTN_BIASED_TILE_MAX_KEY_HEAD:
            # key heads that the tile kernel does not hold: every token on its own
            ops.attn_biased_single(q, o, k_pages, v_pages, gate, scale, None, n, ctx.positions, ctx.seq_of_token,
                                   cache.table, *shape)
            return
        if len(tiles):
            ops.attn_biased_tile(q, o, k_pages, v_pages, gate, scale, ctx.arrays["attention.prefill_tiles"], len(tiles),
                                 ctx.positions, ctx.seq_of_token, cache.table, *shape)
        if len(singles):
            # a block per span of 128 keys, joined by a second kernel: a step of few tokens fills the chip that way
            spans = ops.attn_biased_spans(cache.table.shape[1], cache.page_size, s.window, s.keep_first)
            scratch = None
            if spans > 1:
                scratch = ws.get("cattn.spans", (len(singles) * s.num_heads * spans * (s.value_dim + 2),), torch.float32)
            ops.attn_biased_single(q, o, k_pages, v_pages, gate, scale, ctx.arrays["attention.decode_tokens"],
                                   len(singles), ctx.positions, ctx.seq_of_token, cache.table, *shape, scratch=scratch)
