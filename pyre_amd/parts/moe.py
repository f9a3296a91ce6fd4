"""A mixture of small feed-forward layers with a sigmoid router and a shared expert."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.base import FeedForward, SigmoidMoESpec, TensorSpec, take
from pyre_amd.parts.linear import Linear


class SigmoidMoE(FeedForward):
    """out = sum over the chosen experts e of w_e down_e(relu(up_e h)^2) + the shared expert's result.

    The router's logits are a product of their own (float32 sums); a kernel squashes them, chooses and writes the
    weights as a dense row per token, zero where an expert is not chosen. All experts' ways up (and the shared
    one's behind them) are one product over the row-wise concatenation of their matrices; the activation kernel
    squares, weights and zeroes; all ways down are one product over the column-wise concatenation, which sums the
    weighted results and the shared expert's as it goes. Every token streams through every expert's matrices:
    right for steps whose tokens between them choose most experts anyway."""

    def __init__(self, spec: SigmoidMoESpec):
        if not (0 < spec.top <= spec.experts <= ops.ROUTE_MAX_EXPERTS):
            raise ValueError(f"mixture: {spec.top} of {spec.experts} experts is not a choice the routing kernel makes")
        if spec.expert_size <= 0 or spec.shared_size < 0:
            raise ValueError("mixture: bad expert sizes")
        self.spec = spec
        self.inner = spec.experts * spec.expert_size + spec.shared_size
        self.router = Linear(spec.hidden_size, spec.experts, "moe.router")
        self.up = Linear(spec.hidden_size, self.inner, "moe.up")
        self.down = Linear(self.inner, spec.hidden_size, "moe.down")

    def _experts(self) -> list[str]:
        s = self.spec
        return [f"{s.prefix}.e{i}" for i in range(s.experts)] + ([f"{s.prefix}.shared"] if s.shared_size else [])

    def tensor_specs(self) -> list[TensorSpec]:
        s = self.spec
        specs = [TensorSpec(f"{s.prefix}.router", (s.experts, s.hidden_size))]
        for p in self._experts():
            ff = s.shared_size if p.endswith(".shared") else s.expert_size
            specs += [TensorSpec(f"{p}.up", (ff, s.hidden_size)), TensorSpec(f"{p}.down", (s.hidden_size, ff))]
        return specs

    def bind(self, tensors, runtime) -> None:
        s = self.spec
        self.router.set(take(tensors, f"{s.prefix}.router"))
        ups = [take(tensors, f"{p}.up") for p in self._experts()]
        self.up.set(torch.cat(ups, dim=0))
        del ups
        downs = [take(tensors, f"{p}.down") for p in self._experts()]
        self.down.set(torch.cat(downs, dim=1))
        del downs

    def linears(self) -> list:
        return [self.router, self.up, self.down]

    def forward(self, ctx, h):
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        gates = ws.get("moe.gates", (n, s.experts), torch.float32)
        ops.route_topk(self.router.forward(ctx, h, n), gates, n, s.top)
        act = ws.get("moe.act", (n, self.inner), ctx.dtype)
        ops.expert_act(self.up.forward(ctx, h, n), gates, act, n, s.experts, s.expert_size, s.shared_size)
        return self.down.forward(ctx, act, n)
