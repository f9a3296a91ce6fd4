"""RMSNorm fused with the residual sum that precedes it (`pyre/model.py:22-38,151-152`)."""

from __future__ import annotations

from pyre_amd.hip import ops
from pyre_amd.parts.base import LayerNormSpec, Norm, RMSNormSpec, TensorSpec


class RMSNorm(Norm):
    def __init__(self, spec: RMSNormSpec):
        self.spec = spec
        self.gain = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(f"{self.spec.prefix}.weight", (self.spec.hidden_size,), init="gain")]

    def bind(self, tensors, runtime) -> None:
        self.gain = tensors[f"{self.spec.prefix}.weight"].contiguous()

    def forward(self, ctx, resid, delta, out, rows=None) -> None:
        ops.add_rmsnorm(resid, delta, self.gain, self.spec.eps, out, rows)


class LayerNorm(Norm):
    """(x - mean) / sqrt(var + eps) * gain without a bias, fused with the residual sum before it. The
    pending term may carry a norm of its own (``Partials.post``: a sublayer's result that is normed
    and scaled before it is added); the same kernel applies it."""

    def __init__(self, spec: LayerNormSpec):
        self.spec = spec
        self.gain = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.spec.name, (self.spec.hidden_size,), init="gain")]

    def bind(self, tensors, runtime) -> None:
        self.gain = tensors[self.spec.name].contiguous()

    def forward(self, ctx, resid, delta, out, rows=None) -> None:
        ops.add_layernorm(resid, delta, self.gain, self.spec.eps, out, rows)
