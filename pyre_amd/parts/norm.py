"""RMSNorm fused with the residual sum that precedes it (`pyre/model.py:22-38,151-152`)."""

from __future__ import annotations

from pyre_amd.hip import ops
from pyre_amd.parts.base import Norm, RMSNormSpec, TensorSpec


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
