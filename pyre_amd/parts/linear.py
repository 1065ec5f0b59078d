"""y = x W^T (+ b): the matrix products of a model (`pyre/model.py:84-87,92-94,125,
133-139,172`), with the choice of kernel by element type and shape in one place.

A product returns :class:`~pyre_amd.hip.ops.Partials`: its consumer (rotary and
cache write, residual add and norm, SiLU-gate) finishes the sum and adds the bias
inside its own kernel, so neither costs a pass over memory.
"""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.hip.ops import Partials
from pyre_amd.parts.base import TensorSpec


class Linear:
    def __init__(self, in_features: int, out_features: int, role: str):
        self.in_features = in_features
        self.out_features = out_features
        self.role = role              #: names this product's scratch buffer
        self.weight: torch.Tensor | None = None   # [out, in]
        self.bias: torch.Tensor | None = None

    def set(self, weight: torch.Tensor, bias: torch.Tensor | None = None) -> None:
        if tuple(weight.shape) != (self.out_features, self.in_features):
            raise ValueError(f"{self.role}: weight {tuple(weight.shape)} is not "
                             f"({self.out_features}, {self.in_features})")
        self.weight = weight.contiguous()
        self.bias = None if bias is None else bias.contiguous()

    def forward(self, ctx, x: torch.Tensor, n: int, out: torch.Tensor | None = None) -> Partials:
        """x: [>= n, in] -> partial sums of the n x out product. ``out`` (float32
        [n, out]) makes the product land there, complete but for the bias."""
        from pyre_amd.parts import fast

        done = fast.linear(self, ctx, x, n, out)
        if done is not None:
            return done
        f32 = x.dtype == torch.float32 and self.weight.dtype == torch.float32
        if f32 and out is None:
            # the true 32-bit path: the matrix cores' float32 instruction, k split by the weight's shape alone
            ks = ops.gemm_f32_ksplit(self.out_features, self.in_features, ctx.runtime.compute_units)
            buf = ctx.workspace.get(f"linear.{self.role}", (ks, n, self.out_features), torch.float32)
            ops.gemm_f32(x, self.weight, None, buf if ks > 1 else buf[0], n, ks)
            return Partials(buf, self.bias)
        if out is None:
            out = ctx.workspace.get(f"linear.{self.role}", (n, self.out_features), torch.float32)
        if f32 and out.dtype == torch.float32:
            ops.gemm_f32(x, self.weight, None, out, n)
        else:
            ops.gemm_generic(x, self.weight, None, out, n)  # mixed element types, any sizes
        return Partials(out.view(1, n, self.out_features), self.bias)


def linear_specs(prefix: str, out_features: int, in_features: int, bias: bool) -> list[TensorSpec]:
    specs = [TensorSpec(f"{prefix}.weight", (out_features, in_features))]
    if bias:
        specs.append(TensorSpec(f"{prefix}.bias", (out_features,)))
    return specs
