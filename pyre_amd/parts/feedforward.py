"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)), no biases (`pyre/model.py:128-139`)."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts import fast
from pyre_amd.parts.base import FeedForward, SwiGLUSpec, TensorSpec, take
from pyre_amd.parts.linear import Linear, linear_specs


class SwiGLU(FeedForward):
    """gate and up are one product over [Wgate; Wup]; the SiLU-gate reads its halves."""

    def __init__(self, spec: SwiGLUSpec):
        self.spec = spec
        self.gate_up = Linear(spec.hidden_size, 2 * spec.intermediate_size, "ffn.gate_up")
        self.down = Linear(spec.intermediate_size, spec.hidden_size, "ffn.down")

    def tensor_specs(self) -> list[TensorSpec]:
        s, p = self.spec, self.spec.prefix
        return (linear_specs(f"{p}.gate_proj", s.intermediate_size, s.hidden_size, False)
                + linear_specs(f"{p}.up_proj", s.intermediate_size, s.hidden_size, False)
                + linear_specs(f"{p}.down_proj", s.hidden_size, s.intermediate_size, False))

    def bind(self, tensors, runtime) -> None:
        p = self.spec.prefix
        halves = [take(tensors, f"{p}.gate_proj.weight"), take(tensors, f"{p}.up_proj.weight")]
        fused = torch.cat(halves, dim=0)
        del halves  # the two weights are free before the next layer makes its copy
        self.gate_up.set(fused)
        self.down.set(take(tensors, f"{p}.down_proj.weight"))

    def linears(self) -> list:
        return [self.gate_up, self.down]

    def forward(self, ctx, h):
        n = ctx.n_tokens
        act = ctx.workspace.get("ffn.act", (n, self.spec.intermediate_size), ctx.dtype)
        if not fast.gate_up_silu(self.gate_up, ctx, h, n, act):
            gu = self.gate_up.forward(ctx, h, n)
            ops.silu_mul(gu, act, n)
        return self.down.forward(ctx, act, n)
