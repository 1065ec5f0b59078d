"""Token embedding (`pyre/model.py:162,196`) and output head (`:172,201`)."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.base import EmbeddingSpec, LMHeadSpec, Part, TensorSpec
from pyre_amd.parts.linear import Linear


class TokenEmbedding(Part):
    def __init__(self, spec: EmbeddingSpec):
        self.spec = spec
        self.table = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.spec.name, (self.spec.vocab_size, self.spec.hidden_size))]

    def bind(self, tensors, runtime) -> None:
        self.table = tensors[self.spec.name].contiguous()

    def forward(self, ctx, resid: torch.Tensor) -> None:
        """resid[n] = float32(table[token n]): the residual stream starts here."""
        ops.embed(self.table, ctx.tokens, resid)


class LMHead(Part):
    """logits = h W^T in float32, for the wanted rows only. A tied head shares the
    embedding's memory (the reference copies it, `pyre/loader.py:58-61`)."""

    def __init__(self, spec: LMHeadSpec):
        self.spec = spec
        self.linear = Linear(spec.hidden_size, spec.vocab_size, "head")

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.spec.name, (self.spec.vocab_size, self.spec.hidden_size),
                           alias_of=self.spec.tied_to)]

    def bind(self, tensors, runtime) -> None:
        self.linear.set(tensors[self.spec.name])

    def linears(self) -> list:
        return [self.linear]

    def forward(self, ctx, h: torch.Tensor, m: int) -> torch.Tensor:
        out = ctx.workspace.get("head.logits", (m, self.spec.vocab_size), torch.float32)
        p = self.linear.forward(ctx, h, m, out=out)
        if p.data.data_ptr() != out.data_ptr() or p.count != 1 or p.bias is not None:
            ops.reduce_partials(p, out, m)
        return out
