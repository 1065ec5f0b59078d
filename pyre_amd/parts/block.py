"""The arrangement of a layer's parts around the residual stream (`pyre/model.py:142-153`)."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from pyre_amd.hip.ops import Partials
from pyre_amd.parts.base import Block, BlockSpec, TensorSpec, make_part


@dataclass
class Hidden:
    """The residual stream (float32 [N, H]) and the term not yet added to it: the
    next norm adds it in the same kernel that norms the sum."""

    resid: torch.Tensor
    pending: Partials | None = None


class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += feed_forward(norm2(x))."""

    def __init__(self, spec: BlockSpec):
        self.spec = spec
        self.mixer = make_part("mixer", spec.mixer)
        self.mixer_norm = make_part("norm", spec.mixer_norm)
        self.feed_forward = make_part("feed_forward", spec.feed_forward)
        self.feed_forward_norm = make_part("norm", spec.feed_forward_norm)

    def parts(self):
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    def tensor_specs(self) -> list[TensorSpec]:
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, runtime) -> None:
        for p in self.parts():
            p.bind(tensors, runtime)

    def linears(self) -> list:
        return [lin for p in self.parts() for lin in p.linears()]

    def cache_specs(self) -> list:
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def step_arrays(self) -> list:
        return self.mixer.step_arrays()

    def forward(self, ctx, state: Hidden, caches: list) -> None:
        h = ctx.workspace.get("block.h", (ctx.n_tokens, state.resid.shape[1]), ctx.dtype)
        self.mixer_norm.forward(ctx, state.resid, state.pending, h)
        mixed = self.mixer.forward(ctx, h, caches[0] if caches else None)
        self.feed_forward_norm.forward(ctx, state.resid, mixed, h)
        state.pending = self.feed_forward.forward(ctx, h)
