"""A model assembled from a :class:`~pyre_amd.parts.base.ModelSpec`."""

from __future__ import annotations

import torch

from pyre_amd.parts.base import ModelSpec, Part, TensorSpec, make_part
from pyre_amd.parts.block import Hidden


class LayeredModel(Part):
    """embedding -> layers in the order of ``spec.schedule`` -> final norm -> head.

    The model owns no cache: the engine hands ``forward`` one cache view per entry
    of the order (or None where the entry keeps nothing).
    """

    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = make_part("embedding", spec.embedding)
        self.layers = [make_part("block", b) for b in spec.layers]
        self.final_norm = make_part("norm", spec.final_norm)
        self.head = make_part("head", spec.head)
        self.schedule = list(spec.schedule)
        for pos, call in enumerate(self.schedule):
            if not (0 <= call.layer < len(self.layers)):
                raise ValueError(f"order entry {pos} names layer {call.layer}, there are {len(self.layers)}")
            if call.cache_from is not None and not (0 <= call.cache_from < pos):
                raise ValueError(f"order entry {pos} reads the cache of entry {call.cache_from}, which does not precede it")

    def parts(self):
        return (self.embedding, *self.layers, self.final_norm, self.head)

    def tensor_specs(self) -> list[TensorSpec]:
        seen: dict[str, TensorSpec] = {}
        for p in self.parts():
            for s in p.tensor_specs():
                if s.name in seen and seen[s.name].shape != s.shape:
                    raise ValueError(f"tensor {s.name} is asked for with two shapes")
                seen.setdefault(s.name, s)
        return list(seen.values())

    def linears(self) -> list:
        return [lin for p in self.parts() for lin in p.linears()]

    def step_arrays(self) -> list:
        """The arrays that the mixers ask of every step, each name once."""
        seen = {}
        for layer in self.layers:
            mixer = getattr(layer, "mixer", None)
            for spec in (mixer.step_arrays() if mixer is not None else []):
                seen.setdefault(spec.name, spec)
        return list(seen.values())

    def cache_specs(self) -> list:
        """What each entry of the order keeps; None for an entry that keeps nothing
        or reads another entry's cache."""
        out = []
        for call in self.schedule:
            out.append(None if call.cache_from is not None else self.layers[call.layer].mixer.cache_spec())
        return out

    def bind(self, tensors, runtime) -> None:
        for p in self.parts():
            p.bind(tensors, runtime)

    def forward(self, ctx, caches: list) -> torch.Tensor | None:
        """Run the step's tokens; returns float32 logits [n_logits, vocab] (None if none are wanted)."""
        n = ctx.n_tokens
        resid = ctx.workspace.get("resid", (n, self.spec.hidden_size), torch.float32)
        self.embedding.forward(ctx, resid)
        state = Hidden(resid)
        for pos, call in enumerate(self.schedule):
            self.layers[call.layer].forward(ctx, state, caches[pos])
        m = ctx.n_logits
        if m == 0:
            return None
        h = ctx.workspace.get("head.h", (m, self.spec.hidden_size), ctx.dtype)
        self.final_norm.forward(ctx, state.resid, state.pending, h, rows=ctx.logit_rows)
        return self.head.forward(ctx, h, m)
