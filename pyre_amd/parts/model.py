"""A model assembled from a :class:`~pyre_amd.parts.base.ModelSpec`."""

from __future__ import annotations

import torch

from pyre_amd.parts.base import ModelSpec, Part, TensorBag, TensorSpec, make_part
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
        """The arrays that the layers ask of every step, each name once."""
        seen = {}
        for layer in self.layers:
            for spec in layer.step_arrays():
                seen.setdefault(spec.name, spec)
        return list(seen.values())

    def cache_specs(self) -> list[list]:
        """What each entry of the order keeps: a list of cache descriptions, empty for an
        entry that keeps nothing or reads another entry's caches."""
        out: list[list] = []
        for pos, call in enumerate(self.schedule):
            own = list(self.layers[call.layer].cache_specs())
            if call.cache_from is None:
                out.append(own)
                continue
            theirs = out[call.cache_from]
            if [type(s) for s in own] != [type(s) for s in theirs]:
                raise ValueError(f"order entry {pos} reads the caches of entry {call.cache_from}, which keeps "
                                 f"{len(theirs)} of other kinds than the {len(own)} that this layer wants")
            out.append([])
        return out

    def tensor_uses(self) -> dict[str, int]:
        """How many parts name each tensor (a part inside a layer counts as its layer)."""
        uses: dict[str, int] = {}
        for p in self.parts():
            for s in p.tensor_specs():
                uses[s.name] = uses.get(s.name, 0) + 1
        return uses

    def bind(self, tensors, runtime) -> None:
        """Every part takes its tensors out of ``tensors``, which is left empty: a tensor that
        its part copies (a fused weight) is free as soon as the last part that named it has it."""
        bag = TensorBag(tensors, self.tensor_uses())
        tensors.clear()
        for p in self.parts():
            p.bind(bag, runtime)

    def forward(self, ctx, caches: list, tap=None) -> torch.Tensor | None:
        """Run the step's tokens; returns float32 logits [n_logits, vocab] (None if none are wanted).
        ``caches[pos]`` is the list of cache views of entry ``pos`` of the order. ``tap(pos, rows)``,
        a debugging aid, is called after every entry with the hidden rows [n, hidden] (float32, the
        residual stream with the pending term added: a copy, made for the tap)."""
        n = ctx.n_tokens
        resid = ctx.workspace.get("resid", (n, self.spec.hidden_size), torch.float32)
        self.embedding.forward(ctx, resid)
        state = Hidden(resid)
        for pos, call in enumerate(self.schedule):
            self.layers[call.layer].forward(ctx, state, caches[pos])
            if tap is not None:
                tap(pos, self._hidden_rows(ctx, state))
        m = ctx.n_logits
        if m == 0:
            return None
        h = ctx.workspace.get("head.h", (m, self.spec.hidden_size), ctx.dtype)
        self.final_norm.forward(ctx, state.resid, state.pending, h, rows=ctx.logit_rows)
        return self.head.forward(ctx, h, m)

    def _hidden_rows(self, ctx, state: Hidden) -> torch.Tensor:
        """The residual stream as it stands after a layer, the term that the next norm would add
        included (its partial sums in their order, then the bias)."""
        rows = state.resid[:ctx.n_tokens].clone()
        p = state.pending
        if p is not None:
            for i in range(p.count):
                rows += p.data[i, :ctx.n_tokens].float()
            if p.bias is not None:
                rows += p.bias.float()
        return rows
