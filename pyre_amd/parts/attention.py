"""Grouped-query attention over the paged cache (`pyre/model.py:75-125,251-342`)."""

from __future__ import annotations

import torch

import numpy as np

from pyre_amd.hip import ops
from pyre_amd.parts import attention_work as plan
from pyre_amd.parts import fast
from pyre_amd.parts.base import (AttentionSpec, Mixer, PagedCacheSpec, PagedTensorSpec, StepArraySpec, TensorSpec,
                                 make_part, take)
from pyre_amd.parts.linear import Linear, linear_specs


def KVCacheSpec(num_kv_heads: int, head_dim: int, window: int = 0) -> PagedCacheSpec:
    """What this attention keeps per token, laid out for its kernels: the rotated key as
    ``k [pages, kv_heads, page_size, head_dim]`` (a head's keys of a page lie together, one
    key is one contiguous run) and the value transposed, ``v [pages, kv_heads, head_dim,
    page_size]``, so that the MFMA kernels read runs of tokens for one feature."""
    return PagedCacheSpec((PagedTensorSpec("k", (num_kv_heads, head_dim), token_axis=1),
                           PagedTensorSpec("v", (num_kv_heads, head_dim), token_axis=2)), window)


#: tokens of one request that the prompt-portion attention kernel takes at a time
TILE = 32


def _decode_tokens(hb) -> np.ndarray:
    """Flat indices of the tokens of requests that bring a single token."""
    counts = hb.q_start[1:] - hb.q_start[:-1]
    return hb.q_start[:-1][counts == 1]


def _prefill_tiles(hb) -> np.ndarray:
    """[T, 2] (first token, count <= TILE) of the requests that bring more than one token,
    the tiles that see the most keys first."""
    counts = hb.q_start[1:] - hb.q_start[:-1]
    tiles = []
    for s in np.nonzero(counts != 1)[0]:
        a, b = int(hb.q_start[s]), int(hb.q_start[s + 1])
        tiles.extend((int(hb.positions[t0]) + min(TILE, b - t0), t0, min(TILE, b - t0)) for t0 in range(a, b, TILE))
    tiles.sort(key=lambda t: -t[0])
    return np.asarray([t[1:] for t in tiles], dtype=np.int32).reshape(-1, 2)


STEP_ARRAYS = (
    StepArraySpec("attention.decode_tokens", lambda n_cap, s_cap: n_cap, _decode_tokens),
    StepArraySpec("attention.prefill_tiles", lambda n_cap, s_cap: 2 * (n_cap // TILE + s_cap), _prefill_tiles),
)


class Attention(Mixer):
    """q, k, v = split(h Wqkv^T + b); rotate q, k; store k, v; out = softmax(q k^T scale) v; out Wo^T.

    The three projections are one product over the row-wise concatenation
    [Wq; Wk; Wv] (made at bind time). Query head i reads key/value head
    i // (num_heads / num_kv_heads) (`pyre/model.py:66-72`).
    """

    def __init__(self, spec: AttentionSpec):
        if spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        # what no attention kernel takes is refused when the model is built, not at its first step
        if not (0 < spec.head_dim <= ops.ATTN_MAX_HEAD_DIM):
            raise ValueError(f"attention: head_dim {spec.head_dim} is outside 1..{ops.ATTN_MAX_HEAD_DIM}, the sizes "
                             "that the attention kernels take")
        if spec.num_heads > ops.ATTN_MAX_HEADS:
            raise ValueError(f"attention: {spec.num_heads} query heads are more than a launch holds ({ops.ATTN_MAX_HEADS})")
        if spec.window < 0:
            raise ValueError("attention: the window must not be negative")
        self.spec = spec
        self.units = plan.DEFAULT_UNITS  #: compute units that the work lists are planned for; the engine's at bind
        self.position = make_part("position", spec.position)
        self.scale = spec.scale if spec.scale is not None else spec.head_dim ** -0.5
        self.q_dim = spec.num_heads * spec.head_dim
        self.kv_dim = spec.num_kv_heads * spec.head_dim
        self.qkv = Linear(spec.hidden_size, self.q_dim + 2 * self.kv_dim, "attn.qkv")
        self.out = Linear(self.q_dim, spec.hidden_size, "attn.out")
        self.decode_work_name = f"attention.decode_work.{spec.num_heads}.{spec.num_kv_heads}.{spec.window}"
        self.prefill_work_name = f"attention.prefill_work.{spec.num_heads}.{spec.num_kv_heads}.{spec.window}"

    def cache_spec(self):
        s = self.spec
        return KVCacheSpec(s.num_kv_heads, s.head_dim, s.window)

    def step_arrays(self):
        """The lists of single tokens and of tiles, and the work lists of the decode and the
        prompt-portion kernel, which depend on the head counts and the window and are shared by
        all layers that agree in them."""
        s = self.spec

        def work(hb):
            listed = plan.decode_work(hb.arrays["attention.decode_tokens"], hb.positions, hb.decode_shape()[0],
                                      s.window, s.num_heads, s.num_kv_heads, units=self.units)
            return plan.decode_work_with_places(listed, hb.positions, hb.seq_of_token)

        def portions(hb):
            return plan.prefill_work(hb.arrays["attention.prefill_tiles"], hb.positions, s.window,
                                     plan.prefill_items(s.num_heads, s.num_kv_heads), units=self.units)

        def decode_cap(n_cap, s_cap):
            return 8 * (1 + plan.decode_capacity(s_cap, s.num_heads, s.num_kv_heads, self.units))

        def prefill_cap(n_cap, s_cap):
            return 8 * plan.prefill_capacity(n_cap, s_cap, TILE, plan.prefill_items(s.num_heads, s.num_kv_heads), self.units)

        return [*STEP_ARRAYS, StepArraySpec(self.decode_work_name, decode_cap, work),
                StepArraySpec(self.prefill_work_name, prefill_cap, portions)]

    def linears(self) -> list:
        return [self.qkv, self.out]

    def tensor_specs(self) -> list[TensorSpec]:
        s, p = self.spec, self.spec.prefix
        return (linear_specs(f"{p}.q_proj", self.q_dim, s.hidden_size, s.qkv_bias)
                + linear_specs(f"{p}.k_proj", self.kv_dim, s.hidden_size, s.qkv_bias)
                + linear_specs(f"{p}.v_proj", self.kv_dim, s.hidden_size, s.qkv_bias)
                + linear_specs(f"{p}.o_proj", s.hidden_size, self.q_dim, s.out_bias))

    def bind(self, tensors, runtime) -> None:
        p = self.spec.prefix
        self.units = getattr(runtime, "compute_units", None) or plan.DEFAULT_UNITS
        # the three weights are let go of one by one, so that at most one copy more than the
        # fused matrix lives at any time
        parts = []
        for n in "qkv":
            parts.append(take(tensors, f"{p}.{n}_proj.weight"))
        w = torch.cat(parts, dim=0)
        del parts
        b = None
        if self.spec.qkv_bias:
            b = torch.cat([take(tensors, f"{p}.{n}_proj.bias") for n in "qkv"], dim=0)
        self.qkv.set(w, b)
        self.out.set(take(tensors, f"{p}.o_proj.weight"), take(tensors, f"{p}.o_proj.bias") if self.spec.out_bias else None)

    def forward(self, ctx, h, cache):
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        qkv = self.qkv.forward(ctx, h, n)
        q = ws.get("attn.q", (n, self.q_dim), ctx.dtype)
        cos, sin, rot = self.position.rotary(ctx.runtime)
        k_pages, v_pages = cache["k"], cache["v"]
        o = ws.get("attn.o", (n, self.q_dim), ctx.dtype)
        if fast.rope_in_attention(self, ctx, qkv, cache, rot):
            # a step of single tokens: the attention kernel sums, biases and rotates the product's
            # partial sums itself and writes the new keys and values (one kernel less a layer)
            fast.attention(self, ctx, q, o, cache, rope=(qkv, cos, sin))
            return self.out.forward(ctx, o, n)
        ops.rope_kv_write(qkv, q, k_pages if cache.writes else None, v_pages if cache.writes else None,
                          cos, sin, rot, ctx.positions, cache.slots, n, s.num_heads, s.num_kv_heads,
                          s.head_dim, cache.page_size)
        if not fast.attention(self, ctx, q, o, cache):
            self._attend_plainly(ctx, q, o, cache)
        return self.out.forward(ctx, o, n)

    def _attend_plainly(self, ctx, q, o, cache) -> None:
        """The kernels that take every geometry and element type; the whole of the 32-bit path."""
        s, n = self.spec, ctx.n_tokens
        k_pages, v_pages = cache["k"], cache["v"]
        geometry = (s.num_heads, s.num_kv_heads, s.head_dim, cache.page_size, self.scale, cache.window)
        tiles = ctx.host.arrays["attention.prefill_tiles"]
        if len(tiles) and q.dtype == torch.float32 and k_pages.dtype == torch.float32:
            # prompt portions on the matrix cores' float32 instruction, single tokens one by one
            ops.attn_prefill_f32(q, o, k_pages, v_pages, ctx.arrays["attention.prefill_tiles"], len(tiles),
                                 ctx.positions, ctx.seq_of_token, cache.table, *geometry)
            singles = ctx.host.arrays["attention.decode_tokens"]
            if len(singles):
                ops.attn_generic(q, o, k_pages, v_pages, ctx.positions, ctx.seq_of_token, cache.table, len(singles),
                                 *geometry, tokens=ctx.arrays["attention.decode_tokens"],
                                 scratch=self._spans_scratch(ctx, cache, len(singles)))
        else:
            ops.attn_generic(q, o, k_pages, v_pages, ctx.positions, ctx.seq_of_token, cache.table, n, *geometry,
                             scratch=self._spans_scratch(ctx, cache, n))

    def _spans_scratch(self, ctx, cache, n):
        """Workspace for the partial results of the spans of keys, if the tables are wider than one."""
        s = self.spec
        need = ops.attn_generic_scratch(n, s.num_heads, s.head_dim, cache.table.shape[1], cache.page_size, cache.window)
        return ctx.workspace.get("attn.spans", (need,), torch.float32) if need else None
