"""Choice of the faster kernels of the 16-bit path.

Each function returns None / False when its fast path does not take the case
(element type, sizes, alignment); the caller then runs the general kernel.
Nothing here changes what is computed, only by which kernel. Plain matrix
products with many rows go to the vendor's BLAS through ``torch.mm``, as the
reference's do (`pyre/model.py:84-87` are ``nn.Linear``); the true 32-bit path
never comes here.
"""

from __future__ import annotations

import torch

from pyre_amd.hip.ops import Partials

#: rows from which a 16-bit product goes to the BLAS library
LIBRARY_GEMM_MIN_ROWS = 1


def linear(lin, ctx, x, n, out):
    rt = ctx.runtime
    if rt.dtype != torch.bfloat16 or lin.weight.dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
        return None
    if not rt.options.get("library_gemm", True) or n < LIBRARY_GEMM_MIN_ROWS:
        return None
    if out is not None:
        return None  # float32 results (the head's logits) stay with the engine's own kernels for now
    buf = ctx.workspace.get(f"linear16.{lin.role}", (n, lin.out_features), torch.bfloat16)
    torch.mm(x[:n], lin.weight.t(), out=buf)
    return Partials(buf.view(1, n, lin.out_features), lin.bias)


#: waves the split of decode attention aims at (256 CUs x 8)
DECODE_TARGET_WAVES = 2048
DECODE_MAX_SPLITS = 128


def decode_splits(n_tokens: int, nq: int, nkv: int, max_ctx: int, window: int) -> int:
    """How many ways to split each request's keys so that the chip is full."""
    span = min(max_ctx, window + 32) if window > 0 else max_ctx
    chunks = max(1, -(-span // 32))
    items = n_tokens * nkv * -(-(nq // nkv) // 16)
    return max(1, min(chunks, DECODE_MAX_SPLITS, -(-DECODE_TARGET_WAVES // items)))


def attention(mixer, ctx, q, o, cache) -> bool:
    from pyre_amd.hip import ops

    s = mixer.spec
    if ctx.dtype != torch.bfloat16 or cache.k.dtype != torch.bfloat16:
        return False
    if not ctx.runtime.options.get("mfma_attention", True):
        return False
    if not ops.attn_mfma_supports(s.head_dim, cache.page_size, s.num_heads, s.num_kv_heads):
        return False
    hb = ctx.host
    n_dec, n_tiles = len(hb.decode_tokens), len(hb.prefill_tiles)
    if n_dec:
        nsplits = ctx.runtime.options.get("decode_splits") or decode_splits(
            n_dec, s.num_heads, s.num_kv_heads, hb.max_decode_ctx, cache.window)
        acc = ctx.workspace.get("attn.part_acc", (n_dec, s.num_heads, nsplits, s.head_dim), torch.float32)
        ml = ctx.workspace.get("attn.part_ml", (n_dec, s.num_heads, nsplits, 2), torch.float32)
        ops.attn_decode_bf16(q, o, cache.k, cache.v, ctx.decode_tokens, n_dec, ctx.positions,
                             ctx.seq_of_token, cache.table, acc, ml, nsplits, s.num_heads, s.num_kv_heads,
                             s.head_dim, cache.page_size, mixer.scale, cache.window)
    if n_tiles:
        ops.attn_prefill_bf16(q, o, cache.k, cache.v, ctx.prefill_tiles, n_tiles, ctx.positions,
                              ctx.seq_of_token, cache.table, s.num_heads, s.num_kv_heads, s.head_dim,
                              cache.page_size, mixer.scale, cache.window)
    return True
