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


def attention(mixer, ctx, q, o, cache) -> bool:
    return False
