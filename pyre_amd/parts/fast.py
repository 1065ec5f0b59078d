"""Choice of the MFMA kernels of the 16-bit path.

Each function returns None when its fast kernel does not take the case (element
type, sizes, alignment); the caller then runs the general kernel. Nothing here
changes what is computed, only by which kernel.
"""

from __future__ import annotations


def linear(lin, ctx, x, n, out):
    return None


def attention(mixer, ctx, q, o, cache) -> bool:
    return False
