"""ctypes binding of the kernel library: argument types, error translation.

The library is loaded (and, if need be, compiled) at the first use of ``lib()``.
There is no fallback: if it cannot be built or loaded, the caller gets the error.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

from pyre_amd.hip import build as _build

ABI_VERSION = 19


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


P, I, L, F = c_void_p, c_int, c_long, c_float

_SIGNATURES = {
    "pyre_read_probe": [P, ctypes.c_size_t, I, P, P],
    "pyre_embed": [P, I, P, P, I, I, P],
    "pyre_add_rmsnorm": [P, P, I, I, L, P, I, P, I, P, I, P, I, I, F, P],
    "pyre_rope_kv_write": [P, I, I, L, P, I, P, I, P, P, I, P, P, I, P, P, I, I, I, I, I, I, P],
    "pyre_silu_mul": [P, I, I, L, P, I, I, I, P],
    "pyre_reduce_partials": [P, I, I, L, P, I, P, I, I, I, P],
    "pyre_fill_rows": [P, I, L, I, I, L, P, I, ctypes.c_uint, P],
    "pyre_gemm_generic": [P, I, L, P, P, I, L, P, I, P, I, L, I, I, I, P],
    "pyre_gemm_f32": [P, L, P, L, P, I, P, L, L, I, I, I, I, P],
    "pyre_attn_generic": [P, P, I, P, P, I, P, P, P, P, I, I, I, I, I, I, F, I, I, P, I, P],
    "pyre_attn_generic_spans": [I],
    "pyre_attn_prefill_f32": [P, P, P, P, P, I, P, P, P, I, I, I, I, I, F, I, P],
    "pyre_attn_mfma_supports": [I, I, I, I],
    "pyre_attn_decode_work_bf16": [P, P, P, P, P, I, P, P, P, I, P, P, P, I, I, I, I, I, F, I, P],
    "pyre_attn_decode_work_rope_supports": [I, I, I, I, L],
    "pyre_attn_decode_work_rope_bf16": [P, I, L, P, I, P, P, P, I, I, P, P, P, P, I, P, P, P, I, P, P, P, I, I, I, I, I, F, I, P],
    "pyre_attn_prefill_bf16": [P, P, P, P, P, I, P, P, P, I, I, I, I, I, F, I, P],
    "pyre_attn_prefill_waves": [I, I],
    "pyre_attn_prefill_work_bf16": [P, P, P, P, P, I, P, P, I, P, P, P, I, I, I, I, I, F, I, P],
    "pyre_argmax": [P, L, P, P, I, I, P],
    "pyre_argmax_static": [P, L, P, I, I, P],
    "pyre_argmax_static_init": [],
    "pyre_compute_units": [],
    "pyre_gemm_skinny_supports": [I, I, I, L, L],
    "pyre_gemm_skinny_bf16": [P, L, P, L, P, I, I, I, I, P],
    "pyre_gemm_skinny_silu_bf16": [P, L, P, L, P, I, I, I, P],
    "pyre_gemm_mid_supports": [I, I, I, L, L],
    "pyre_gemm_mid_bf16": [P, L, P, L, P, I, I, I, I, I, P],
    "pyre_gemm_mid_silu_blocks": [I, I],
    "pyre_gemm_mid_silu_bf16": [P, L, P, L, P, I, I, I, P],
    "pyre_sample": [P, L, P, P, P, I, I, P],
    "pyre_feed_tokens": [P, P, P, I, P],
}

_lib = None


def _open(path) -> ctypes.CDLL:
    handle = ctypes.CDLL(str(path))
    handle.pyre_last_error.restype = ctypes.c_char_p
    handle.pyre_abi_version.restype = c_int
    return handle


def _fits(handle) -> bool:
    """The library speaks this binding's ABI and was compiled from the sources of this tree."""
    if handle.pyre_abi_version() != ABI_VERSION or not hasattr(handle, "pyre_sources_digest"):
        return False
    handle.pyre_sources_digest.restype = ctypes.c_char_p
    return handle.pyre_sources_digest().decode() == _build.sources_digest()


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        handle = _open(_build.ensure_built())
        if not _fits(handle):
            # A library from other sources under a stamp that says otherwise (a copied build
            # folder, an older checkout): rebuild once. The loader keeps the mapping of a path
            # it has already opened, so the new build is opened under a name of its own.
            import os
            import shutil

            path = _build.build(force=True)
            fresh = path.with_name(f"{path.stem}.{os.getpid()}{path.suffix}")
            shutil.copyfile(path, fresh)
            try:
                handle = _open(fresh)
            finally:
                os.unlink(fresh)
            if not _fits(handle):
                raise KernelError(f"kernel library has ABI {handle.pyre_abi_version()} and the binding expects "
                                  f"{ABI_VERSION}, or it does not carry the digest of the sources it was built "
                                  "from: sources and binding are out of step")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = c_int
        _lib = handle
    return _lib


def loaded_path() -> str | None:
    return None if _lib is None else _lib._name


_entry_points: dict = {}


def call(name: str, *args) -> None:
    fn = _entry_points.get(name)
    if fn is None:
        fn = _entry_points[name] = getattr(lib(), name)
    if fn(*args) != 0:
        raise KernelError(lib().pyre_last_error().decode(errors="replace"))
