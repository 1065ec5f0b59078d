"""The kernels as functions of torch tensors.

torch is the allocator and the owner of the stream here, nothing more: every
function checks shapes, element types, device and contiguity on the host, then
hands raw pointers to the HIP library. There is no CPU path; a tensor that is
not on a GPU is an error.
"""

from __future__ import annotations

from dataclasses import dataclass
from functools import lru_cache

import torch

from pyre_amd.hip.lib import KernelError, call

_DT = {torch.float32: 0, torch.bfloat16: 1}


def dtype_code(t: torch.Tensor | torch.dtype) -> int:
    dt = t if isinstance(t, torch.dtype) else t.dtype
    try:
        return _DT[dt]
    except KeyError:
        raise KernelError(f"unsupported element type {dt}; kernels take float32 and bfloat16") from None


_STREAM: int | None = None


def use_stream(handle: int | None) -> None:
    """Put every kernel on this HIP stream until told otherwise (None: ask torch for its
    current stream at every call again). A step asks once instead of once per kernel."""
    global _STREAM
    _STREAM = handle


def _stream() -> int:
    return _STREAM if _STREAM is not None else torch.cuda.current_stream().cuda_stream


def _dev(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operand is not on a GPU (there is no CPU path)")


def _contig(name: str, t: torch.Tensor) -> None:
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")


def _i32(name: str, t: torch.Tensor, n: int | None = None) -> None:
    if t.dtype != torch.int32:
        raise KernelError(f"{name} must be int32, got {t.dtype}")
    _contig(name, t)
    if n is not None and t.numel() < n:
        raise KernelError(f"{name} holds {t.numel()} entries, {n} needed")


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


@dataclass
class Partials:
    """What a matrix product hands to its consumer: ``S`` partial sums ``[S, M, N]``
    (``S`` = 1 unless the product was split along K) and a bias not yet added.
    The consumer adds them up in the order 0..S-1, then the bias."""

    data: torch.Tensor
    bias: torch.Tensor | None = None

    def __post_init__(self) -> None:
        if self.data.dim() != 3 or not self.data.is_contiguous():
            raise KernelError("partials must be a contiguous [S, M, N] tensor")

    @property
    def count(self) -> int:
        return self.data.shape[0]

    @property
    def rows(self) -> int:
        return self.data.shape[1]

    @property
    def width(self) -> int:
        return self.data.shape[2]

    @property
    def stride(self) -> int:
        return self.data.stride(0)

    def _args(self, width: int):
        if self.width != width:
            raise KernelError(f"partials are {self.width} wide, {width} expected")
        if self.bias is not None and self.bias.numel() != width:
            raise KernelError(f"bias has {self.bias.numel()} entries, {width} expected")
        return (self.data.data_ptr(), dtype_code(self.data), self.count, self.stride,
                _ptr(self.bias), dtype_code(self.bias) if self.bias is not None else 0)


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    """out[n] = float32(table[ids[n]]); ids must already be checked against the vocabulary."""
    _dev(table, ids, out)
    n, hidden = out.shape
    if table.dim() != 2 or table.shape[1] != hidden or out.dtype != torch.float32:
        raise KernelError("embed: table [V, H] and float32 out [N, H] expected")
    _contig("table", table), _contig("out", out), _i32("ids", ids, n)
    call("pyre_embed", table.data_ptr(), dtype_code(table), ids.data_ptr(), out.data_ptr(), n, hidden,
         _stream())


def add_rmsnorm(resid: torch.Tensor, delta: Partials | None, gain: torch.Tensor, eps: float,
                out: torch.Tensor, rows: torch.Tensor | None = None) -> None:
    """resid += delta (all partials, then bias); out = rmsnorm(resid) * gain.

    With ``rows`` only those rows are normed, into ``out[0:len(rows)]``, and
    ``resid`` is left as it was.
    """
    _dev(resid, gain, out, rows)
    hidden = resid.shape[-1]
    if resid.dtype != torch.float32 or resid.dim() != 2:
        raise KernelError("add_rmsnorm: the residual stream is float32 [N, H]")
    n = resid.shape[0] if rows is None else rows.numel()
    if out.shape[-1] != hidden or out.shape[0] < n or gain.numel() != hidden:
        raise KernelError("add_rmsnorm: shapes of out / gain do not fit the residual")
    _contig("resid", resid), _contig("out", out), _contig("gain", gain)
    if rows is not None:
        _i32("rows", rows)
    if delta is not None:
        if delta.rows < resid.shape[0]:
            raise KernelError("add_rmsnorm: delta has fewer rows than the residual")
        d = delta._args(hidden)
    else:
        d = (None, 0, 0, 0, None, 0)
    call("pyre_add_rmsnorm", resid.data_ptr(), *d, gain.data_ptr(), dtype_code(gain), out.data_ptr(),
         dtype_code(out), _ptr(rows), n, hidden, float(eps), _stream())


def rope_kv_write(qkv: Partials, q_out: torch.Tensor, k_cache: torch.Tensor | None,
                  v_cache: torch.Tensor | None, cos: torch.Tensor | None, sin: torch.Tensor | None,
                  rotary_dim: int, positions: torch.Tensor, slots: torch.Tensor | None, n: int,
                  nq: int, nkv: int, hd: int, page_size: int) -> None:
    """Finish the q/k/v projection (partials + bias), rotate q and k by position,
    store q in ``q_out [N, nq*hd]`` and, when a cache is given, k and v in their pages.

    ``k_cache`` is one layer's ``[pages, nkv, page_size, hd]``; ``v_cache`` the same
    layer's ``[pages, nkv, hd, page_size]``. ``slots[n] = page * page_size + offset``,
    or -1 for a token that is not to be stored.
    """
    _dev(qkv.data, q_out, k_cache, v_cache, cos, sin, positions, slots)
    width = (nq + 2 * nkv) * hd
    q = qkv._args(width)
    if qkv.rows < n or q_out.numel() < n * nq * hd:
        raise KernelError("rope_kv_write: buffers are smaller than the batch")
    _contig("q_out", q_out), _i32("positions", positions, n)
    write = k_cache is not None
    cache_dt = 0
    if write:
        if v_cache is None or slots is None:
            raise KernelError("rope_kv_write: k cache without v cache or slots")
        _i32("slots", slots, n), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
        if tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
            raise KernelError(f"rope_kv_write: cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} "
                              f"do not fit nkv={nkv} page={page_size} hd={hd}")
        cache_dt = dtype_code(k_cache)
    if rotary_dim:
        if cos is None or sin is None or cos.dtype != torch.float32 or sin.dtype != torch.float32:
            raise KernelError("rope_kv_write: float32 cos/sin tables needed")
        if cos.dim() != 2 or cos.shape[1] != rotary_dim // 2 or cos.shape != sin.shape:
            raise KernelError("rope_kv_write: cos/sin tables must be [positions, rotary_dim/2]")
        _contig("cos", cos), _contig("sin", sin)
    call("pyre_rope_kv_write", *q, q_out.data_ptr(), dtype_code(q_out), _ptr(k_cache), _ptr(v_cache),
         cache_dt, _ptr(cos), _ptr(sin), rotary_dim, positions.data_ptr(), _ptr(slots), n, nq, nkv, hd,
         page_size, 1 if write else 0, _stream())


def silu_mul(gu: Partials, out: torch.Tensor, n: int) -> None:
    """out[n, i] = silu(gate[n, i]) * up[n, i] with gate = gu[:, :I], up = gu[:, I:]."""
    _dev(gu.data, out)
    inter = out.shape[-1]
    if gu.width != 2 * inter or gu.rows < n or out.shape[0] < n:
        raise KernelError("silu_mul: gate/up buffer does not fit the output")
    if gu.bias is not None:
        raise KernelError("silu_mul: a pending bias is not supported")
    _contig("out", out)
    call("pyre_silu_mul", gu.data.data_ptr(), dtype_code(gu.data), gu.count, gu.stride, out.data_ptr(),
         dtype_code(out), n, inter, _stream())


def reduce_partials(p: Partials, out: torch.Tensor, n: int) -> None:
    _dev(p.data, out)
    if out.shape[-1] != p.width or out.shape[0] < n or p.rows < n:
        raise KernelError("reduce_partials: shapes do not fit")
    _contig("out", out)
    call("pyre_reduce_partials", *p._args(p.width), out.data_ptr(), dtype_code(out), n, p.width, _stream())


_FILL_PATTERNS = {(4, "zero"): 0, (2, "zero"): 0, (4, "nan"): 0x7FC00000, (2, "nan"): 0x7FC0}


def fill_rows(tensor: torch.Tensor, ids: list[int], value: float) -> None:
    """tensor[:, id] = value for every listed id; ``tensor`` is contiguous ``[outer, rows, ...]``
    of float32 or bfloat16, ``value`` is 0.0 or NaN (state slots are zeroed with it, freed pages
    poisoned)."""
    import ctypes
    import math

    _dev(tensor)
    _contig("tensor", tensor)
    if tensor.dim() < 2 or tensor.dtype not in _DT:
        raise KernelError("fill_rows: a float32 or bfloat16 tensor [outer, rows, ...] expected")
    if not ids:
        return
    kind = "nan" if math.isnan(value) else "zero" if value == 0.0 else None
    if kind is None:
        raise KernelError("fill_rows: the value must be 0 or NaN")
    outer, rows = tensor.shape[0], tensor.shape[1]
    row_elems = tensor.stride(1)
    arr = (ctypes.c_int * len(ids))(*[int(i) for i in ids])
    with torch.cuda.device(tensor.device):
        call("pyre_fill_rows", tensor.data_ptr(), tensor.element_size(), tensor.stride(0), outer, rows, row_elems,
             ctypes.cast(arr, ctypes.c_void_p), len(ids), _FILL_PATTERNS[(tensor.element_size(), kind)], _stream())


def gemm_generic(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor,
                 m: int, a_rows: torch.Tensor | None = None) -> None:
    """out[0:m] = a[0:m] (or a[a_rows]) @ w.T (+ bias), fp32 accumulation in ascending k."""
    _dev(a, w, bias, out, a_rows)
    n_out, k = w.shape
    if a.dim() != 2 or a.shape[1] != k or out.dim() != 2 or out.shape[1] != n_out:
        raise KernelError(f"gemm: a {tuple(a.shape)} @ w {tuple(w.shape)}.T -> out {tuple(out.shape)} do not fit")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: rows must be contiguous")
    if out.shape[0] < m or (a_rows is None and a.shape[0] < m):
        raise KernelError("gemm: fewer rows than m")
    if a_rows is not None:
        _i32("a_rows", a_rows, m)
    if bias is not None and bias.numel() != n_out:
        raise KernelError("gemm: bias length")
    call("pyre_gemm_generic", a.data_ptr(), dtype_code(a), a.stride(0), _ptr(a_rows), w.data_ptr(),
         dtype_code(w), w.stride(0), _ptr(bias), dtype_code(bias) if bias is not None else 0,
         out.data_ptr(), dtype_code(out), out.stride(0), m, n_out, k, _stream())


F32_KSPLIT_MAX = 8

#: compute units that launch plans are made for when nobody names a device (an MI355X)
DEFAULT_UNITS = 256


def compute_units(device=None) -> int:
    """Compute units of ``device`` (torch's current one if None), as the kernel library sees
    them: its kernels that fill the chip in one round of blocks go by the same number."""
    from pyre_amd.hip.lib import lib

    if device is None:
        return int(lib().pyre_compute_units())
    with torch.cuda.device(device):
        return int(lib().pyre_compute_units())


def gemm_f32_ksplit(n_out: int, k: int, units: int = DEFAULT_UNITS) -> int:
    """Into how many parts of k the float32 product is split: enough blocks of 128 output
    columns for the ``units`` compute units, parts of at least 512. A function of the weight's
    shape (and the engine's device) alone, never of the rows, so that a row's result does not
    depend on its step."""
    blocks = -(-n_out // 128)
    return max(1, min(F32_KSPLIT_MAX, units // blocks, k // 512))


def gemm_f32(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor, m: int,
             ksplit: int = 1) -> None:
    """out[0:m] = a[0:m] @ w.T (+ bias) with float32 operands and result, on the matrix cores'
    float32 instruction; the order of an element's additions depends on k alone. With
    ``ksplit`` > 1, ``out`` is [ksplit, m, N]: partial sums over parts of k (the bias in part 0)."""
    _dev(a, w, bias, out)
    n_out, k = w.shape
    if a.dtype != torch.float32 or w.dtype != torch.float32 or out.dtype != torch.float32:
        raise KernelError("gemm_f32: float32 operands and result expected")
    if a.dim() != 2 or a.shape[1] != k or out.shape[-1] != n_out or out.dim() != (2 if ksplit == 1 else 3):
        raise KernelError(f"gemm_f32: a {tuple(a.shape)} @ w {tuple(w.shape)}.T -> out {tuple(out.shape)} do not fit")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(-1) != 1:
        raise KernelError("gemm_f32: rows must be contiguous")
    if out.shape[-2] < m or a.shape[0] < m or (ksplit > 1 and (out.shape[0] != ksplit or out.shape[1] != m)):
        raise KernelError("gemm_f32: fewer rows than m, or partial sums that are not [ksplit, m, N]")
    if bias is not None and bias.numel() != n_out:
        raise KernelError("gemm_f32: bias length")
    call("pyre_gemm_f32", a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), _ptr(bias),
         dtype_code(bias) if bias is not None else 0, out.data_ptr(), out.stride(-2),
         out.stride(0) if ksplit > 1 else 0, m, n_out, k, ksplit, _stream())


def attn_generic(q: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                 n: int, nq: int, nkv: int, hd: int, page_size: int, scale: float,
                 window: int = 0, tokens: torch.Tensor | None = None,
                 scratch: torch.Tensor | None = None, matrix_cores: bool = True) -> None:
    """Causal attention of n tokens over the paged cache (``tokens``: which of the flat batch,
    else the first n); see attention_generic.hip. ``scratch``: float32 memory of
    ``attn_generic_scratch(...)`` elements for the partial results of the spans of keys; without
    it the memory is allocated here when the block table is wider than one span. ``matrix_cores``:
    float32 queries and caches with a head size of 16, 32, ..., 128 and pages of a multiple of 16
    tokens go to the kernel that serves the query heads of a key/value head from one read of its
    keys and values, on the matrix cores' float32 instruction (its sums run in another order than
    those of one block per head, which False asks for: a difference of rounding)."""
    _dev(q, out, k_cache, v_cache, positions, seq_of_token, block_table, tokens, scratch)
    if q.dtype != out.dtype or q.numel() < n * nq * hd or out.numel() < n * nq * hd:
        raise KernelError("attn: q/out buffers do not fit")
    if tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
        raise KernelError("attn: cache shapes do not fit the head geometry")
    if k_cache.dtype != v_cache.dtype:
        raise KernelError("attn: k and v caches differ in element type")
    _contig("q", q), _contig("out", out), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
    _i32("positions", positions, n), _i32("seq_of_token", seq_of_token, n)
    if tokens is not None:
        _i32("tokens", tokens, n)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("attn: block table must be int32 [rows, pages]")
    max_keys = _attn_generic_keys(block_table.shape[1], page_size, window)
    need = attn_generic_scratch(n, nq, hd, block_table.shape[1], page_size, window)
    if need and scratch is None:
        scratch = torch.empty(need, dtype=torch.float32, device=q.device)
    if need and (scratch.dtype != torch.float32 or not scratch.is_contiguous() or scratch.numel() < need):
        raise KernelError(f"attn: scratch of {need} float32 elements needed")
    per_launch = _attn_generic_rows(n, nq, hd, max_keys)
    flat_q, flat_out = q.view(-1), out.view(-1)
    for at in range(0, n, per_launch):
        rows = min(per_launch, n - at)
        if tokens is not None:  # the list moves on; q, out and positions are indexed by its entries
            args = (flat_q, flat_out, tokens[at:], positions, seq_of_token)
        else:
            args = (flat_q[at * nq * hd:], flat_out[at * nq * hd:], None, positions[at:], seq_of_token[at:])
        call("pyre_attn_generic", args[0].data_ptr(), args[1].data_ptr(), dtype_code(q), k_cache.data_ptr(),
             v_cache.data_ptr(), dtype_code(k_cache), _ptr(args[2]), args[3].data_ptr(), args[4].data_ptr(),
             block_table.data_ptr(), block_table.stride(0), rows, nq, nkv, hd, page_size, float(scale),
             int(window), max_keys, _ptr(scratch) if need else None, int(bool(matrix_cores)), _stream())


ATTN_GENERIC_SCRATCH = 1 << 25   #: float32 elements of scratch that one launch of attn_generic may use
#: the largest head that any attention kernel takes (attention_generic.hip's kMaxHead: a block of
#: 256 threads holds one element each) and the most query heads of a launch (a grid dimension)
ATTN_MAX_HEAD_DIM = 256
ATTN_MAX_HEADS = 65535


def _attn_generic_keys(table_width: int, page_size: int, window: int) -> int:
    """No token sees more keys than its block table holds, or than its window."""
    keys = max(1, table_width * page_size)
    return min(keys, window) if window > 0 else keys


def _attn_generic_rows(n: int, nq: int, hd: int, max_keys: int) -> int:
    """Tokens to a launch: all of them, or as many as the scratch of one launch allows."""
    from pyre_amd.hip.lib import lib

    spans = int(lib().pyre_attn_generic_spans(max_keys))
    return n if spans <= 1 else max(1, min(n, ATTN_GENERIC_SCRATCH // (nq * spans * (hd + 2))))


def attn_generic_scratch(n: int, nq: int, hd: int, table_width: int, page_size: int, window: int = 0) -> int:
    """Float32 elements of scratch that ``attn_generic`` needs for such a call (0: none)."""
    from pyre_amd.hip.lib import lib

    max_keys = _attn_generic_keys(table_width, page_size, window)
    spans = int(lib().pyre_attn_generic_spans(max_keys))
    return 0 if spans <= 1 or n <= 0 else _attn_generic_rows(n, nq, hd, max_keys) * nq * spans * (hd + 2)


def attn_prefill_f32(q, out, k_cache, v_cache, tiles, n_tiles, positions, seq_of_token, block_table,
                     nq, nkv, hd, page_size, scale, window=0) -> None:
    """Attention of prompt portions in true float32 on the matrix cores; ``tiles`` is int32
    [n_tiles, 2] = (first token, count <= 32)."""
    _dev(q, out, k_cache, v_cache, tiles, positions, seq_of_token, block_table)
    for name, t in (("q", q), ("out", out), ("k_cache", k_cache), ("v_cache", v_cache)):
        if t.dtype != torch.float32:
            raise KernelError(f"attn_prefill_f32: {name} must be float32")
        _contig(name, t)
    if tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
        raise KernelError("attn_prefill_f32: cache shapes do not fit the head geometry")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("attn_prefill_f32: block table must be int32 [rows, pages]")
    _i32("positions", positions), _i32("seq_of_token", seq_of_token), _i32("tiles", tiles, 2 * n_tiles)
    call("pyre_attn_prefill_f32", q.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         tiles.data_ptr(), n_tiles, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
         block_table.stride(0), nq, nkv, hd, page_size, float(scale), int(window), _stream())


ARGMAX_SCRATCH_PER_ROW = 128  #: 4-byte words of scratch per row of logits


def argmax(logits: torch.Tensor, out: torch.Tensor, scratch: torch.Tensor | None = None) -> None:
    """out[i] = index of the largest logit of row i (the lowest index among equals).
    ``scratch``: int32 or float32 device memory of 128 words per row (allocated if absent)."""
    _dev(logits, out, scratch)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax: float32 [M, V] logits expected")
    m = logits.shape[0]
    _i32("out", out, m)
    if scratch is None:
        scratch = torch.empty(m * ARGMAX_SCRATCH_PER_ROW, dtype=torch.int32, device=logits.device)
    if scratch.element_size() != 4 or scratch.numel() < m * ARGMAX_SCRATCH_PER_ROW or not scratch.is_contiguous():
        raise KernelError("argmax: scratch must hold 128 four-byte words per row")
    call("pyre_argmax", logits.data_ptr(), logits.stride(0), out.data_ptr(), scratch.data_ptr(), m,
         logits.shape[1], _stream())


ARGMAX_STATIC_MAX_ROWS = 256  #: rows that the library's built-in scratch holds


def argmax_static_init(device=None) -> None:
    """Look the built-in scratch's address up on ``device`` (torch's current one if None). The
    first :func:`argmax_static` on a device does this by itself, which must not happen while a
    stream is capturing: whoever captures calls this beforehand."""
    if device is None:
        call("pyre_argmax_static_init")
    else:
        with torch.cuda.device(device):
            call("pyre_argmax_static_init")


def argmax_static(logits: torch.Tensor, out: torch.Tensor) -> None:
    """:func:`argmax` for callers that must not allocate: the partial results go to an
    array inside the library's device image (at most 256 rows; calls that overlap on one
    GPU race)."""
    _dev(logits, out)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax: float32 [M, V] logits expected")
    m = logits.shape[0]
    _i32("out", out, m)
    with torch.cuda.device(logits.device):
        call("pyre_argmax_static", logits.data_ptr(), logits.stride(0), out.data_ptr(), m, logits.shape[1],
             _stream())


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
           out: torch.Tensor) -> None:
    """Rows with temperature > 0 get a token drawn by inverse CDF with their
    uniform number; rows with temperature <= 0 keep what ``out`` holds."""
    _dev(logits, temperature, uniform, out)
    m = logits.shape[0]
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample: float32 [M, V] logits expected")
    for name, t in (("temperature", temperature), ("uniform", uniform)):
        if t.dtype != torch.float32 or t.numel() < m or not t.is_contiguous():
            raise KernelError(f"sample: {name} must be contiguous float32 [M]")
    _i32("out", out, m)
    call("pyre_sample", logits.data_ptr(), logits.stride(0), temperature.data_ptr(), uniform.data_ptr(),
         out.data_ptr(), m, logits.shape[1], _stream())


def feed_tokens(tokens: torch.Tensor, src: torch.Tensor, ids: torch.Tensor, n: int) -> None:
    """tokens[i] = ids[src[i]] for i < n with src[i] >= 0 (all int32 on the device)."""
    _dev(tokens, src, ids)
    _i32("tokens", tokens, n), _i32("src", src, n), _i32("ids", ids)
    call("pyre_feed_tokens", tokens.data_ptr(), src.data_ptr(), ids.data_ptr(), n, _stream())


@lru_cache(maxsize=4096)
def attn_mfma_supports(hd: int, page_size: int, nq: int, nkv: int) -> bool:
    from pyre_amd.hip.lib import lib

    return bool(lib().pyre_attn_mfma_supports(hd, page_size, nq, nkv))


def _attn_common(q, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size):
    _dev(q, out, k_cache, v_cache, positions, seq_of_token, block_table)
    for name, t in (("q", q), ("out", out), ("k_cache", k_cache), ("v_cache", v_cache)):
        if t.dtype != torch.bfloat16:
            raise KernelError(f"attn (MFMA): {name} must be bfloat16")
        _contig(name, t)
    if tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
        raise KernelError("attn (MFMA): cache shapes do not fit the head geometry")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("attn (MFMA): block table must be int32 [rows, pages]")
    _i32("positions", positions), _i32("seq_of_token", seq_of_token)


def attn_decode_work_bf16(q, out, k_cache, v_cache, work, capacity, positions, seq_of_token, block_table,
                          part_acc, part_ml, counters, alone, nq, nkv, hd, page_size, scale, window=0) -> None:
    """Attention of single new tokens over the paged cache from a work list (int32
    ``[1 + blocks, 8]``: see ``pyre_attn_decode_work_bf16`` in pyre_api.h) in a launch of
    ``capacity`` blocks per key/value head, one (``alone``) or two to a compute unit.
    ``counters`` must be zero and is left at zero."""
    _attn_common(q, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size)
    _i32("work", work, 8 * (1 + capacity))
    items = nkv * -(-(nq // nkv) // 16)
    if part_acc.dtype != torch.float32 or part_acc.numel() < capacity * items * 16 * hd:
        raise KernelError("attn_decode_work: partial accumulators too small")
    if part_ml.dtype != torch.float32 or part_ml.numel() < capacity * items * 32:
        raise KernelError("attn_decode_work: partial max/sum buffer too small")
    if counters.dtype != torch.int32 or counters.numel() < capacity * items:
        raise KernelError("attn_decode_work: too few counters")
    call("pyre_attn_decode_work_bf16", q.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         work.data_ptr(), capacity, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
         block_table.stride(0), part_acc.data_ptr(), part_ml.data_ptr(), counters.data_ptr(), int(bool(alone)), nq,
         nkv, hd, page_size, float(scale), int(window), _stream())


@lru_cache(maxsize=4096)
def attn_decode_work_rope_supports(hd: int, page_size: int, nq: int, nkv: int, partial_stride: int) -> bool:
    from pyre_amd.hip.lib import lib

    return bool(lib().pyre_attn_decode_work_rope_supports(hd, page_size, nq, nkv, partial_stride))


def attn_decode_work_rope_bf16(qkv: Partials, cos, sin, slots, out, k_cache, v_cache, write_kv, work, capacity,
                               positions, seq_of_token, block_table, part_acc, part_ml, counters, alone, nq, nkv, hd,
                               page_size, scale, window=0) -> None:
    """:func:`attn_decode_work_bf16` for a step of single tokens, straight from the step's q/k/v
    product (float32 partial sums and bias): the kernel sums, biases and rotates the queries itself and
    writes each token's rotated key and its value into the cache (``write_kv``) with the arithmetic
    of :func:`rope_kv_write`, the same bits, so that no kernel runs between product and attention.
    ``cos``/``sin``: float32 ``[positions, hd / 2]`` (full-head rotation)."""
    _attn_common(out, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size)
    _dev(qkv.data, cos, sin, slots, work, part_acc, part_ml, counters)
    width = (nq + 2 * nkv) * hd
    args = qkv._args(width)
    if qkv.data.dtype != torch.float32:
        raise KernelError("attn_decode_work_rope: float32 partial sums expected")
    if not attn_decode_work_rope_supports(hd, page_size, nq, nkv, qkv.stride):
        raise KernelError(f"attn_decode_work_rope: head_dim {hd}, page_size {page_size}, heads {nq}/{nkv} are not taken")
    if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.dim() != 2 or cos.shape[1] != hd // 2 \
            or cos.shape != sin.shape:
        raise KernelError("attn_decode_work_rope: float32 cos/sin tables [positions, hd / 2] needed")
    _contig("cos", cos), _contig("sin", sin), _i32("slots", slots, qkv.rows), _i32("work", work, 8 * (1 + capacity))
    items = nkv * -(-(nq // nkv) // 16)
    if part_acc.dtype != torch.float32 or part_acc.numel() < capacity * items * 16 * hd:
        raise KernelError("attn_decode_work: partial accumulators too small")
    if part_ml.dtype != torch.float32 or part_ml.numel() < capacity * items * 32:
        raise KernelError("attn_decode_work: partial max/sum buffer too small")
    if counters.dtype != torch.int32 or counters.numel() < capacity * items:
        raise KernelError("attn_decode_work: too few counters")
    call("pyre_attn_decode_work_rope_bf16", args[0], args[2], args[3], args[4], args[5], cos.data_ptr(), sin.data_ptr(),
         slots.data_ptr(), qkv.rows, int(bool(write_kv)), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         work.data_ptr(), capacity, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
         block_table.stride(0), part_acc.data_ptr(), part_ml.data_ptr(), counters.data_ptr(), int(bool(alone)), nq,
         nkv, hd, page_size, float(scale), int(window), _stream())


def attn_prefill_bf16(q, out, k_cache, v_cache, tiles, n_tiles, positions, seq_of_token, block_table,
                      nq, nkv, hd, page_size, scale, window=0) -> None:
    """Attention of prompt portions, every wave reading the cache directly; ``tiles`` is int32
    [n_tiles, 2] = (first token, count <= 32)."""
    _attn_common(q, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size)
    _i32("tiles", tiles, 2 * n_tiles)
    call("pyre_attn_prefill_bf16", q.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         tiles.data_ptr(), n_tiles, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
         block_table.stride(0), nq, nkv, hd, page_size, float(scale), int(window), _stream())


@lru_cache(maxsize=4096)
def attn_prefill_waves(nq: int, nkv: int) -> int:
    from pyre_amd.hip.lib import lib

    return int(lib().pyre_attn_prefill_waves(nq, nkv))


def attn_prefill_work_bf16(q, out, k_cache, v_cache, work, n_items, partials, counters, n_slots, positions,
                           seq_of_token, block_table, nq, nkv, hd, page_size, scale, window=0) -> None:
    """Attention of prompt portions for heads of up to 128 elements from a work list (int32
    ``[n_items, 8]``: see ``pyre_attn_prefill_work_bf16`` in pyre_api.h) whose tiles of several
    blocks use the partial slots 0..n_slots-1. ``counters`` must be zero and is left at zero."""
    _attn_common(q, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size)
    _i32("work", work, 8 * n_items)
    waves = attn_prefill_waves(nq, nkv)
    per_slot = nkv * -(-(nq // nkv) // waves) * waves
    if n_slots:
        if partials.dtype != torch.float32 or partials.numel() < n_slots * per_slot * (hd // 32 * 1024 + 128):
            raise KernelError("attn_prefill_work: partial results do not fit")
        if counters.dtype != torch.int32 or counters.numel() < n_slots * per_slot:
            raise KernelError("attn_prefill_work: too few counters")
    call("pyre_attn_prefill_work_bf16", q.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         work.data_ptr(), n_items, _ptr(partials) if n_slots else None, _ptr(counters) if n_slots else None,
         n_slots, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0),
         nq, nkv, hd, page_size, float(scale), int(window), _stream())


@lru_cache(maxsize=4096)
def gemm_skinny_supports(m: int, n: int, k: int, ldx: int, ldw: int) -> bool:
    from pyre_amd.hip.lib import lib

    return bool(lib().pyre_gemm_skinny_supports(m, n, k, ldx, ldw))


def _skinny_common(x, w, m):
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny: bfloat16 operands expected")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.shape[0] < m:
        raise KernelError(f"gemm_skinny: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit {m} rows")
    if x.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError("gemm_skinny: rows must be contiguous")


def gemm_skinny_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, ksplit: int) -> None:
    """out[s] (float32 [ksplit, m, N]) = partial sums over k of x[0:m] @ w.T, 1 <= m <= 64."""
    _skinny_common(x, w, m)
    n = w.shape[0]
    if out.dtype != torch.float32 or not out.is_contiguous() or out.numel() < ksplit * m * n or not out.is_cuda:
        raise KernelError("gemm_skinny: out must be contiguous float32 [ksplit, m, N] on the GPU")
    call("pyre_gemm_skinny_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), m, n,
         w.shape[1], ksplit, _stream())


def gemm_skinny_silu_bf16(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, m: int) -> None:
    """out[0:m] (bfloat16 [m, I]) = silu(x @ gate.T) * (x @ up.T) with w_gate_up = [gate; up]."""
    _skinny_common(x, w_gate_up, m)
    two_i = w_gate_up.shape[0]
    if (out.dtype != torch.bfloat16 or not out.is_contiguous() or not out.is_cuda or out.dim() != 2
            or out.shape[1] * 2 != two_i or out.shape[0] < m):
        raise KernelError("gemm_skinny_silu: out must be contiguous bfloat16 [>= m, I] on the GPU")
    call("pyre_gemm_skinny_silu_bf16", x.data_ptr(), x.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
         out.data_ptr(), m, two_i, w_gate_up.shape[1], _stream())


@lru_cache(maxsize=4096)
def gemm_mid_supports(m: int, n: int, k: int, ldx: int, ldw: int) -> bool:
    from pyre_amd.hip.lib import lib

    return bool(lib().pyre_gemm_mid_supports(m, n, k, ldx, ldw))


def gemm_mid_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, ksplit: int, wide: bool = False) -> None:
    """out[s] (float32 [ksplit, m, N]) = partial sums over k of x[0:m] @ w.T, 1 <= m <= 256. ``wide``:
    a block takes 128 rows of w instead of 64."""
    _skinny_common(x, w, m)
    n = w.shape[0]
    if out.dtype != torch.float32 or not out.is_contiguous() or out.numel() < ksplit * m * n or not out.is_cuda:
        raise KernelError("gemm_mid: out must be contiguous float32 [ksplit, m, N] on the GPU")
    call("pyre_gemm_mid_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), m, n,
         w.shape[1], ksplit, int(wide), _stream())


@lru_cache(maxsize=4096)
def gemm_mid_silu_blocks(m: int, two_i: int) -> int:
    from pyre_amd.hip.lib import lib

    return int(lib().pyre_gemm_mid_silu_blocks(m, two_i))


def gemm_mid_silu_bf16(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, m: int) -> None:
    """out[0:m] (bfloat16 [m, I]) = silu(x @ gate.T) * (x @ up.T) with w_gate_up = [gate; up], 1 <= m <= 256."""
    _skinny_common(x, w_gate_up, m)
    two_i = w_gate_up.shape[0]
    if (out.dtype != torch.bfloat16 or not out.is_contiguous() or not out.is_cuda or out.dim() != 2
            or out.shape[1] * 2 != two_i or out.shape[0] < m):
        raise KernelError("gemm_mid_silu: out must be contiguous bfloat16 [>= m, I] on the GPU")
    call("pyre_gemm_mid_silu_bf16", x.data_ptr(), x.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
         out.data_ptr(), m, two_i, w_gate_up.shape[1], _stream())


def read_bandwidth(device: str = "cuda:0", gib: float = 2.0, blocks: int = 4096, repeats: int = 10) -> float:
    """Measured streaming-read bandwidth in GB/s (a buffer larger than every cache)."""
    import time

    n = int(gib * (1 << 30)) // 16 * 16
    buf = torch.empty(n, dtype=torch.uint8, device=device)
    buf.zero_()
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    with torch.cuda.device(buf.device):
        for _ in range(2):
            call("pyre_read_probe", buf.data_ptr(), n, blocks, sink.data_ptr(), _stream())
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(repeats):
            call("pyre_read_probe", buf.data_ptr(), n, blocks, sink.data_ptr(), _stream())
        torch.cuda.synchronize()
    return n * repeats / (time.perf_counter() - t) / 1e9
