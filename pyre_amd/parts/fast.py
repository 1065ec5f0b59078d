"""Choice of the faster kernels of the 16-bit path.

Each function returns None / False when its fast path does not take the case
(element type, sizes, alignment); the caller then runs the general kernel.
Nothing here changes what is computed, only by which kernel. Plain matrix
products with many rows go to the vendor's BLAS through ``torch.mm``, as the
reference's do (`pyre/model.py:84-87` are ``nn.Linear``); the true 32-bit path
never comes here.
"""

from __future__ import annotations

import math

import numpy as np
import torch

from pyre_amd.hip.ops import Partials

#: most rows the weight-streaming MFMA kernel takes; above, 16-bit products go to the BLAS library
SKINNY_MAX_ROWS = 64
#: the most partial sums of a weight-streaming product
SKINNY_MAX_KSPLIT = 12
#: up to this many rows the gate/up product and the SiLU-gate are one kernel
FUSED_SILU_MAX_ROWS = 64


def skinny_ksplit(m: int, n_out: int, k: int) -> int:
    """Into how many parts of k to split a weight-streaming product. A block (64 rows of the
    weights, 128 of wide ones) walks its part of k in dependent runs of 128, about 0.9 us
    each, and the blocks of a compute unit share its time: the product takes as long as the
    longest walk or as the unit with the most blocks needs for its bytes (6.5 TB/s over the
    256 units, measured on the 7B shapes), whichever is more; every part costs its consumer
    one more addend. The split with the least of that is chosen, at least four runs a part."""
    units, run_us, bytes_per_us, part_us = 256, 0.9, 6.5e6, 0.1
    tiles = -(-n_out // 16)
    row_blocks = -(-n_out // (128 if tiles >= 2048 else 64))
    runs = -(-k // 128)
    stream_us = 2.0 * n_out * k / bytes_per_us
    best, best_cost = 1, None
    for ks in range(1, SKINNY_MAX_KSPLIT + 1):
        per = -(-runs // ks)
        if ks > 1 and per < 4:
            break
        if -(-runs // per) != ks:
            continue  # would leave parts empty
        blocks = row_blocks * ks
        busiest = -(-blocks // units)
        cost = max(per * run_us, stream_us * busiest * units / blocks) + part_us * ks
        if best_cost is None or cost < best_cost - 1e-9:
            best, best_cost = ks, cost
    return best


#: products whose library result is kept in float32 instead of being rounded to 16 bits:
#: q/k/v (rotated and rounded once afterwards) and the attention output projection (added
#: to the float32 residual). Measured on the tiny test models this halves the 16-bit
#: path's distance from an exact run; it costs about 2 % of a 2,048-token prefill.
LIBRARY_F32_ROLES = frozenset({"attn.qkv", "attn.out"})


def _is_bf16(ctx, lin, x) -> bool:
    return (ctx.runtime.dtype == torch.bfloat16 and lin.weight.dtype == torch.bfloat16
            and x.dtype == torch.bfloat16)


def linear(lin, ctx, x, n, out):
    from pyre_amd.hip import ops

    rt = ctx.runtime
    if not _is_bf16(ctx, lin, x):
        return None
    k, n_out = lin.in_features, lin.out_features
    skinny = rt.options.get("skinny_gemm", True) and ops.gemm_skinny_supports(
        min(n, SKINNY_MAX_ROWS), n_out, k, x.stride(0), lin.weight.stride(0))
    library = rt.options.get("library_gemm", True)
    if skinny and (n <= SKINNY_MAX_ROWS or (out is not None and not library)):
        if out is not None:
            # float32 results wanted in place (the head's logits): no split, 64 rows at a time
            for r0 in range(0, n, SKINNY_MAX_ROWS):
                rows = min(SKINNY_MAX_ROWS, n - r0)
                ops.gemm_skinny_bf16(x[r0:r0 + rows], lin.weight, out[r0:r0 + rows], rows, 1)
            return Partials(out.view(1, n, n_out), lin.bias)
        ks = skinny_ksplit(n, n_out, k)
        buf = ctx.workspace.get(f"linear.{lin.role}.partials", (ks, n, n_out), torch.float32)
        ops.gemm_skinny_bf16(x, lin.weight, buf, n, ks)
        return Partials(buf, lin.bias)
    if not library:
        return None
    if out is not None:
        # many rows of float32 results in place (the head's logits of a large decode step, or of
        # every row of a portion): one pass over the weights in the library
        torch.mm(x if n == x.shape[0] else x[:n], lin.weight.t(), out_dtype=torch.float32, out=out)
        return Partials(out.view(1, n, n_out), lin.bias)
    if lin.role in rt.options.get("library_f32_roles", LIBRARY_F32_ROLES):
        buf = ctx.workspace.get(f"linear32.{lin.role}", (n, n_out), torch.float32)
        torch.mm(x if n == x.shape[0] else x[:n], lin.weight.t(), out_dtype=torch.float32, out=buf)
    else:
        buf = ctx.workspace.get(f"linear16.{lin.role}", (n, n_out), torch.bfloat16)
        torch.mm(x if n == x.shape[0] else x[:n], lin.weight.t(), out=buf)
    return Partials(buf.view(1, n, n_out), lin.bias)


def gate_up_silu(lin, ctx, x, n, act) -> bool:
    """silu(x gate^T) * (x up^T) in one kernel for a decode step's few rows."""
    from pyre_amd.hip import ops

    if not _is_bf16(ctx, lin, x) or n > FUSED_SILU_MAX_ROWS or lin.bias is not None:
        return False
    if not ctx.runtime.options.get("skinny_gemm", True):
        return False
    if not ops.gemm_skinny_supports(n, lin.out_features, lin.in_features, x.stride(0), lin.weight.stride(0)):
        return False
    ops.gemm_skinny_silu_bf16(x, lin.weight, act, n)
    return True


#: compute units; a unit runs one block of the decode kernel at a time, or two
DECODE_UNITS = 256
#: keys per chunk of the decode kernel, and the fewest chunks a block is given if its request has them
DECODE_CHUNK = 32
DECODE_MIN_CHUNKS_PER_BLOCK = 8
#: the most blocks that share one request (the kernel's limit)
DECODE_MAX_BLOCKS_PER_REQUEST = 64


def decode_items(nq: int, nkv: int) -> int:
    """Independent pieces of one request's attention: key/value heads times groups of 16 query heads."""
    return nkv * -(-(nq // nkv) // 16)


def decode_alone(rows: int, nq: int, nkv: int) -> bool:
    """Whether a step of ``rows`` single-token requests runs one block per compute unit: a
    block for every request and item then fits the chip at once. (Measured on the 7B heads:
    64 requests of 4,096 tokens take 79 us that way and 87 to 115 us with two blocks a unit,
    which the dispatcher does not spread evenly; 256 requests take 405 and 332 us.)"""
    return rows * decode_items(nq, nkv) <= DECODE_UNITS


def _decode_slots(rows: int, nq: int, nkv: int) -> int:
    """Blocks per item that run at once."""
    at_once = DECODE_UNITS if decode_alone(rows, nq, nkv) else 2 * DECODE_UNITS
    return max(1, at_once // decode_items(nq, nkv))


def decode_capacity(rows: int, nq: int, nkv: int) -> int:
    """Blocks that the work list of a step with ``rows`` single-token requests can come to."""
    return rows + 2 * _decode_slots(rows, nq, nkv) + 1


def decode_work(tokens: np.ndarray, positions: np.ndarray, rows: int, window: int, nq: int, nkv: int,
                size: int | None = None) -> np.ndarray:
    """The decode kernel's work list (int32 ``[1 + blocks, 4]``) for the single tokens
    ``tokens`` (flat indices) at ``positions``, planned as for ``rows`` requests (the rounded
    number: the missing ones count as requests of one chunk, which is what the padding of a
    captured step is, so that an eager step and a replayed one split alike).

    A request of c chunks of 32 keys gets ceil(c / size) blocks of four waves and deals its
    chunks evenly to them. The chip runs ``slots`` blocks per key/value item at once. If all
    blocks can run in one round, ``size`` is the smallest at which they do: the step then
    takes as long as one block. Otherwise (or if that is slower) ``size`` is half of what a
    slot has to work off in all, and the list starts with the longest requests, so that the
    rounds stay full to the end. Row 0 is (blocks, 0, 0, 0), row 1 + i is (token, block of its
    request + 65536 * blocks of its request, chunks per wave, first partial slot of the
    request). ``size`` fixes the block size instead (for tests of the kernel)."""
    n = len(tokens)
    if n == 0:
        return np.zeros((1, 4), dtype=np.int32)
    pos = positions[tokens].astype(np.int64)
    lo = np.maximum(0, pos - window + 1) if window > 0 else np.zeros_like(pos)
    chunks = pos // DECODE_CHUNK - lo // DECODE_CHUNK + 1
    padding = max(0, rows - n)
    total, longest = int(chunks.sum()) + padding, int(chunks.max())
    slots = _decode_slots(rows, nq, nkv)
    if size is None:
        size = -(-total // (2 * slots))  # many rounds: half a slot's share
        if n + padding <= slots:
            a, b = 1, longest  # the smallest block size at which one round holds all blocks
            while a < b:
                mid = (a + b) // 2
                if int((-(-chunks // mid)).sum()) + padding <= slots:
                    b = mid
                else:
                    a = mid + 1
            if a <= 3 * size:  # one round of blocks of a, against total / slots + size for many rounds
                size = a
        size = max(size, DECODE_MIN_CHUNKS_PER_BLOCK)
    size = max(size, -(-longest // DECODE_MAX_BLOCKS_PER_REQUEST))
    nb = -(-chunks // size)
    per = -(-chunks // (4 * nb))
    nb = -(-chunks // (4 * per))  # blocks that are left without a chunk by the rounding are dropped
    order = np.argsort(-chunks, kind="stable")
    nb_sorted = nb[order]
    first = np.cumsum(nb_sorted) - nb_sorted
    n_blocks = int(nb_sorted.sum())
    which = np.repeat(np.arange(n), nb_sorted)
    work = np.empty((1 + n_blocks, 4), dtype=np.int32)
    work[0] = (n_blocks, 0, 0, 0)
    work[1:, 0] = tokens[order][which]
    work[1:, 1] = np.arange(n_blocks) - first[which] + 65536 * nb_sorted[which]
    work[1:, 2] = per[order][which]
    work[1:, 3] = first[which]
    return work


#: keys per chunk of the prompt-portion kernel; a block of it fills a compute unit (its LDS)
PREFILL_CHUNK = 64
#: What a further block costs its tile, in chunks' worth of time: each block of a tile that has
#: several stores a partial result of 16 KB per head (4), and the wave that comes last reads
#: them all back (0.25 per block). Fitted to the kernel's times on the 7B heads: whole prompts
#: of 1,024 to 4,096 tokens and portions of 128 and 512 tokens after 4,096 to 32,768, each with
#: blocks of 6 to 512 chunks; the fit picks the fastest of the measured sizes in every case.
PREFILL_BLOCK_COST = 4.0
PREFILL_JOIN_COST = 0.25
#: block sizes that are tried, as parts of the longest tile
PREFILL_SIZES = (1, 3 / 4, 1 / 2, 3 / 8, 1 / 4, 3 / 16, 1 / 8, 3 / 32, 1 / 16, 3 / 64, 1 / 32, 1 / 64)


def prefill_items(nq: int, nkv: int) -> int:
    """Blocks per tile of the prompt-portion kernel: key/value heads times groups of as many
    query heads as a block has waves."""
    from pyre_amd.hip import ops

    return nkv * -(-(nq // nkv) // ops.attn_prefill_waves(nq, nkv))


def _deal(chunks: np.ndarray, size: int):
    """Blocks per tile and chunks per block when no block takes more than ``size`` chunks."""
    nb = -(-chunks // size)
    per = -(-chunks // nb)
    return -(-chunks // per), per


def _time_of(chunks: np.ndarray, size: int, slots: int) -> float:
    """How long the blocks of this deal take, in chunks' worth of time, when the dispatcher
    hands them, longest tile first, to whichever of ``slots`` units is free next."""
    nb, per = _deal(chunks, size)
    cost = np.where(nb > 1, per + PREFILL_BLOCK_COST + PREFILL_JOIN_COST * nb, per).astype(np.float64)
    jobs = np.repeat(cost, nb)  # tiles come longest first, their blocks together
    loads = np.zeros(slots)
    for i in range(0, len(jobs), slots):
        batch = jobs[i:i + slots]
        loads.sort()
        loads[:len(batch)] += batch
    return float(loads.max())


def prefill_work(tiles: np.ndarray, positions: np.ndarray, window: int, items: int, size: int | None = None) -> np.ndarray:
    """The prompt-portion kernel's work list (int32 ``[blocks, 8]``) for ``tiles`` ([T, 2]:
    first token, count) at ``positions``; ``items`` blocks run per tile and chunk range.

    A tile of c chunks of 64 keys gets ceil(c / size) blocks and deals its chunks evenly to
    them; a block fills a compute unit. ``size`` is the one of a few candidates (parts of the
    longest tile) with which the step is over soonest by a replay of the
    dispatcher on the blocks' estimated times. So the few tiles of a portion late in a long
    context spread over the whole chip, and the long tiles at the end of a whole prompt do not
    run alone, while many tiles are left whole. The longest tiles come first.
    Row i is (first token, tokens, first chunk, last chunk, first partial slot of the tile,
    this block's number among the tile's, their number, 0); tiles of one block use no slot.
    ``size`` fixes the block size instead (for tests of the kernel)."""
    if len(tiles) == 0:
        return np.zeros((0, 8), dtype=np.int32)
    t0, ntok = tiles[:, 0].astype(np.int64), tiles[:, 1].astype(np.int64)
    pos0 = positions[t0].astype(np.int64)
    lo = np.maximum(0, pos0 - window + 1) if window > 0 else np.zeros_like(pos0)
    first, last = lo // PREFILL_CHUNK, (pos0 + ntok - 1) // PREFILL_CHUNK
    chunks = last - first + 1
    order = np.argsort(-chunks, kind="stable")
    n, longest = len(tiles), int(chunks.max())
    slots = max(1, DECODE_UNITS // items)
    if size is None:
        size = longest
        if n < 4 * slots:  # with many tiles the units stay busy to the end anyway
            sorted_chunks = chunks[order]
            best = _time_of(sorted_chunks, size, slots)
            for part in PREFILL_SIZES[1:]:
                cand = math.ceil(longest * part)
                if cand < 2 or int(_deal(sorted_chunks, cand)[0].sum()) > n + 2 * slots:
                    break  # the list holds the tiles and two rounds of blocks more at most
                t = _time_of(sorted_chunks, cand, slots)
                if t < 0.97 * best:
                    size, best = cand, t
    nb, per = _deal(chunks, size)
    nb_sorted = nb[order]
    which = np.repeat(np.arange(n), nb_sorted)
    n_blocks = int(nb_sorted.sum())
    b = np.arange(n_blocks) - (np.cumsum(nb_sorted) - nb_sorted)[which]
    shared = np.where(nb_sorted > 1, nb_sorted, 0)
    slot0 = np.where(shared > 0, np.cumsum(shared) - shared, 0)[which]
    src = order[which]
    work = np.zeros((n_blocks, 8), dtype=np.int32)
    work[:, 0], work[:, 1] = t0[src], ntok[src]
    work[:, 2] = first[src] + b * per[src]
    work[:, 3] = np.minimum(last[src], work[:, 2] + per[src] - 1)
    work[:, 4], work[:, 5], work[:, 6] = slot0, b, nb_sorted[which]
    return work


def prefill_slots(work: np.ndarray) -> int:
    """Partial slots that a work list of :func:`prefill_work` uses."""
    shared = work[:, 6] > 1
    return int((work[shared, 4] + work[shared, 6]).max()) if shared.any() else 0


def attention(mixer, ctx, q, o, cache) -> bool:
    from pyre_amd.hip import ops

    s = mixer.spec
    k_pages, v_pages = cache["k"], cache["v"]
    if ctx.dtype != torch.bfloat16 or k_pages.dtype != torch.bfloat16:
        return False
    if not ctx.runtime.options.get("mfma_attention", True):
        return False
    if not ops.attn_mfma_supports(s.head_dim, cache.page_size, s.num_heads, s.num_kv_heads):
        return False
    hb = ctx.host
    dec, tiles = hb.arrays["attention.decode_tokens"], hb.arrays["attention.prefill_tiles"]
    n_dec, n_tiles = len(dec), len(tiles)
    if n_dec:
        # The launch's size follows from the step's rounded sizes and the list from the rounded
        # number of requests, so that a step gives bit for bit the same result whether it runs
        # eagerly or as a replayed graph at those sizes.
        rows, _ = hb.decode_shape()
        capacity = decode_capacity(rows, s.num_heads, s.num_kv_heads)
        items = decode_items(s.num_heads, s.num_kv_heads)
        acc = ctx.workspace.get("attn.part_acc", (capacity, items, 16, s.head_dim), torch.float32)
        ml = ctx.workspace.get("attn.part_ml", (capacity, items, 16, 2), torch.float32)
        counters = ctx.workspace.get("attn.counters", (capacity, items), torch.int32, zeroed=True)
        ops.attn_decode_work_bf16(q, o, k_pages, v_pages, ctx.arrays[mixer.decode_work_name], capacity, ctx.positions,
                                  ctx.seq_of_token, cache.table, acc, ml, counters,
                                  decode_alone(rows, s.num_heads, s.num_kv_heads), s.num_heads, s.num_kv_heads,
                                  s.head_dim, cache.page_size, mixer.scale, cache.window)
    if n_tiles and s.head_dim <= 128:
        work = hb.arrays[mixer.prefill_work_name]
        n_slots = prefill_slots(work)
        per_slot = prefill_items(s.num_heads, s.num_kv_heads) * ops.attn_prefill_waves(s.num_heads, s.num_kv_heads)
        partials = counters = None
        if n_slots:
            partials = ctx.workspace.get("attn.prefill_partials", (n_slots, per_slot, s.head_dim // 32 * 1024 + 128),
                                         torch.float32)
            counters = ctx.workspace.get("attn.prefill_counters", (n_slots, per_slot), torch.int32, zeroed=True)
        ops.attn_prefill_work_bf16(q, o, k_pages, v_pages, ctx.arrays[mixer.prefill_work_name], len(work), partials,
                                   counters, n_slots, ctx.positions, ctx.seq_of_token, cache.table, s.num_heads,
                                   s.num_kv_heads, s.head_dim, cache.page_size, mixer.scale, cache.window)
    elif n_tiles:
        ops.attn_prefill_bf16(q, o, k_pages, v_pages, ctx.arrays["attention.prefill_tiles"], n_tiles, ctx.positions,
                              ctx.seq_of_token, cache.table, s.num_heads, s.num_kv_heads, s.head_dim,
                              cache.page_size, mixer.scale, cache.window)
    return True
