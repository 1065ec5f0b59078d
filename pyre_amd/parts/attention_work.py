"""The work lists of the MFMA attention kernels, planned on the host for every step.

Both kernels take their blocks from a list that deals each request's keys to blocks in
proportion to its context (``decode_work`` for single tokens, ``prefill_work`` for the tiles
of prompt portions); the lists are step arrays of the attention mixer, built from the step's
positions alone, so that a captured step replays with any mix of lengths. Nothing here
changes what is computed, only which block computes what and in how many parts a sum is
formed.
"""

from __future__ import annotations

import math

import numpy as np

#: compute units of the device that is planned for when nobody says (an MI355X). An engine reads
#: its device's number once (``Runtime.compute_units``) and plans with it; a unit runs one block of
#: the decode kernel at a time, or two
DEFAULT_UNITS = 256
#: keys per chunk of the decode kernel, and the fewest chunks a block is given if its request has them
DECODE_CHUNK = 32
DECODE_MIN_CHUNKS_PER_BLOCK = 8
#: the same when the blocks take several rounds anyway: every block has a start and an end worth
#: several chunks' time, and nothing is idle that more blocks could fill (measured in the serving
#: workload of 256 requests: 2.73 ms a captured step with 16, 2.77 with 8, 2.75 with 24, 2.80 with 32)
DECODE_MIN_CHUNKS_MANY_ROUNDS = 16
#: the most blocks that share one request (the kernel's limit)
DECODE_MAX_BLOCKS_PER_REQUEST = 64


def decode_items(nq: int, nkv: int) -> int:
    """Independent pieces of one request's attention: key/value heads times groups of 16 query heads."""
    return nkv * -(-(nq // nkv) // 16)


def decode_alone(rows: int, nq: int, nkv: int, units: int = DEFAULT_UNITS) -> bool:
    """Whether a step of ``rows`` single-token requests runs one block per compute unit: a
    block for every request and item then fits the chip at once. (Measured on the 7B heads:
    64 requests of 4,096 tokens take 79 us that way and 87 to 115 us with two blocks a unit,
    which the dispatcher does not spread evenly; 256 requests take 405 and 332 us.)"""
    return rows * decode_items(nq, nkv) <= units


def _decode_slots(rows: int, nq: int, nkv: int, units: int = DEFAULT_UNITS) -> int:
    """Blocks per item that run at once."""
    at_once = units if decode_alone(rows, nq, nkv, units) else 2 * units
    return max(1, at_once // decode_items(nq, nkv))


def decode_capacity(rows: int, nq: int, nkv: int, units: int = DEFAULT_UNITS) -> int:
    """Blocks that the work list of a step with ``rows`` single-token requests can come to."""
    return rows + 2 * _decode_slots(rows, nq, nkv, units) + 1


def decode_work(tokens: np.ndarray, positions: np.ndarray, rows: int, window: int, nq: int, nkv: int,
                size: int | None = None, units: int = DEFAULT_UNITS) -> np.ndarray:
    """The decode kernel's work list (int32 ``[1 + blocks, 4]``) for the single tokens
    ``tokens`` (flat indices) at ``positions``, planned as for ``rows`` requests (the rounded
    number: the missing ones count as requests of one chunk, which is what the padding of a
    captured step is, so that an eager step and a replayed one split alike).

    A request of c chunks of 32 keys gets ceil(c / size) blocks of four waves and deals its
    chunks evenly to them. The chip runs ``slots`` blocks per key/value item at once. If all
    blocks can run in one round, ``size`` is the smallest at which they do (but not so small
    that joining a request's blocks takes longer than the blocks): the step then takes as long
    as one block. Otherwise (or if that is slower) ``size`` is half of what a
    slot has to work off in all, and the list starts with the longest requests, so that the
    rounds stay full to the end. Row 0 is (blocks, 0, 0, 0), row 1 + i is (token, block of its
    request + 65536 * blocks of its request, chunks per wave, first partial slot of the
    request). ``size`` fixes the block size instead (for tests of the kernel). The device gets the
    list from :func:`decode_work_with_places`."""
    n = len(tokens)
    if n == 0:
        return np.zeros((1, 4), dtype=np.int32)
    pos = positions[tokens].astype(np.int64)
    lo = np.maximum(0, pos - window + 1) if window > 0 else np.zeros_like(pos)
    chunks = pos // DECODE_CHUNK - lo // DECODE_CHUNK + 1
    padding = max(0, rows - n)
    total, longest = int(chunks.sum()) + padding, int(chunks.max())
    slots = _decode_slots(rows, nq, nkv, units)
    if size is None:
        size = -(-total // (2 * slots))  # many rounds: half a slot's share
        least = DECODE_MIN_CHUNKS_MANY_ROUNDS
        if n + padding <= slots:
            a, b = 1, longest  # the smallest block size at which one round holds all blocks
            while a < b:
                mid = (a + b) // 2
                if int((-(-chunks // mid)).sum()) + padding <= slots:
                    b = mid
                else:
                    a = mid + 1
            if a <= 3 * size:  # one round of blocks of a, against total / slots + size for many rounds
                # The block that joins a request's blocks takes about half a chunk's time for each
                # of them: size + chunks / (2 size) is least at sqrt(chunks / 2).
                size, least = max(a, math.isqrt(longest // 2)), DECODE_MIN_CHUNKS_PER_BLOCK
        size = max(size, least)
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


def decode_work_with_places(work: np.ndarray, positions: np.ndarray, seq_of_token: np.ndarray) -> np.ndarray:
    """The list as the kernel reads it (int32 ``[1 + blocks, 8]``): each row of :func:`decode_work`
    followed by (position of its token, row of its request's block table, 0, 0), so that a block
    finds them with the row itself and not by two more loads that depend on it."""
    out = np.zeros((len(work), 8), dtype=np.int32)
    out[:, :4] = work
    tok = work[1:, 0]
    out[1:, 4] = positions[tok]
    out[1:, 5] = seq_of_token[tok]
    return out


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


def prefill_work(tiles: np.ndarray, positions: np.ndarray, window: int, items: int, size: int | None = None,
                 units: int = DEFAULT_UNITS) -> np.ndarray:
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
    slots = max(1, units // items)
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


def prefill_capacity(max_tokens: int, max_seqs: int, tile: int, items: int, units: int = DEFAULT_UNITS) -> int:
    """Blocks that the work list of a step of up to ``max_tokens`` tokens in ``max_seqs`` requests can
    come to: its tiles, and the two rounds of blocks more that :func:`prefill_work` allows itself."""
    return max_tokens // tile + max_seqs + 2 * max(1, units // items) + 1


def prefill_slots(work: np.ndarray) -> int:
    """Partial slots that a work list of :func:`prefill_work` uses."""
    shared = work[:, 6] > 1
    return int((work[shared, 4] + work[shared, 6]).max()) if shared.any() else 0
