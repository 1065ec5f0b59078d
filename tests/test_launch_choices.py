"""The host-side choices of how a kernel's work is cut: they decide nothing about the
result's value, but a bad one leaves parts of k undone or asks a kernel for more
than it takes."""

import random

import numpy as np

from pyre_amd.parts.attention_work import (DECODE_MAX_BLOCKS_PER_REQUEST, DEFAULT_UNITS, decode_alone, decode_capacity,
                                           decode_work, prefill_slots, prefill_work)
from pyre_amd.parts.fast import SKINNY_MAX_KSPLIT, skinny_ksplit


def test_split_k_leaves_no_part_empty_and_is_a_function_of_the_sizes():
    rng = random.Random(0)
    shapes = [(4608, 3584), (3584, 3584), (3584, 18944), (152064, 3584), (2048, 1536), (1536, 8960), (64, 64),
              (96, 256), (131, 8), (70000, 96)]
    shapes += [(rng.randrange(1, 9000), 8 * rng.randrange(1, 3000)) for _ in range(200)]
    for n_out, k in shapes:
        ks = skinny_ksplit(8, n_out, k)
        assert 1 <= ks <= SKINNY_MAX_KSPLIT
        runs = -(-k // 128)
        per = -(-runs // ks)                       # runs of 128 k per part, as the kernel rounds
        assert (ks - 1) * per < runs, (n_out, k, ks)  # the last part starts inside k
        assert ks == 1 or per >= 4
        assert ks == skinny_ksplit(64, n_out, k) == skinny_ksplit(8, n_out, k)  # rows do not matter: eager = replayed


def test_split_k_of_the_7b_products():
    # 56 row blocks x 9 parts = 504 blocks for 256 compute units; 72 x 7 = 504
    assert skinny_ksplit(8, 3584, 18944) == 9
    assert skinny_ksplit(8, 4608, 3584) == 7


def _chunks(pos, window):
    lo = np.maximum(0, pos - window + 1) if window > 0 else np.zeros_like(pos)
    return pos // 32 - lo // 32 + 1


def _check_work(work, tokens, positions, rows, window, nq, nkv):
    """What the decode kernel relies on: every chunk of every request belongs to exactly one
    wave of one block, slots are disjoint, and the list fits the launch."""
    n_blocks = int(work[0, 0])
    assert work.shape == (1 + n_blocks, 4)
    assert n_blocks <= decode_capacity(rows, nq, nkv)
    chunks = dict(zip(tokens.tolist(), _chunks(positions[tokens].astype(np.int64), window).tolist()))
    seen, slots = {}, set()
    for tok, b_nb, per, slot0 in work[1:].tolist():
        b, nb = b_nb % 65536, b_nb // 65536
        assert 1 <= nb <= DECODE_MAX_BLOCKS_PER_REQUEST and 0 <= b < nb and per >= 1
        assert 4 * per * nb >= chunks[tok] > 4 * per * (nb - 1)        # all chunks covered, no block without one
        seen.setdefault(tok, []).append(b)
        assert slot0 + b not in slots and 0 <= slot0 and slot0 + nb <= n_blocks
        slots.add(slot0 + b)
    assert sorted(seen) == sorted(tokens.tolist())
    assert all(sorted(bs) == list(range(len(bs))) for bs in seen.values())
    longest_first = [chunks[t] for t in dict.fromkeys(work[1:, 0].tolist())]
    assert longest_first == sorted(longest_first, reverse=True)


def test_decode_work_lists_cover_every_key_once():
    rng = np.random.default_rng(1)
    for case in range(300):
        n = int(rng.integers(1, 300))
        rows = n + int(rng.integers(0, 20))
        nkv = int(rng.choice([1, 2, 4, 8]))
        nq = nkv * int(rng.choice([1, 2, 7, 8, 20]))
        window = int(rng.choice([0, 0, 50, 4096]))
        top = int(rng.choice([40, 700, 5000, 70000]))
        # single tokens somewhere in a flat batch of other tokens, contexts log-uniform
        flat = n + int(rng.integers(0, 50))
        tokens = np.sort(rng.choice(flat, n, replace=False)).astype(np.int32)
        positions = np.zeros(flat, dtype=np.int32)
        positions[tokens] = np.exp(rng.uniform(0, np.log(top), n)).astype(np.int32) - 1
        work = decode_work(tokens, positions, rows, window, nq, nkv)
        _check_work(work, tokens, positions, rows, window, nq, nkv)
        # the padding of a captured step (requests at position 0) changes nothing for the others
        pad = rows - n
        padded_tokens = np.concatenate([tokens, np.arange(flat, flat + pad, dtype=np.int32)])
        padded_pos = np.concatenate([positions, np.zeros(pad, dtype=np.int32)])
        padded = decode_work(padded_tokens, padded_pos, rows, window, nq, nkv)
        _check_work(padded, padded_tokens, padded_pos, rows, window, nq, nkv)
        real = padded[1:][np.isin(padded[1:, 0], tokens)]
        assert (real[:, :3] == work[1:, :3]).all()                    # same blocks, same chunks per wave
    assert (decode_work(np.zeros(0, np.int32), np.zeros(4, np.int32), 8, 0, 4, 2) == 0).all()


def test_decode_work_carries_position_and_table_row_to_the_device():
    from pyre_amd.parts.attention_work import decode_work_with_places

    positions = np.asarray([5, 900, 0, 4000, 33], dtype=np.int32)
    seq_of = np.asarray([3, 0, 4, 1, 2], dtype=np.int32)
    tokens = np.asarray([1, 3, 4], dtype=np.int32)
    work = decode_work(tokens, positions, 4, 0, 8, 2)
    wide = decode_work_with_places(work, positions, seq_of)
    assert wide.shape == (len(work), 8) and wide.dtype == np.int32
    assert (wide[:, :4] == work).all() and (wide[0, 4:] == 0).all() and (wide[:, 6:] == 0).all()
    for tok, pos, seq in wide[1:, [0, 4, 5]].tolist():
        assert pos == positions[tok] and seq == seq_of[tok]


def test_decode_work_of_known_shapes():
    # 7B heads (28 query, 4 key/value: 64 blocks per key/value head at once), 4,096 tokens of context
    pos = lambda n, ctx: np.full(n, ctx, dtype=np.int32)  # noqa: E731
    tok = lambda n: np.arange(n, dtype=np.int32)          # noqa: E731
    assert decode_alone(8, 28, 4) and decode_alone(64, 28, 4) and not decode_alone(65, 28, 4)
    w = decode_work(tok(8), pos(8, 4096), 8, 0, 28, 4)
    assert w[0, 0] == 56 and (w[1:, 1] // 65536 == 7).all() and (w[1:, 2] == 5).all()   # 7 blocks of 4 x 5 for 129 chunks
    w = decode_work(tok(64), pos(64, 4096), 64, 0, 28, 4)
    assert w[0, 0] == 64 and (w[1:, 1] == 65536).all() and (w[1:, 2] == 33).all()       # a block each: nothing crosses blocks
    w = decode_work(tok(48), pos(48, 4096), 48, 0, 28, 4)
    assert w[0, 0] <= 64                                               # still one round
    for n in (96, 256):                                                # two blocks a unit: whole requests again
        w = decode_work(tok(n), pos(n, 4096), n, 0, 28, 4)
        assert w[0, 0] == n and (w[1:, 2] == 33).all()
    # one request of 16,384 tokens: 513 chunks in blocks of sqrt(513 / 2) = 16, not of the 9 that 64 blocks would hold
    w = decode_work(tok(1), pos(1, 16384), 1, 0, 28, 4)
    assert w[0, 0] == 33 and (w[1:, 2] == 4).all()
    # 256 requests of very different lengths on two key/value heads: the long ones are cut
    rng = np.random.default_rng(0)
    p = np.exp(rng.uniform(np.log(16), np.log(2560), 256)).astype(np.int32)
    w = decode_work(tok(256), p, 256, 0, 12, 2)
    assert w[1, 1] // 65536 >= 4 and w[1, 0] == int(np.argmax(p))
    assert 4 * w[1:, 2].max() * 32 <= p.sum() // 256 + 256             # a block is about half a slot's share
    chunks_of = dict(zip(range(256), (p // 32 + 1).tolist()))
    assert all(nb == 1 for t, nb in zip(w[1:, 0].tolist(), (w[1:, 1] // 65536).tolist()) if chunks_of[t] <= 16)   # and 16 chunks at least


def test_prefill_work_lists_cover_every_chunk_once():
    rng = np.random.default_rng(2)
    for case in range(200):
        items = int(rng.choice([1, 2, 4, 8, 16]))
        window = int(rng.choice([0, 0, 100, 3000]))
        # a few requests with portions of any length at any depth of their context
        tiles, positions = [], []
        for _ in range(int(rng.integers(1, 6))):
            start = int(rng.choice([0, 0, 37, 5000, 30000]))
            n = int(rng.integers(2, int(rng.choice([40, 700, 3000]))))
            base = len(positions)
            positions += list(range(start, start + n))
            tiles += [(t0, min(32, base + n - t0)) for t0 in range(base, base + n, 32)]
        tiles, positions = np.asarray(tiles, dtype=np.int32), np.asarray(positions, dtype=np.int32)
        work = prefill_work(tiles, positions, window, items)
        assert len(work) <= len(tiles) + 2 * DEFAULT_UNITS
        seen, slots = {}, set()
        for t0, ntok, c0, c1, slot0, b, nb, _ in work.tolist():
            assert c0 <= c1 and 0 <= b < nb
            seen.setdefault((t0, ntok), []).append((b, nb, c0, c1))
            if nb > 1:
                assert slot0 + b not in slots and slot0 + nb <= prefill_slots(work)
                slots.add(slot0 + b)
        assert sorted(seen) == sorted(map(tuple, tiles.tolist()))
        for (t0, ntok), blocks in seen.items():
            pos0 = int(positions[t0])
            lo = max(0, pos0 - window + 1) if window else 0
            blocks.sort()
            assert [b for b, *_ in blocks] == list(range(blocks[0][1]))
            assert blocks[0][2] == lo // 64 and blocks[-1][3] == (pos0 + ntok - 1) // 64
            assert all(x[3] + 1 == y[2] for x, y in zip(blocks, blocks[1:]))     # neither a gap nor an overlap
        assert len(slots) == prefill_slots(work)
    # 512 tokens at the end of 32,768 on 4 key/value heads: 16 tiles, each dealt to 4 blocks (64 blocks a head)
    positions = np.arange(32768 - 512, 32768, dtype=np.int32)
    tiles = np.asarray([(t0, 32) for t0 in range(0, 512, 32)], dtype=np.int32)
    work = prefill_work(tiles, positions, 0, 4)
    assert len(work) == 64 and (work[:, 6] == 4).all()
    # a whole prompt of 8,192 tokens: 256 tiles are plenty, none is cut
    positions = np.arange(8192, dtype=np.int32)
    tiles = np.asarray([(t0, 32) for t0 in range(0, 8192, 32)], dtype=np.int32)
    work = prefill_work(tiles, positions, 0, 4)
    assert len(work) == 256 and work[0, 0] in (8128, 8160)               # a longest tile first
    assert prefill_work(np.zeros((0, 2), np.int32), positions, 0, 4).shape == (0, 8)


def test_workspace_hands_out_the_same_memory_until_a_buffer_grows():
    import torch

    from pyre_amd.engine.context import Workspace

    ws = Workspace(torch.device("cpu"))
    a = ws.get("x", (4, 8), torch.float32)
    assert ws.get("x", (4, 8), torch.float32) is a                     # the cached view
    b = ws.get("x", (2, 8), torch.float32)
    assert b.data_ptr() == a.data_ptr() and b.shape == (2, 8)          # a smaller view of the same buffer
    assert ws.get("x", (4, 8), torch.bfloat16).data_ptr() != a.data_ptr()  # another element type, another buffer
    big = ws.get("x", (16, 8), torch.float32)                          # grows: the old views are forgotten
    assert ws.get("x", (4, 8), torch.float32).data_ptr() == big.data_ptr()
    ws.keep_replaced = True                                            # as after a captured step
    before = big.data_ptr()
    bigger = ws.get("x", (64, 8), torch.float32)
    assert any(t.data_ptr() == before for t in ws._replaced)           # the captured step's memory stays allocated
    big = bigger
    ws.frozen = True
    assert ws.get("x", (64, 8), torch.float32) is big
    try:
        ws.get("x", (128, 8), torch.float32)
    except RuntimeError as e:
        assert "grow" in str(e)
    else:
        raise AssertionError("a frozen workspace must not grow")


def test_mid_ksplit_fills_one_round_and_leaves_no_part_empty():
    """The kernel that keeps up to 256 rows in a block is chosen where at least two parts of 384 k or more fill the
    256 compute units in one round of blocks of 64 output columns."""
    from pyre_amd.parts.fast import MID_MAX_KSPLIT, mid_ksplit

    assert mid_ksplit(1536, 8960) == 10 and mid_ksplit(3584, 18944) == 4 and mid_ksplit(4608, 3584) == 3
    assert mid_ksplit(37888, 3584) == 0 and mid_ksplit(17920, 1536) == 0 and mid_ksplit(152064, 3584) == 0
    assert mid_ksplit(96, 64) == 0 and mid_ksplit(64, 500) == 0
    for n_out in (1, 64, 65, 700, 2048, 8192, 9000):
        for k in (8, 256, 511, 512, 1000, 4096, 20000):
            ks = mid_ksplit(n_out, k)
            if ks:
                blocks = -(-n_out // 64)
                kper = -(-(-(-k // ks)) // 64) * 64
                assert 2 <= ks <= MID_MAX_KSPLIT and blocks * ks <= 256 and k // ks >= 384 and (ks - 1) * kper < k


def test_which_kernel_takes_a_product_is_a_function_of_its_sizes():
    """The choice between the weight-streaming kernel, the kernel that keeps a step's rows in a
    block (with 64 or 128 rows of the weights a block) and the BLAS library, for the shapes it was
    measured on; within the row counts between two sizes at which decode steps are captured the
    answer does not change, so that an eager step and its replay run the same kernels."""
    from pyre_amd.engine.batch import DECODE_ROW_BUCKETS
    from pyre_amd.parts.fast import MID_MAX_ROWS, narrow_kernel

    qkv7, down7 = (4608, 3584), (3584, 18944)
    assert narrow_kernel(8, *qkv7) == ("stream", 7, False) and narrow_kernel(24, *down7) == ("stream", 9, False)
    assert narrow_kernel(25, *qkv7) == narrow_kernel(64, *qkv7) == ("block", 7, True)       # 36 x 7 blocks of 128 rows
    assert narrow_kernel(48, *down7) == ("block", 9, True)
    assert narrow_kernel(65, *qkv7) == narrow_kernel(256, *qkv7) == ("block", 7, True)
    assert narrow_kernel(65, 2048, 1536) == narrow_kernel(256, 2048, 1536) == ("block", 4, False)   # 32 x 4 blocks of 64 rows
    assert narrow_kernel(257, *qkv7) == ("", 0, False)
    assert narrow_kernel(64, 5120, 27648) == ("block", 6, True)                             # the 32B shape's way down
    # the 1.5B shape: too few blocks either way, the kernel with the ring in LDS from one row on
    assert narrow_kernel(1, 2048, 1536) == narrow_kernel(64, 2048, 1536) == ("block", 4, False)
    assert narrow_kernel(8, 1536, 8960) == ("block", 10, False)
    assert narrow_kernel(8, 1536, 8960, {"mid_small": False})[0] == "stream"
    # a tiny model: the weight-streaming kernel, then the library; for tests the other kernel if asked for
    assert narrow_kernel(8, 96, 64)[0] == "stream" and narrow_kernel(100, 96, 64) == ("", 0, False)
    assert narrow_kernel(100, 96, 64, {"mid_gemm": 2}) == ("block", 1, False)
    assert narrow_kernel(8, *qkv7, {"mid_gemm": 0}) == ("stream", 7, False) and narrow_kernel(100, *qkv7, {"mid_gemm": 0})[0] == ""
    edges = [0] + [b for b in DECODE_ROW_BUCKETS if b <= MID_MAX_ROWS]
    for shape in (qkv7, down7, (3584, 3584), (2048, 1536), (1536, 8960), (7168, 5120), (5120, 27648), (96, 64), (1000, 4096)):
        for lo, hi in zip(edges, edges[1:]):
            assert len({narrow_kernel(n, *shape) for n in range(lo + 1, hi + 1)}) == 1, (shape, lo, hi)
