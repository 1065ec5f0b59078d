"""The host-side choices of how a kernel's work is cut: they decide nothing about the
result's value, but a bad one leaves parts of k undone or asks a kernel for more
than it takes."""

import random

from pyre_amd.parts.fast import (DECODE_MAX_SPLITS, DECODE_MIN_KEYS_PER_SPLIT, SKINNY_MAX_KSPLIT, decode_splits,
                                 skinny_ksplit)


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


def test_decode_splits_stay_within_what_the_kernel_takes():
    rng = random.Random(1)
    for _ in range(300):
        n = rng.randrange(1, 65)
        nkv = rng.choice([1, 2, 4, 8])
        nq = nkv * rng.choice([1, 2, 7, 8, 20])
        ctx = rng.randrange(1, 40000)
        window = rng.choice([0, 0, 50, 4096])
        s = decode_splits(n, nq, nkv, ctx, window)
        assert 1 <= s <= DECODE_MAX_SPLITS
        span = min(ctx, window + 32) if window > 0 else ctx
        assert s == 1 or (s - 1) * DECODE_MIN_KEYS_PER_SPLIT < span  # no split without keys of its own


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
