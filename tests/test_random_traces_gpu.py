"""Random traces: requests of random lengths, cut into random portions (down to one
token), up to four live at a time in a random order, some left out of a step, on a pool
so small that pages are used again at once; every position's logits against the plain
implementation. The fixed traces of the other files each show one way of cutting; these
look for a combination nobody thought of."""

from __future__ import annotations

import random

import pytest
import torch

from helpers import TOL, first_bad, make_engine, plain_logits, random_ids, replay

pytestmark = pytest.mark.gpu


def random_trace(vocab: int, seed: int, max_live: int = 4, n_requests: int = 9):
    rng = random.Random(seed)
    reqs = {f"r{i}": random_ids(vocab, rng.choice([2, 3, 17, 31, 32, 33, 64, 65, 100, 129, 160]), seed * 100 + i)
            for i in range(n_requests)}
    fed = {r: 0 for r in reqs}
    waiting, live, steps = list(reqs), [], []
    while waiting or live:
        while waiting and len(live) < max_live and rng.random() < 0.7:
            live.append(waiting.pop(0))
        if not live:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in rng.sample(live, len(live)):
            if len(live) > 1 and rng.random() < 0.2:
                continue  # left out of this step; goes on later
            rest = len(reqs[r]) - fed[r]
            n = min(rest, rng.choice([1, 1, 1, 2, 3, 5, 16, 17, 32, 40, 64, 70]))
            want = sorted(rng.sample(range(n), rng.randint(0, min(n, 3)))) if rng.random() < 0.8 else list(range(n))
            entries.append((r, reqs[r][fed[r]:fed[r] + n], want))
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        if not entries:
            continue
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    return reqs, steps


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("model,dtype", [("tiny-a", "float32"), ("tiny-c", "bfloat16"), ("tiny-b", "bfloat16"),
                                         ("tiny-d", "float32")])
def test_random_trace(model, dtype, seed, model_dirs, plain_models, poison=False, page=16):
    plain = plain_models[model]
    reqs, steps = random_trace(plain[0]["vocab_size"], seed)
    rounding = torch.bfloat16 if dtype == "bfloat16" else None
    want = {r: plain_logits(plain, ids, rounding) for r, ids in reqs.items()}
    # four live requests of at most 160 tokens: 4 * 10 pages of 16, and not one more
    eng = make_engine(model_dirs[model], dtype, num_pages=40 * 16 // page, page_size=page, max_cached_tokens=None,
                      max_num_seqs=4, max_num_batched_tokens=512, use_graphs=seed == 1, debug_poison=poison)
    got = replay(eng, steps)
    assert got, "the trace asked for no logits"
    bad, worst = first_bad(got, want, TOL[dtype])
    assert bad is None, f"seed {seed}: {bad}"
    eng.cache.check_invariants()
    assert eng.cache.page_groups[0].allocator.num_used == 0


@pytest.mark.parametrize("model,dtype,seed,page", [("tiny-c", "bfloat16", 1, 16), ("tiny-b", "float32", 0, 8),
                                                   ("tiny-c", "bfloat16", 2, 32), ("tiny-d", "float32", 2, 16)])
def test_random_trace_on_poisoned_pages(model, dtype, seed, page, model_dirs, plain_models):
    """The same with every freed page and slot filled with NaN (and other page sizes): what a
    request reads of memory it does not hold would show as NaN in its logits."""
    test_random_trace(model, dtype, seed, model_dirs, plain_models, poison=True, page=page)
