"""The engine against the plain implementation: the same requests whole, with the
last 32 tokens one by one, in portions of changing size, and mixed with other
requests on so few pages that they are used again; in float32 and in bfloat16."""

from __future__ import annotations

import pytest
import torch

from helpers import TOL, cut, first_bad, make_engine, plain_logits, random_ids, replay

pytestmark = pytest.mark.gpu

#: (model, element type, page size): every shape on 16-token pages, and the shape whose workload
#: is defined on 8-token pages (and a tied one) on those
CASES = [(m, d, 16) for m in ("tiny-a", "tiny-b", "tiny-c", "tiny-d") for d in ("float32", "bfloat16")]
CASES += [("tiny-b", "float32", 8), ("tiny-b", "bfloat16", 8), ("tiny-a", "float32", 8), ("tiny-c", "bfloat16", 32)]
LENGTHS = {"a": 97, "b": 64, "c": 33, "d": 150}


def _requests(vocab):
    return {r: random_ids(vocab, n, seed=ord(r) * 7 + n) for r, n in LENGTHS.items()}


def _expected(plain, reqs, dtype):
    rounding = torch.bfloat16 if dtype == "bfloat16" else None
    return {r: plain_logits(plain, ids, rounding) for r, ids in reqs.items()}


@pytest.fixture(scope="module")
def engines(model_dirs):
    cache = {}

    def get(model, dtype, **kw):
        key = (model, dtype, tuple(sorted(kw.items())))
        if key not in cache:
            cache[key] = make_engine(model_dirs[model], dtype, **kw)
        return cache[key]

    return get


@pytest.mark.parametrize("model,dtype,page", CASES)
def test_whole(model, dtype, page, engines, plain_models):
    plain = plain_models[model]
    reqs = _requests(plain[0]["vocab_size"])
    eng = engines(model, dtype, page_size=page)
    steps = [([(r, ids, list(range(len(ids))))], [r]) for r, ids in reqs.items()]
    got = replay(eng, steps)
    assert len(got) == sum(LENGTHS.values())
    bad, worst = first_bad(got, _expected(plain, reqs, dtype), TOL[dtype])
    assert bad is None, bad
    eng.cache.check_invariants()
    assert eng.cache.page_groups[0].allocator.num_used == 0


@pytest.mark.parametrize("model,dtype,page", CASES)
def test_tail_token_by_token(model, dtype, page, engines, plain_models):
    plain = plain_models[model]
    reqs = _requests(plain[0]["vocab_size"])
    eng = engines(model, dtype, page_size=page)
    steps = []
    for r, ids in reqs.items():
        head = len(ids) - 32
        steps.append(([(r, ids[:head], [head - 1])], []))
        for i in range(head, len(ids)):
            steps.append(([(r, ids[i:i + 1], [0])], [r] if i == len(ids) - 1 else []))
    got = replay(eng, steps)
    bad, worst = first_bad(got, _expected(plain, reqs, dtype), TOL[dtype])
    assert bad is None, bad
    assert eng.cache.page_groups[0].allocator.num_used == 0


@pytest.mark.parametrize("model,dtype,page", CASES)
def test_ragged_portions(model, dtype, page, engines, plain_models):
    plain = plain_models[model]
    reqs = _requests(plain[0]["vocab_size"])
    eng = engines(model, dtype, page_size=page)
    steps = []
    for r, ids in reqs.items():
        pos = 0
        portions = cut(len(ids), [17, 5, 2, 32, 3, 2, 21])
        for k, n in enumerate(portions):
            steps.append(([(r, ids[pos:pos + n], list(range(n)))], [r] if k == len(portions) - 1 else []))
            pos += n
    got = replay(eng, steps)
    assert len(got) == sum(LENGTHS.values())
    bad, worst = first_bad(got, _expected(plain, reqs, dtype), TOL[dtype])
    assert bad is None, bad


@pytest.mark.parametrize("model,dtype,page", CASES)
def test_mixed_with_page_reuse(model, dtype, page, engines, plain_models):
    """Up to four live requests; portions of some beside decoded tokens of others.
    The pool holds 320 tokens (20 pages of 16) while the requests need 24 pages of 16 in
    total, so later requests get pages that earlier ones gave back."""
    plain = plain_models[model]
    vocab = plain[0]["vocab_size"]
    lengths = {"p": 70, "q": 45, "r": 100, "s": 38, "t": 66, "u": 51}
    reqs = {r: random_ids(vocab, n, seed=n) for r, n in lengths.items()}
    eng = engines(model, dtype, max_cached_tokens=320, page_size=page)
    pool = 320 // page
    order = list(reqs)
    fed = {r: 0 for r in reqs}
    prefill_until = {r: lengths[r] - 12 for r in reqs}   # then one token at a time
    live, waiting, steps = [], order[:], []
    k = 0
    while live or waiting:
        while waiting and len(live) < 4:
            # admit only if the whole request fits beside the live ones
            need = sum(-(-lengths[r] // page) for r in live) + -(-lengths[waiting[0]] // page)
            if need > pool:
                break
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            ids = reqs[r]
            if fed[r] < prefill_until[r]:
                n = min([9, 23, 2, 14][k % 4], prefill_until[r] - fed[r])
                if prefill_until[r] - fed[r] - n == 1:
                    n += 1
            else:
                n = 1
            k += 1
            entries.append((r, ids[fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
            if fed[r] == lengths[r]:
                end.append(r)
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    got = replay(eng, steps)
    assert len(got) == sum(lengths.values())
    bad, worst = first_bad(got, _expected(plain, reqs, dtype), TOL[dtype])
    assert bad is None, bad
    eng.cache.check_invariants()
    assert eng.cache.page_groups[0].allocator.num_used == 0


@pytest.mark.parametrize("model,dtype,graphs,mid", [
    ("tiny-c", "bfloat16", True, 1), ("tiny-c", "bfloat16", False, 1), ("tiny-c", "float32", True, 1),
    ("tiny-b", "bfloat16", True, 1), ("tiny-d", "float32", True, 1), ("tiny-c", "bfloat16", True, 0),
    ("tiny-b", "bfloat16", False, 0)])
def test_decode_steps_of_many_requests(model, dtype, graphs, mid, model_dirs, plain_models):
    """64 live requests, one token each per step, shrinking to 49, 33, 24 and 17 as requests
    end: every row of every step against the plain implementation. Captured steps run at
    padded sizes (49 as 64, 33 as 48, 17 as 24); their padding rows must change nothing.
    ``mid = 0``: all products of these steps in the weight-streaming kernels, which otherwise
    leave the gate/up product of a model this small to the kernel that keeps all rows in a block."""
    plain = plain_models[model]
    vocab = plain[0]["vocab_size"]
    prompt = [2 + (13 * i) % 61 for i in range(64)]                 # 2 to 62 tokens: page ends fall everywhere
    reqs = {i: random_ids(vocab, n + 10, 500 + i) for i, n in enumerate(prompt)}
    want = _expected(plain, reqs, dtype)
    eng = make_engine(model_dirs[model], dtype, use_graphs=graphs, max_num_seqs=64, max_cached_tokens=64 * 80,
                      max_num_batched_tokens=1024)
    eng.runtime.options["mid_gemm"] = mid
    steps = [([(i, reqs[i][:prompt[i]], [prompt[i] - 1]) for i in range(lo, min(lo + 16, 64))], []) for lo in range(0, 64, 16)]
    live = list(range(64))
    for k, keep in enumerate((64, 64, 64, 49, 49, 33, 33, 24, 17, 17)):
        end = live[keep:]
        if end:                                                     # they leave before this step
            steps[-1] = (steps[-1][0], end)
        live = live[:keep]
        steps.append(([(i, [reqs[i][prompt[i] + k]], [0]) for i in live], []))
    steps[-1] = (steps[-1][0], list(live))
    got = replay(eng, steps)
    assert len(got) == 64 + 3 * 64 + 2 * 49 + 2 * 33 + 24 + 2 * 17
    bad, worst = first_bad(got, want, TOL[dtype])
    assert bad is None, bad
    eng.cache.check_invariants()
    assert eng.cache.page_groups[0].allocator.num_used == 0
    if graphs:
        assert eng.graph_replays >= 4


@pytest.mark.parametrize("model,page,per_launch", [("tiny-c", 16, None), ("tiny-c", 32, None), ("tiny-c", 16, 5)])
def test_portions_late_in_a_long_prompt(model, page, per_launch, model_dirs, plain_models, monkeypatch):
    """700 tokens at once, then portions of 64, 40, 2 and 33 tokens, beside a second request's
    whole prompt: the few tiles of a late portion are dealt to several blocks each (the
    planner's choice is asserted), whose partial results join through memory. With five rows
    of the work list per launch the blocks of a tile also lie in different launches."""
    from pyre_amd.parts import attention_work as fast
    from pyre_amd.parts import fast as kernel_choice

    if per_launch:
        monkeypatch.setattr(kernel_choice, "PREFILL_MAX_LAUNCH", per_launch)

    plain = plain_models[model]
    cfg = plain[0]
    ids = random_ids(cfg["vocab_size"], 839, seed=5)
    other = random_ids(cfg["vocab_size"], 90, seed=6)
    eng = make_engine(model_dirs[model], "bfloat16", page_size=page, max_cached_tokens=1200, max_num_batched_tokens=1024)
    cuts = [0, 700, 764, 804, 806, 839]
    steps = []
    for k, (a, b) in enumerate(zip(cuts, cuts[1:])):
        entries = [("a", ids[a:b], list(range(b - a)) if a else [b - a - 1])]
        if k == 2:
            entries.append(("b", other, list(range(90))))
        steps.append((entries, ["a", "b"] if b == 839 else []))
    got = replay(eng, steps)
    want = {"a": plain_logits(plain, ids, torch.bfloat16), "b": plain_logits(plain, other, torch.bfloat16)}
    bad, worst = first_bad(got, want, TOL["bfloat16"])
    assert bad is None, bad
    import numpy as np
    tiles = np.asarray([[0, 32], [32, 32]], dtype=np.int32)
    work = fast.prefill_work(tiles, np.arange(700, 764, dtype=np.int32), 0,
                             fast.prefill_items(cfg["num_attention_heads"], cfg["num_key_value_heads"]))
    assert work[:, 6].min() >= 2


@pytest.mark.parametrize("others,graphs", [(30, True), (30, False), (150, True)])
def test_decode_steps_of_requests_of_very_different_lengths(others, graphs, model_dirs, plain_models):
    """One request of 900 tokens and one of 400 among many of 3 to 40: the decode kernel's
    work list deals the long ones to several blocks, which join their results through memory,
    and puts them first; with 150 others two blocks share a compute unit. Ten decoded tokens
    each, captured and replayed (or eager), every row against the plain implementation."""
    plain = plain_models["tiny-c"]
    vocab = plain[0]["vocab_size"]
    prompt = {0: 40, 1: 900, 2: 7, 3: 400}
    prompt.update({i: 3 + (11 * i) % 38 for i in range(4, others + 2)})
    reqs = {i: random_ids(vocab, n + 10, 1300 + i) for i, n in prompt.items()}
    want = _expected(plain, reqs, "bfloat16")
    n = len(reqs)
    eng = make_engine(model_dirs["tiny-c"], "bfloat16", use_graphs=graphs, max_num_seqs=n,
                      max_cached_tokens=1400 + 64 * n, max_num_batched_tokens=1024)
    ids = sorted(reqs)
    steps, batch, size = [], [], 0
    for i in ids:                                                    # whole prompts, packed into steps of up to 1,000 tokens
        if size + prompt[i] > 1000:
            steps.append((batch, []))
            batch, size = [], 0
        batch.append((i, reqs[i][:prompt[i]], [prompt[i] - 1]))
        size += prompt[i]
    steps.append((batch, []))
    for k in range(10):
        steps.append(([(i, [reqs[i][prompt[i] + k]], [0]) for i in ids], ids if k == 9 else []))
    got = replay(eng, steps)
    assert len(got) == 11 * n
    bad, worst = first_bad(got, want, TOL["bfloat16"])
    assert bad is None, bad
    eng.cache.check_invariants()
    if graphs:
        assert eng.graph_replays >= 7


@pytest.mark.parametrize("model,dtype,graphs,mid", [("tiny-c", "bfloat16", True, 1), ("tiny-c", "bfloat16", False, 1),
                                                    ("tiny-b", "float32", True, 1), ("tiny-c", "bfloat16", True, 2),
                                                    ("tiny-a", "bfloat16", False, 2)])
def test_decode_steps_beyond_the_weight_streaming_kernels(model, dtype, graphs, mid, model_dirs, plain_models):
    """200, 150, 100 and 70 live requests: decode steps whose products go to the BLAS library
    (more than 64 rows) or, with mid = 2, all to the kernel that keeps a step's rows in a block, which a tiny
    model's sizes would not choose; captured at 256, 192, 128 and 96 rows and replayed several
    times, each replay against the plain implementation (a library call that records a clearing
    of memory into the graph would be right once and wrong afterwards)."""
    plain = plain_models[model]
    vocab = plain[0]["vocab_size"]
    prompt = [2 + (13 * i) % 37 for i in range(200)]
    reqs = {i: random_ids(vocab, n + 12, 900 + i) for i, n in enumerate(prompt)}
    want = _expected(plain, reqs, dtype)
    eng = make_engine(model_dirs[model], dtype, use_graphs=graphs, max_num_seqs=200, max_cached_tokens=200 * 64,
                      max_num_batched_tokens=2048)
    eng.runtime.options["mid_gemm"] = mid
    steps = [([(i, reqs[i][:prompt[i]], []) for i in range(lo, lo + 50)], []) for lo in range(0, 200, 50)]
    live, counts = list(range(200)), (200, 200, 200, 150, 150, 150, 100, 100, 100, 70, 70, 70)
    for k, keep in enumerate(counts):
        end = live[keep:]
        if end:
            steps[-1] = (steps[-1][0], end)
        live = live[:keep]
        steps.append(([(i, [reqs[i][prompt[i] + k]], [0]) for i in live], []))
    steps[-1] = (steps[-1][0], list(live))
    got = replay(eng, steps)
    assert len(got) == sum(counts)
    bad, worst = first_bad(got, want, TOL[dtype])
    assert bad is None, bad
    assert eng.cache.page_groups[0].allocator.num_used == 0
    if graphs:
        assert eng.graph_replays == 8      # of each size: once eagerly, then captured and replayed twice


@pytest.mark.parametrize("model,dtype", [("tiny-c", "bfloat16"), ("tiny-c", "float32"), ("tiny-b", "bfloat16")])
def test_decode_steps_of_more_requests_than_a_captured_step_takes(model, dtype, model_dirs, plain_models):
    """300, then 257 live requests, one token each per step: more rows than the largest captured
    step (256) and than the kernels that keep a step's rows in a block take. Such a step runs
    eagerly at its own size, its products in the BLAS library (or the 32-bit tile kernel), the
    decode attention's list planned for two blocks a compute unit; every row of every step
    against the plain implementation. Then 256 of them, which is captured again."""
    plain = plain_models[model]
    vocab = plain[0]["vocab_size"]
    prompt = [2 + (17 * i) % 45 for i in range(300)]
    reqs = {i: random_ids(vocab, n + 8, 2100 + i) for i, n in enumerate(prompt)}
    want = _expected(plain, reqs, dtype)
    eng = make_engine(model_dirs[model], dtype, use_graphs=True, max_num_seqs=300, max_cached_tokens=300 * 64,
                      max_num_batched_tokens=2048)
    steps = [([(i, reqs[i][:prompt[i]], []) for i in range(lo, lo + 60)], []) for lo in range(0, 300, 60)]
    live, counts = list(range(300)), (300, 300, 257, 257, 256, 256, 256)
    for k, keep in enumerate(counts):
        end = live[keep:]
        if end:
            steps[-1] = (steps[-1][0], end)
        live = live[:keep]
        steps.append(([(i, [reqs[i][prompt[i] + k]], [0]) for i in live], []))
    steps[-1] = (steps[-1][0], list(live))
    got = replay(eng, steps)
    assert len(got) == sum(counts)
    bad, worst = first_bad(got, want, TOL[dtype])
    assert bad is None, bad
    eng.cache.check_invariants()
    assert eng.cache.page_groups[0].allocator.num_used == 0
    assert eng.graph_replays == 2                                    # the steps of 256: once eagerly, then captured and replayed


@pytest.mark.parametrize("model,dtype,page", [("tiny-b", "float32", 8), ("tiny-c", "bfloat16", 16), ("tiny-a", "bfloat16", 16)])
def test_mixed_with_page_reuse_on_poisoned_pages(model, dtype, page, model_dirs, plain_models):
    """The mixed trace again with the debug mode that fills every freed page with NaN: a
    kernel that read a page its request does not hold would put NaN into the logits."""
    test_mixed_with_page_reuse(model, dtype, page, lambda m, d, **kw: make_engine(model_dirs[m], d, debug_poison=True, **kw),
                               plain_models)


@pytest.mark.parametrize("model,dtype,page", [("tiny-c", "bfloat16", 16), ("tiny-b", "float32", 8), ("tiny-a", "bfloat16", 16)])
def test_long_decoding_against_plain(model, dtype, page, model_dirs, plain_models):
    """A prompt of five tokens, then 250 tokens one by one (captured steps, replayed): every
    row against the plain implementation while the context crosses many page ends and the
    block table grows past its first width."""
    plain = plain_models[model]
    ids = random_ids(plain[0]["vocab_size"], 255, seed=77)
    eng = make_engine(model_dirs[model], dtype, use_graphs=True, page_size=page)
    steps = [([("a", ids[:5], list(range(5)))], [])]
    steps += [([("a", ids[i:i + 1], [0])], ["a"] if i == 254 else []) for i in range(5, 255)]
    got = replay(eng, steps)
    assert len(got) == 255
    bad, worst = first_bad(got, {"a": plain_logits(plain, ids, torch.bfloat16 if dtype == "bfloat16" else None)}, TOL[dtype])
    assert bad is None, bad
    assert eng.graph_replays > 200


@pytest.mark.parametrize("graphs", [False, True])
def test_single_tokens_with_and_without_the_kernel_between_product_and_attention(graphs, model_dirs, plain_models):
    """Steps of single tokens leave the rotary kernel out on the 16-bit path (the attention kernel
    finishes the q/k/v product itself); with the option off they run it. Three requests decoded side
    by side after prompts of different lengths, one joining late, pages filling up: the same bits
    either way, in the logits of every step."""
    plain = plain_models["tiny-c"]
    vocab = plain[0]["vocab_size"]
    reqs = {r: random_ids(vocab, n, seed=n) for r, n in (("a", 70), ("b", 41), ("c", 90))}
    steps = [([(r, reqs[r][:n], [n - 1])], []) for r, n in (("a", 20), ("b", 9))]
    steps += [([("a", reqs["a"][20 + i:21 + i], [0]), ("b", reqs["b"][9 + i:10 + i], [0])], []) for i in range(12)]
    steps += [([("c", reqs["c"][:50], [49])], [])]
    steps += [([("a", reqs["a"][32 + i:33 + i], [0]), ("b", reqs["b"][21 + i:22 + i], [0]), ("c", reqs["c"][50 + i:51 + i], [0])],
               ["b"] if i == 19 else []) for i in range(20)]
    steps += [([("a", reqs["a"][52 + i:53 + i], [0]), ("c", reqs["c"][70 + i:71 + i], [0])], ["a", "c"] if i == 17 else [])
              for i in range(18)]
    outs = []
    for fused in (True, False):
        eng = make_engine(model_dirs["tiny-c"], "bfloat16", use_graphs=graphs, page_size=16)
        eng.runtime.options["rope_in_attention"] = fused
        outs.append(replay(eng, steps))
    assert outs[0].keys() == outs[1].keys() and len(outs[0]) == 3 + 24 + 60 + 36
    assert all(torch.equal(outs[0][k], outs[1][k]) for k in outs[0])
    want = {r: plain_logits(plain, ids, torch.bfloat16) for r, ids in reqs.items()}
    bad, _ = first_bad(outs[0], want, TOL["bfloat16"])
    assert bad is None, bad


def test_weights_stored_in_32_bits_run_in_either_mode(tmp_path, plain_models):
    """A tensor stored in 32 bits stays so: a float32 checkpoint runs in the 16-bit
    mode with float32 weights (mixed products), and exactly in the 32-bit mode."""
    import plain_qwen2 as P
    from conftest import TINY, tiny_config
    from pyre_amd.weights import write_random_model

    folder = write_random_model(tmp_path / "f32", tiny_config("tiny-b"), dtype="float32", **TINY["tiny-b"])
    plain = (P.read_config(folder), P.read_weights(folder))
    ids = random_ids(1000, 90, seed=5)
    for dtype in ("float32", "bfloat16"):
        eng = make_engine(folder, dtype)
        assert eng.model.layers[0].mixer.qkv.weight.dtype == torch.float32
        steps = [([("a", ids[:50], list(range(50)))], []), ([("a", ids[50:], list(range(40)))], ["a"])]
        got = replay(eng, steps)
        want = {"a": plain_logits(plain, ids, torch.bfloat16 if dtype == "bfloat16" else None)}
        bad, _ = first_bad(got, want, TOL[dtype])
        assert bad is None, bad


def test_requests_longer_than_the_models_own_limit(model_dirs, plain_models):
    """max_position_embeddings is a default, not a bound (the reference never consults it)."""
    plain = plain_models["tiny-a"]                       # max_position_embeddings = 256
    ids = random_ids(512, 300, seed=8)
    eng = make_engine(model_dirs["tiny-a"], "float32", max_model_len=320)
    got = replay(eng, [([("a", ids[:280], [0, 279])], []), ([("a", ids[280:], list(range(20)))], ["a"])])
    bad, _ = first_bad(got, {"a": plain_logits(plain, ids)}, TOL["float32"])
    assert bad is None, bad
