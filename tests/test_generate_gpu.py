"""Generation through the entry points: greedy tokens against the plain
implementation, long decoding, sampling that does not depend on batch-mates,
captured (HIP graph) decode steps against eager ones, preemption when pages run out."""

from __future__ import annotations

import pytest
import torch

import plain_qwen2 as P
from helpers import random_ids

pytestmark = pytest.mark.gpu


def _load(folder, dtype, **kw):
    from pyre_amd.api import load_model

    args = dict(page_size=16, max_cached_tokens=2048, max_num_seqs=8, max_num_batched_tokens=256,
                prefill_chunk=32)
    args.update(kw)
    return load_model(str(folder), device="cuda:0", dtype=dtype, **args)[0]


def _plain_greedy_with_margin(plain, prompt, n):
    """Greedy tokens of the plain implementation and, for each, the gap between the
    two largest logits relative to the largest magnitude."""
    cfg, w = plain
    ids, toks, margins = list(prompt), [], []
    for _ in range(n):
        row = P.forward(w, cfg, ids)[-1]
        top = row.topk(2).values
        toks.append(int(row.argmax()))
        margins.append(float((top[0] - top[1]) / row.abs().max()))
        ids.append(toks[-1])
    return toks, margins


@pytest.mark.parametrize("model", ["tiny-a", "tiny-b", "tiny-c"])
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_matches_plain_fp32(model, graphs, model_dirs, plain_models):
    """32-bit greedy generation is token for token the plain implementation's
    (the reference's chain of exact equalities, tests/test_cache.py:71-96,
    tests/test_scheduler.py:20-64), prompts of 1, 7, 33 and 64 tokens together."""
    from pyre_amd.api import generate

    plain = plain_models[model]
    vocab = plain[0]["vocab_size"]
    prompts = [random_ids(vocab, n, seed=n) for n in (1, 7, 33, 64)]
    eng = _load(model_dirs[model], "float32", use_graphs=graphs)
    got = generate(eng, prompts, max_new_tokens=16)
    for p, g in zip(prompts, got):
        want, margins = _plain_greedy_with_margin(plain, p, 16)
        for i, (a, b) in enumerate(zip(g, want)):
            if a != b:
                assert margins[i] < 1e-5, f"token {i} differs ({a} vs {b}) with margin {margins[i]:.2e}"
                break
    assert eng.cache.page_groups[0].allocator.num_used == 0
    if graphs:
        assert eng.graph_replays > 0


@pytest.mark.parametrize("model", ["tiny-b", "tiny-c"])
def test_greedy_bf16_follows_plain_until_a_near_tie(model, model_dirs, plain_models):
    from pyre_amd.api import generate

    plain = plain_models[model]
    prompts = [random_ids(plain[0]["vocab_size"], n, seed=n + 3) for n in (5, 40)]
    eng = _load(model_dirs[model], "bfloat16")
    got = generate(eng, prompts, max_new_tokens=24)
    for p, g in zip(prompts, got):
        want, margins = _plain_greedy_with_margin(plain, p, 24)
        for i, (a, b) in enumerate(zip(g, want)):
            if a != b:
                assert margins[i] < 4e-2, f"token {i} differs ({a} vs {b}) with margin {margins[i]:.2e}"
                break


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_graph_equals_eager(dtype, model_dirs):
    """300 decoded tokens cross many page edges; captured steps must give the
    tokens of eager steps."""
    from pyre_amd.api import generate

    prompts = [random_ids(777, 9, seed=1), random_ids(777, 30, seed=2), random_ids(777, 3, seed=3)]
    outs = []
    for graphs in (False, True):
        eng = _load(model_dirs["tiny-c"], dtype, use_graphs=graphs)
        outs.append(generate(eng, prompts, max_new_tokens=300, temperature=0.7, seed=11))
    assert outs[0] == outs[1]
    assert all(len(o) == 300 for o in outs[0])


def test_sampling_does_not_depend_on_batch_mates(model_dirs):
    """The tokens a request draws are a function of (seed, request, index) and its
    own logits: alone or among others, the same."""
    from pyre_amd.api import Scheduler

    eng = _load(model_dirs["tiny-b"], "float32", page_size=8)
    prompts = [random_ids(1000, n, seed=n) for n in (12, 50, 3, 77, 25, 31)]

    def run(which):
        sched = Scheduler(eng, max_batch=4, max_num_batched_tokens=48, prefill_chunk=32)
        ids = {}
        for i in range(len(prompts)):
            sid = sched.add_request(prompts[i], 24, temperature=0.8, seed=5)
            if i not in which:
                sched.waiting.pop()      # keep seq ids aligned with prompt numbers
            else:
                ids[sid] = i
        out = sched.run()
        return {ids[s]: t for s, t in out.items()}

    together = run(set(range(len(prompts))))
    for i in (0, 3, 5):
        assert run({i})[i] == together[i]
    # and temperature matters: greedy differs somewhere
    sched = Scheduler(eng)
    sid = sched.add_request(prompts[1], 24)
    assert sched.run()[sid] != together[1]


def _check_against_plain_sampler(plain, prompt, tokens, temperature, seed, seq_id, tol):
    """Every token of a generated sequence against the plain implementation, given the
    engine's own tokens before it: the plain logits of prompt + tokens[:k], the plain
    sampler with the same uniform number. A token may differ only where that number lies
    within ``tol`` of an edge of the chosen token's interval of the cumulative distribution
    (greedy: where the two largest logits are within ``tol`` of the logit scale). Returns
    how many did."""
    from pyre_amd.sampling.rng import uniform

    cfg, w = plain
    ids, near = list(prompt), 0
    for k, tok in enumerate(tokens):
        row = P.forward(w, cfg, ids)[-1]
        if temperature > 0:
            u = uniform(seed, seq_id, k)
            twin = P.sample_inverse_cdf(row, temperature, u)
            if twin != tok:
                c = torch.cumsum(torch.softmax(row.double() / temperature, -1), -1)
                lo, hi = (float(c[tok - 1]) if tok > 0 else 0.0), float(c[tok])
                margin = 0.0 if lo <= u < hi else min(abs(u - lo), abs(u - hi))
                assert margin < tol, f"token {k}: {tok} drawn, the plain sampler draws {twin}; u={u} is {margin:.2e} outside [{lo}, {hi})"
                near += 1
        else:
            twin = int(row.argmax())
            if twin != tok:
                margin = float((row[twin] - row[tok]) / row.abs().max())
                assert margin < tol, f"token {k}: {tok} chosen, plain argmax is {twin}, margin {margin:.2e}"
                near += 1
        ids.append(tok)
    return near


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_config_b_workload_against_the_plain_sampler(dtype, model_dirs, plain_models):
    """Six prompts of 3 to 120 tokens arrive one every other step, so that prompt portions
    of 32 share steps with decoding requests; temperature 0.8 with a seeded stream, 24 new
    tokens each, pages of 8 tokens. Every token is the plain sampler's on the plain logits
    with the same uniform number (`tests/test_scheduler.py:20-64` of the reference compares
    batched with alone; here both are compared with the trusted path)."""
    import random

    from pyre_amd.api import Scheduler

    plain = plain_models["tiny-b"]
    rng = random.Random(1)
    prompts = [random_ids(1000, rng.randint(3, 120), seed=10 + i) for i in range(6)]
    eng = _load(model_dirs["tiny-b"], dtype, page_size=8, max_cached_tokens=1024, prefill_chunk=32,
                max_num_batched_tokens=40)
    sched = Scheduler(eng, max_batch=4)
    ids = []
    mixed = 0
    for p in prompts:
        ids.append(sched.add_request(p, 24, temperature=0.8, seed=1))
        for _ in range(2):
            plan_before = len(sched.running)
            sched.step()
            mixed += plan_before > 0
    out = sched.run()
    assert mixed > 0 and eng.cache.page_groups[0].allocator.num_used == 0
    assert all(len(out[i]) == 24 for i in ids)
    tol = 1e-5 if dtype == "float32" else 4e-2
    near = sum(_check_against_plain_sampler(plain, p, out[i], 0.8, 1, i, tol) for p, i in zip(prompts, ids))
    assert near <= (1 if dtype == "float32" else 8), f"{near} of 144 tokens were decided by rounding"


@pytest.mark.parametrize("model,dtype,graphs", [("tiny-c", "bfloat16", True), ("tiny-c", "bfloat16", False),
                                                ("tiny-b", "float32", True), ("tiny-c", "float32", True)])
def test_many_live_requests_generate_the_plain_tokens(model, dtype, graphs, model_dirs, plain_models):
    """20, 50 and 150 requests of unequal lengths decode together (steps of 17 to 150 rows,
    padded to their captured sizes; beyond 64 rows the products are the BLAS library's), some
    greedy, some sampled; every token against the plain implementation."""
    from pyre_amd.api import Scheduler

    plain = plain_models[model]
    vocab = plain[0]["vocab_size"]
    eng = _load(model_dirs[model], dtype, use_graphs=graphs, max_num_seqs=160, max_cached_tokens=160 * 96,
                max_num_batched_tokens=512, prefill_chunk=64)
    tol = 1e-5 if dtype == "float32" else 4e-2
    for count in (20, 50, 150) if graphs and dtype == "bfloat16" else (20, 50):
        prompts = [random_ids(vocab, 3 + (11 * i) % 47, seed=count + i) for i in range(count)]
        new = [6 + (5 * i) % 9 for i in range(count)]         # they end at different steps: the batch shrinks
        sched = Scheduler(eng, max_batch=160)
        ids = [sched.add_request(p, n, temperature=0.7 if i % 3 == 0 else 0.0, seed=9) for i, (p, n) in
               enumerate(zip(prompts, new))]
        out = sched.run()
        assert eng.cache.page_groups[0].allocator.num_used == 0
        near = 0
        for i, (p, sid) in enumerate(zip(prompts, ids)):
            assert len(out[sid]) == new[i]
            near += _check_against_plain_sampler(plain, p, out[sid], 0.7 if i % 3 == 0 else 0.0, 9, sid, tol)
        assert near <= (1 if dtype == "float32" else count), f"{near} tokens were decided by rounding"
    if graphs:
        assert eng.graph_replays > 0


def test_preemption_recomputes_and_gives_the_same_tokens(model_dirs):
    """With so few pages that running requests cannot all grow, the latest one is
    preempted and recomputed; tokens equal those of a roomy pool."""
    from pyre_amd.api import Scheduler

    prompts = [random_ids(777, n, seed=n) for n in (40, 45, 38)]
    outs = []
    for pages in (64, 11):
        eng = _load(model_dirs["tiny-c"], "float32", num_pages=pages, max_cached_tokens=None)
        sched = Scheduler(eng, max_batch=4, prefill_chunk=64)
        ids = [sched.add_request(p, 40) for p in prompts]
        res = sched.run()
        outs.append([res[i] for i in ids])
        assert eng.cache.page_groups[0].allocator.num_used == 0
        if pages == 11:
            assert sum(r.preemptions for r in sched.finished.values()) > 0
    assert outs[0] == outs[1]


def test_cli_generates(model_dirs, plain_models, tmp_path, capsys):
    """The command line's tokens are the plain implementation's greedy tokens."""
    from helpers import check_greedy
    from pyre_amd.cli import main

    out = tmp_path / "res.json"
    rc = main(["--model", str(model_dirs["tiny-b"]), "--dtype", "float32", "--prompt-ids", "5,17,3",
               "--prompt-ids", "9", "--max-new-tokens", "6", "--max-batch", "4", "--num-blocks", "32",
               "--out", str(out)])
    assert rc == 0
    import json

    res = json.loads(out.read_text())
    assert res["prompts"] == [[5, 17, 3], [9]] and [len(g) for g in res["generated"]] == [6, 6]
    for prompt, tokens in zip(res["prompts"], res["generated"]):
        assert check_greedy(plain_models["tiny-b"], prompt, tokens, 1e-5) == 0
    printed = capsys.readouterr().out.splitlines()
    assert printed[0] == "request 0: prompt of 3 tokens -> " + ",".join(map(str, res["generated"][0]))


def test_the_generate_program_as_a_process(model_dirs, plain_models, tmp_path):
    """``bin/pyre_generate`` as a user starts it: a process of its own, the reference's spellings
    of the options (``--tokens``), a JSON result file; its tokens against the plain implementation."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    from helpers import check_greedy

    root = Path(__file__).resolve().parent.parent
    out = tmp_path / "res.json"
    proc = subprocess.run([sys.executable, str(root / "bin" / "pyre_generate"), "--model", str(model_dirs["tiny-c"]),
                           "--dtype", "bfloat16", "--prompt-ids", "700,3,3,41,9,100,5", "--tokens", "5",
                           "--num-blocks", "16", "--max-batch", "2", "--out", str(out)],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    res = json.loads(out.read_text())
    assert res["dtype"] == "bfloat16" and len(res["generated"][0]) == 5
    assert proc.stdout.splitlines()[0] == "request 0: prompt of 7 tokens -> " + ",".join(map(str, res["generated"][0]))
    assert check_greedy(plain_models["tiny-c"], res["prompts"][0], res["generated"][0], 4e-2) <= 1
    bad = subprocess.run([sys.executable, str(root / "bin" / "pyre_generate"), "--model", str(tmp_path / "nothing")],
                         capture_output=True, text=True, timeout=300)
    assert bad.returncode != 0 and "neither a model folder nor a preset" in bad.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_one_step_ahead_changes_no_token(dtype, model_dirs):
    """Staggered requests of different lengths, some sampled with a temperature, one
    ending early by its end-of-sequence token, on few pages: the tokens with steps put on
    the device one step ahead (tokens fed there), prompt portions and admissions among
    them, are those of a scheduler that waits for every step."""
    from pyre_amd.api import Scheduler

    eng = _load(model_dirs["tiny-c"], dtype, use_graphs=True, max_cached_tokens=640)
    vocab = eng.vocab_size
    prompts = [random_ids(vocab, n, seed=100 + n) for n in (5, 40, 17, 64, 9, 33)]
    lens = [30, 12, 44, 20, 37, 25]

    mixed_ahead = [0]
    real_step = eng.step

    def counting_step(entries, fed_ids=None):
        # a step that ran ahead (a token fed on the device) and carries a prompt portion too
        mixed_ahead[0] += any(e.feed is not None for e in entries) and any(len(e.tokens) > 1 for e in entries)
        return real_step(entries, fed_ids=fed_ids)

    eng.step = counting_step

    def run(ahead, eos):
        s = Scheduler(eng, max_batch=4)
        s.lookahead = ahead
        ids, steps = [], 0
        for i, (p, n) in enumerate(zip(prompts, lens)):
            ids.append(s.add_request(p, n, eos_id=eos if i == 2 else None, temperature=0.7 if i % 2 else 0.0, seed=i))
            s.step()                      # requests arrive while others run
            steps += 1
        out = s.run()
        assert eng.cache.page_groups[0].allocator.num_used == 0
        return [out[i] for i in ids], s

    base, _ = run(False, None)
    eos = base[2][10]                     # request 2 will now end at the first occurrence of this token
    want, s0 = run(False, eos)
    assert mixed_ahead[0] == 0
    got, s1 = run(True, eos)
    assert got == want
    assert mixed_ahead[0] >= 3            # prompts in portions of 32 rode in steps that ran ahead
    assert len(want[2]) <= 11 and want[2][-1] == eos
    assert s1.lookahead and not s0.lookahead
    # the steps that ran ahead are fewer host round trips, not fewer engine steps
    assert eng.graph_replays > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_after_steps_were_captured(dtype, model_dirs):
    """Decode steps are captured while every buffer is still small (a 3-token prompt); then a
    prompt of 200 tokens in portions of 128 makes scratch buffers grow. The captured steps go
    on using their memory: the first request's tokens are those of an engine without graphs."""
    from pyre_amd.api import Scheduler

    short, long_ = random_ids(777, 3, seed=5), random_ids(777, 200, seed=6)
    outs = []
    for graphs in (False, True):
        eng = _load(model_dirs["tiny-c"], dtype, use_graphs=graphs, prefill_chunk=128)
        s = Scheduler(eng, max_batch=4)
        a = s.add_request(short, max_new_tokens=60, temperature=0.7, seed=3)
        for _ in range(12):
            s.step()
        if graphs:
            assert eng.graph_replays > 0
        b = s.add_request(long_, max_new_tokens=20, temperature=0.7, seed=4)
        # other tensors take what the allocator has to give between the steps
        junk = [torch.full((1 << 16,), float("nan"), device="cuda:0") for _ in range(32)]
        done = s.run()
        del junk
        outs.append((done[a], done[b]))
    assert outs[0] == outs[1]
