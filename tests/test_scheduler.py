"""The scheduler's decisions (CPU), with a stand-in engine: admission, token budget,
portions, finishing, and what happens when pages run out."""

from __future__ import annotations

from dataclasses import dataclass

import pytest

from pyre_amd.cache import CacheManager
from pyre_amd.cache.allocator import OutOfPages
from pyre_amd.engine.scheduler import Scheduler
from pyre_amd.parts.base import PagedCacheSpec, PagedTensorSpec

ONE_RECORD = PagedCacheSpec((PagedTensorSpec("record", (8,)),))


@dataclass
class FakeConfig:
    max_num_seqs: int = 4
    max_num_batched_tokens: int = 64
    prefill_chunk: int = 32


class FakeEngine:
    """Keeps the real cache bookkeeping; its "logits" are the entries themselves."""

    vocab_size = 100

    def __init__(self, pages=64, page_size=16, max_len=512, **cfg):
        self.engine_config = FakeConfig(**cfg)
        self.cache = CacheManager([ONE_RECORD], page_size, pages, self.engine_config.max_num_seqs, max_len)
        self.max_model_len = max_len
        self.steps = []

    def step(self, entries):
        for e in entries:
            if e.rid not in self.cache:
                self.cache.add_request(e.rid)
        for e in entries:
            self.cache.reserve(e.rid, len(e.tokens))
        for e in entries:
            self.cache.commit(e.rid, len(e.tokens))
        self.cache.check_invariants()
        self.steps.append([(e.rid, len(e.tokens), list(e.want)) for e in entries])
        return [e for e in entries if e.want]

    def finish(self, rid):
        self.cache.free_request(rid)


class FakeSampler:
    """Next token = (sum of the request's tokens so far) mod vocabulary: a function of
    the request alone, like a real model's greedy choice."""

    def __init__(self, sched):
        self.sched = sched

    def sample(self, rows, temps, us):
        out = []
        for e in rows:
            r = next(x for x in self.sched.running if x.seq_id == e.rid)
            out.append(sum(r.tokens) % 100)
        return out


def make(**kw):
    eng = FakeEngine(**kw)
    s = Scheduler(eng)
    s.sampler = FakeSampler(s)
    return eng, s


def expected(prompt, n, eos=None):
    toks, out = list(prompt), []
    for _ in range(n):
        t = sum(toks) % 100
        toks.append(t)
        out.append(t)
        if eos is not None and t == eos:
            break
    return out


def test_portions_under_the_budget_and_decodes_first():
    eng, s = make()
    a = s.add_request(list(range(1, 71)), 5)                 # 70 tokens: 32 + 32 + 6
    s.step()
    assert eng.steps[-1] == [(a, 32, [])]
    b = s.add_request([7] * 10, 5)
    s.step()                                                 # a's second portion, then b whole
    assert eng.steps[-1] == [(a, 32, []), (b, 10, [9])]
    s.step()                                                 # oldest first: a's last portion, then b's decoded token
    assert eng.steps[-1] == [(a, 6, [5]), (b, 1, [0])]
    s.step()
    assert eng.steps[-1] == [(a, 1, [0]), (b, 1, [0])]
    out = s.run()
    assert out[a] == expected(range(1, 71), 5) and out[b] == expected([7] * 10, 5)
    assert eng.cache.page_groups[0].allocator.num_used == 0 and not s.has_work


def test_budget_caps_a_step():
    eng, s = make(max_num_batched_tokens=40)
    for _ in range(3):
        s.add_request([1] * 30, 2)
    s.step()
    assert [n for _, n, _ in eng.steps[-1]] == [30, 10]       # the second prompt is cut by the budget
    s.step()
    assert sum(n for _, n, _ in eng.steps[-1]) <= 40
    s.run()


def test_max_batch_and_first_come_first_served():
    eng, s = make(max_num_seqs=2)
    ids = [s.add_request([i + 1] * 4, 3) for i in range(4)]
    s.step()
    assert [r for r, _, _ in eng.steps[-1]] == ids[:2]
    out = s.run()
    assert list(out) == ids and all(len(v) == 3 for v in out.values())
    assert max(len(st) for st in eng.steps) == 2


def test_finishing_by_length_and_by_eos():
    eng, s = make()
    p = [3, 4]
    toks = expected(p, 6)
    a = s.add_request(p, 6, eos_id=toks[2])
    b = s.add_request(p, 6, eos_id=toks[2], ignore_eos=True)
    c = s.add_request(p, 1)                                   # one new token means one (pyre/scheduler.py:84 gives two)
    out = s.run()
    assert out[a] == toks[:3] and s.finished[a].finish_reason == "eos"
    assert out[b] == toks and s.finished[b].finish_reason == "length"
    assert out[c] == toks[:1]
    assert [n for st in eng.steps for r, n, _ in st if r == c] == [2]   # a finished request never enters a step again


def test_requests_that_can_never_run_are_refused():
    eng, s = make(pages=4, max_len=512)
    with pytest.raises(ValueError, match="could never run"):
        s.add_request([1] * 60, 10)                           # 69 cached tokens = 5 pages > 4
    s.add_request([1] * 55, 10)                               # 64 cached tokens = 4 pages: fits alone
    with pytest.raises(ValueError, match="longest request"):
        s.add_request([1] * 500, 20)
    with pytest.raises(ValueError, match="vocabulary"):
        s.add_request([100], 2)
    with pytest.raises(ValueError, match="at least one"):
        s.add_request([], 2)
    assert len(s.run()) == 1


def test_no_admission_without_pages():
    eng, s = make(pages=6)
    a = s.add_request([1] * 60, 4)                            # 4 pages
    b = s.add_request([2] * 40, 4)                            # 3 pages: does not fit beside a
    while s.running or not s.finished:
        s.step()
        if a in s.finished:
            break
        assert all(r == a for r, _, _ in eng.steps[-1])
    out = s.run()
    assert out[a] == expected([1] * 60, 4) and out[b] == expected([2] * 40, 4)
    assert s.finished[b].preemptions == 0


def test_preemption_takes_the_latest_and_recomputes():
    """Two requests fit at admission but not when both grow: the one admitted last
    goes back to the front of the queue, keeps its tokens, and is recomputed."""
    eng, s = make(pages=5, max_num_seqs=4)
    a = s.add_request([1] * 30, 40)                           # grows to 69 cached tokens: 5 pages alone
    b = s.add_request([2] * 14, 40)
    c = s.add_request([3] * 5, 3)
    out = s.run()
    assert out[a] == expected([1] * 30, 40) and out[b] == expected([2] * 14, 40) and out[c] == expected([3] * 5, 3)
    assert s.finished[a].preemptions == 0 and s.finished[b].preemptions >= 1
    # after a preemption the victim's next entry starts from position 0 again and covers prompt + generated
    first_again = [st for st in eng.steps if any(r == b and n > 1 for r, n, _ in st)]
    assert len(first_again) >= 2
    assert eng.cache.page_groups[0].allocator.num_used == 0 and eng.cache.slots.num_used == 0


def test_batched_equals_alone():
    """tests/test_scheduler.py:20-64 of the reference: caps 24/16/32, different prompts."""
    prompts = {0: [5] * 9, 1: [8, 1, 4], 2: list(range(20))}
    caps = {0: 24, 1: 16, 2: 32}
    eng, s = make(pages=32)
    ids = {s.add_request(prompts[i], caps[i]): i for i in prompts}
    together = {ids[k]: v for k, v in s.run().items()}
    for i in prompts:
        e2, s2 = make(pages=32)
        sid = s2.add_request(prompts[i], caps[i])
        assert s2.run()[sid] == together[i]
    assert not s.running and not s.waiting


# ---------------------------------------------------------------------------
# Running one step ahead: the next decode step goes to the engine before this
# step's tokens are read; its tokens come from the sampler's ids "on the device".
# ---------------------------------------------------------------------------
class AheadEngine(FakeEngine):
    accepts_fed_ids = True

    def __init__(self, **kw):
        super().__init__(**kw)
        self.fed = {}  #: rid -> every token the engine has been given for it, in order
        self.ahead_steps = 0
        self.mixed_ahead_steps = 0  #: of them, steps that also carry tokens the host knows (prompt portions)

    def step(self, entries, fed_ids=None):
        for e in entries:
            toks = [fed_ids[e.feed]] if e.feed is not None else list(e.tokens)
            self.fed.setdefault(e.rid, []).extend(toks)
        self.ahead_steps += any(e.feed is not None for e in entries)
        self.mixed_ahead_steps += any(e.feed is not None for e in entries) and any(e.feed is None for e in entries)
        return super().step(entries)


class AheadSampler(FakeSampler):
    """``ids`` stands for the ids on the device: written at launch, read by the engine
    when a step that ran ahead is fed from them."""

    ids = ()

    def launch(self, rows, temps, us):
        running = {r.seq_id: r for r in self.sched.running}
        # a request that has ended has a surplus row in a step that ran ahead: any id will do
        self.ids = [sum(running[e.rid].tokens) % 100 if e.rid in running else -1 for e in rows]
        return list(self.ids)

    def collect(self, handle):
        return handle


@pytest.mark.parametrize("eos", [None, 37])
def test_running_ahead_gives_the_same_tokens(eos):
    prompts = [[1, 2, 3], [7] * 20, [5, 9], [4, 4, 4, 4, 11]]
    lens = [9, 17, 30, 12]

    def run(ahead):
        eng = AheadEngine(pages=64, max_num_seqs=4)
        s = Scheduler(eng)
        s.sampler = AheadSampler(s)
        s.lookahead = ahead
        ids = [s.add_request(p, n, eos_id=eos) for p, n in zip(prompts, lens)]
        out = s.run()
        eng.cache.check_invariants()
        assert eng.cache.free_pages() == 64
        return eng, s, [out[i] for i in ids]

    eng0, _, plain = run(False)
    eng1, s1, ahead = run(True)
    assert ahead == plain == [expected(p, n, eos) for p, n in zip(prompts, lens)]
    assert eng0.ahead_steps == 0 and eng1.ahead_steps > 10
    # every request was fed exactly its prompt and the tokens it generated, bar the last one,
    # plus at most one surplus token after an end-of-sequence token
    for rid, (p, g) in enumerate(zip(prompts, ahead)):
        want = p + g[:-1]
        assert eng1.fed[rid][:len(want)] == want and len(eng1.fed[rid]) <= len(want) + 1


def test_a_request_added_meanwhile_waits_one_step():
    eng = AheadEngine(pages=64, max_num_seqs=4)
    s = Scheduler(eng)
    s.sampler = AheadSampler(s)
    s.lookahead = True
    a = s.add_request([1, 2, 3], 8)
    s.step(), s.step()                      # the second step has put a third one on the device
    b = s.add_request([9, 9], 4)
    s.step()                                # consumes the step that ran ahead, without b; the next one has it
    assert len(eng.steps) == 4
    assert b not in [rid for rid, _, _ in eng.steps[2]] and b in [rid for rid, _, _ in eng.steps[3]]
    out = s.run()
    assert out[a] == expected([1, 2, 3], 8) and out[b] == expected([9, 9], 4)


def test_running_ahead_while_others_wait_for_a_free_place():
    """With as many running as may run, nobody can be admitted next step, so the steps run
    ahead although requests wait; when one reaches its length, the next step is planned
    as usual and admits the first of them."""
    prompts = [[i + 1, i + 2] for i in range(6)]
    lens = [12, 7, 9, 12, 5, 6]

    def run(ahead):
        eng = AheadEngine(pages=64, max_num_seqs=2)
        s = Scheduler(eng)
        s.sampler = AheadSampler(s)
        s.lookahead = ahead
        ids = [s.add_request(p, n) for p, n in zip(prompts, lens)]
        out = s.run()
        assert eng.cache.free_pages() == 64
        return eng, [out[i] for i in ids]

    eng0, plain = run(False)
    eng1, ahead = run(True)
    assert ahead == plain == [expected(p, n) for p, n in zip(prompts, lens)]
    assert eng1.ahead_steps > 15
    # the order of admission is first come, first served in both
    first_seen = lambda eng: [rid for step in eng.steps for rid, _, _ in step if not any(rid == r for st in eng.steps[:eng.steps.index(step)] for r, _, _ in st)]  # noqa: E731
    assert first_seen(eng1) == first_seen(eng0) == list(range(6))


def test_steps_with_prompt_portions_run_ahead_too():
    """Long prompts arrive while others decode: the steps that carry their portions, and the
    steps that admit them, are put on the device before the tokens of the step before are
    read; the tokens are those of a run that waits for every step."""
    prompts = [[3, 1], [2] * 70, [9, 8, 7], [5] * 90, [6] * 40]
    lens = [40, 10, 25, 6, 12]

    def run(ahead):
        eng = AheadEngine(pages=64, max_num_seqs=3, max_num_batched_tokens=24, prefill_chunk=16)
        s = Scheduler(eng)
        s.sampler = AheadSampler(s)
        s.lookahead = ahead
        ids = [s.add_request(p, n) for p, n in zip(prompts, lens)]
        out = s.run()
        eng.cache.check_invariants()
        assert eng.cache.free_pages() == 64
        return eng, [out[i] for i in ids]

    eng0, plain = run(False)
    eng1, ahead = run(True)
    assert ahead == plain == [expected(p, n) for p, n in zip(prompts, lens)]
    assert eng1.mixed_ahead_steps >= 10
    for step in eng1.steps:   # the budget and the number of requests hold in steps that ran ahead as well
        assert sum(n for _, n, _ in step) <= 24 and len(step) <= 3
    for rid, (p, g) in enumerate(zip(prompts, ahead)):
        assert eng1.fed[rid] == p + g[:-1]   # no end token here: nothing surplus


class FailingAheadEngine(AheadEngine):
    """Refuses the steps that run ahead whose number is in ``fail_on`` (before it touches the
    cache, as the real engine's all-or-nothing preparation does)."""

    def __init__(self, fail_on, error, **kw):
        super().__init__(**kw)
        self.fail_on, self.error, self.ahead_calls, self.refused = set(fail_on), error, 0, 0

    def step(self, entries, fed_ids=None):
        if fed_ids is not None:
            self.ahead_calls += 1
            if self.ahead_calls in self.fail_on:
                self.refused += 1
                raise self.error("the step that ran ahead is refused")
        return super().step(entries, fed_ids)


@pytest.mark.parametrize("error", [OutOfPages, ValueError])
def test_a_refused_step_ahead_costs_no_token(error):
    """If the engine refuses the step that was to run ahead, this step's tokens are still
    collected, the requests that the refused step had admitted wait again in their order, and
    the next step is planned as usual: the same tokens as without running ahead."""
    prompts = [[3, 1], [2] * 70, [9, 8, 7], [5] * 90, [6] * 40, [1, 2, 3, 4]]
    lens = [40, 10, 25, 6, 12, 9]

    def run(fail_on):
        eng = FailingAheadEngine(fail_on, error, pages=64, max_num_seqs=3, max_num_batched_tokens=24, prefill_chunk=16)
        s = Scheduler(eng)
        s.sampler = AheadSampler(s)
        s.lookahead = True
        ids = [s.add_request(p, n) for p, n in zip(prompts, lens)]
        out = s.run()
        eng.cache.check_invariants()
        assert eng.cache.free_pages() == 64 and eng.cache.slots.num_used == 0
        return eng, [out[i] for i in ids]

    eng0, plain = run(())
    eng1, got = run({1, 2, 5, 11, 12, 30})
    assert eng1.refused == 6 and eng1.ahead_steps > 10
    assert got == plain == [expected(p, n) for p, n in zip(prompts, lens)]
    first_seen = lambda eng: list(dict.fromkeys(rid for step in eng.steps for rid, _, _ in step))  # noqa: E731
    assert first_seen(eng1) == first_seen(eng0) == list(range(6))      # first come, first served all the same


def test_finished_requests_are_handed_over_and_forgotten():
    eng, s = make(pages=64, max_num_seqs=4)
    a = s.add_request([1, 2, 3], 4)
    b = s.add_request([9] * 20, 2)
    out = s.run()
    assert out == {a: expected([1, 2, 3], 4), b: expected([9] * 20, 2)}
    taken = s.take_finished()
    assert sorted(taken) == [a, b] and taken[a].finish_reason == "length" and not s.finished
    assert s.take_finished() == {}
    # a stream driven by step() whose caller never asks: the oldest are dropped beyond the cap
    s.max_finished_kept = 3
    ids = [s.add_request([i + 1], 1) for i in range(8)]
    results = s.run()
    assert sorted(results) == ids                                       # run() hands every result over all the same
    assert list(s.finished) == ids[-3:]


@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("ahead", [False, True])
def test_random_workloads_give_every_request_its_own_tokens(seed, ahead):
    """Random prompts, lengths and end tokens, requests arriving while others run, a pool
    so small that requests are preempted and recomputed: every request's tokens are a
    function of its prompt alone, nothing is left in the cache, and with steps running
    ahead nothing changes."""
    import random

    rng = random.Random(seed)
    eng = AheadEngine(pages=rng.choice([6, 8, 12, 40]), page_size=8, max_len=96, max_num_seqs=rng.choice([2, 3, 4]),
                      max_num_batched_tokens=rng.choice([16, 24, 64]), prefill_chunk=rng.choice([5, 16, 32]))
    s = Scheduler(eng)
    s.sampler = AheadSampler(s)
    s.lookahead = ahead
    todo = []
    for _ in range(rng.randint(5, 14)):
        n = rng.randint(1, 30)
        prompt = [rng.randrange(100) for _ in range(n)]
        new = rng.randint(1, min(40, 96 - n))
        if eng.cache.pages_needed(None, n + new - 1) > eng.cache.page_groups[0].num_pages:
            continue  # could never run: refused at add_request, tested elsewhere
        todo.append((prompt, new, rng.choice([None, None, rng.randrange(100)])))
    ids, want = [], []
    while todo or s.has_work:
        while todo and rng.random() < 0.5:
            p, new, eos = todo.pop(0)
            ids.append(s.add_request(p, new, eos_id=eos))
            want.append(expected(p, new, eos))
        if s.has_work:
            s.step()
            eng.cache.check_invariants()
    out = s.finished
    assert [out[i].generated for i in ids] == want
    assert eng.cache.free_pages() == eng.cache.page_groups[0].num_pages and eng.cache.slots.num_used == 0
