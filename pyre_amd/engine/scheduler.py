"""Continuous batching above the step function (`pyre/scheduler.py:13-114`).

Each call of :meth:`Scheduler.step` plans one batch under a token budget, runs it
through the engine, samples one token for every request whose last known token was
in the batch, finishes what is done and frees its pages. The reference prefills a
whole prompt alone at admission and then decodes all running requests
(`pyre/scheduler.py:46-97`); here portions of prompts ride in the same step as the
decoded tokens of the others.

When pages run out: a request is admitted only if the pages for all the tokens it
has so far (its prompt, and what it generated before a preemption) are free beside
those that running prompts are still going to take, with one page to spare for
every running request; if a running request needs a page and none is free, the request admitted
last is preempted: its pages and slot are given back and it re-enters the front
of the waiting queue to be recomputed from its prompt and the tokens it has
generated so far (which it keeps). A request that could not fit the pool even
alone is refused when it is added. (The reference lets ``MemoryError`` escape,
`pyre/paged_cache.py:58-67`.)

Where it can, the next step is put on the device before the host has seen this step's
tokens: it is planned as if every request that this step samples for had one more token
(those that reach their length aside, which are left out), and those tokens are fed on the
device from the sampler's ids. The host then reads this step's tokens while the next step
runs, and the device does not wait while the host plans. Portions of prompts and newly
admitted requests ride in such a step like in any other; a place or pages that become free
with this step's results are seen one step later. A request that turns out to have ended
(its end-of-sequence token) has one surplus row in that next step, which is ignored. If
the next step would have to preempt somebody it is planned with the tokens known, as
usual. This needs an engine whose ``step`` takes ``fed_ids`` and a sampler with
``launch``/``collect``/``ids``; with others every step waits for its tokens as before.

This module needs neither torch nor a GPU: the engine and the sampler are passed in.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from pyre_amd.engine.batch import Entry
from pyre_amd.sampling.params import SamplingParams
from pyre_amd.sampling.rng import uniform


@dataclass(eq=False)
class Request:
    seq_id: int
    prompt_ids: list[int]
    params: SamplingParams
    generated: list[int] = field(default_factory=list)
    num_computed: int = 0            #: tokens of prompt + generated that are in the cache
    finish_reason: str | None = None  #: "eos" | "length"
    preemptions: int = 0
    #: while the next step is planned ahead of this step's tokens: one token more that is
    #: on the device only / the request reaches its length with that token
    pending: int = 0
    ending: bool = False

    @property
    def tokens(self) -> list[int]:
        return self.prompt_ids + self.generated

    def token_slice(self, start: int, count: int) -> list[int]:
        """``tokens[start:start + count]`` without joining the two lists."""
        n = len(self.prompt_ids)
        if start >= n:
            return self.generated[start - n:start - n + count]
        if start + count <= n:
            return self.prompt_ids[start:start + count]
        return self.prompt_ids[start:] + self.generated[:start + count - n]

    @property
    def cur_len(self) -> int:        # pyre/scheduler.py:22-24
        return len(self.prompt_ids) + len(self.generated) + self.pending

    @property
    def done(self) -> bool:
        return self.finish_reason is not None


@dataclass
class PlannedEntry:
    request: Request
    start: int                       #: first token of the portion (index into request.tokens)
    count: int
    samples: bool                    #: the portion ends with the last known token


@dataclass
class StepPlan:
    entries: list[PlannedEntry]
    preempted: list[Request]
    admitted: list[Request]

    @property
    def num_tokens(self) -> int:
        return sum(e.count for e in self.entries)


class Scheduler:
    def __init__(self, engine, max_batch: int | None = None, max_num_batched_tokens: int | None = None,
                 prefill_chunk: int | None = None, sampler=None):
        """``engine`` provides ``cache``, ``step``, ``finish``, ``vocab_size``,
        ``max_model_len`` and ``engine_config``; ``max_batch`` (the reference's name,
        `pyre/scheduler.py:28`) bounds the requests that run at a time."""
        ec = engine.engine_config
        self.engine = engine
        self.cache = engine.cache
        self.max_batch = min(max_batch or ec.max_num_seqs, ec.max_num_seqs)
        self.token_budget = min(max_num_batched_tokens or ec.max_num_batched_tokens, ec.max_num_batched_tokens)
        self.prefill_chunk = prefill_chunk or ec.prefill_chunk
        self.sampler = sampler
        self.waiting: list[Request] = []
        self.running: list[Request] = []
        #: finished requests that nobody has taken yet (:meth:`take_finished`), the oldest first;
        #: at most ``max_finished_kept`` of them, so that a stream driven by ``step()`` whose
        #: caller reads the tokens that ``step`` returns and never comes here does not grow
        self.finished: dict[int, Request] = {}
        self.max_finished_kept = 4096
        self.last_finished: list[Request] = []  #: the requests that the last step finished
        self._next_seq = 0
        self.steps = 0
        #: put the next decode step on the device before this step's tokens are read
        self.lookahead = bool(getattr(engine, "accepts_fed_ids", False)) and all(
            hasattr(sampler, a) for a in ("launch", "collect", "ids"))
        self._ahead: tuple[StepPlan, object] | None = None  #: (plan, logits) of a step already on the device

    # ------------------------------------------------------------------ requests

    def add_request(self, prompt_ids, max_new_tokens: int = 16, eos_id: int | None = None,
                    temperature: float = 0.0, seed: int = 0, ignore_eos: bool = False) -> int:
        prompt = [int(t) for t in prompt_ids]
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        for t in prompt:
            if not (0 <= t < self.engine.vocab_size):
                raise ValueError(f"token id {t} is outside the vocabulary (0..{self.engine.vocab_size - 1})")
        params = SamplingParams(max_new_tokens, temperature, eos_id, ignore_eos, seed)
        total = len(prompt) + max_new_tokens
        if total > self.engine.max_model_len:
            raise ValueError(f"prompt ({len(prompt)}) + max_new_tokens ({max_new_tokens}) exceeds "
                             f"the engine's longest request ({self.engine.max_model_len})")
        # The last generated token is never fed back, so total - 1 tokens are cached.
        need = self.cache.pages_needed(None, total - 1)
        for g in self.cache.page_groups:
            if need > g.num_pages:
                raise ValueError(f"request needs {need} pages, the pool has {g.num_pages}: it could never run")
        r = Request(self._next_seq, prompt, params)
        self._next_seq += 1
        self.waiting.append(r)
        return r.seq_id

    @property
    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ planning

    def plan(self, ahead: bool = False) -> StepPlan | None:
        """Decide the next batch. Changes queue membership (admission, preemption)
        and frees preempted requests' pages; reserves nothing. ``ahead``: requests marked
        ``ending`` are left out, and None is returned, with nothing changed, if somebody
        would have to be preempted."""
        budget = self.token_budget
        free = self.cache.free_pages()
        entries: list[PlannedEntry] = []
        preempted: list[Request] = []
        admitted: list[Request] = []

        def portion(r: Request, budget: int) -> int:
            return min(r.cur_len - r.num_computed, self.prefill_chunk, budget)

        # 1. running requests, oldest first: decoded tokens and prompt portions
        i = 0
        while i < len(self.running) and budget > 0:
            r = self.running[i]
            if ahead and r.ending:
                i += 1
                continue
            n = portion(r, budget)
            need = self.cache.pages_needed(r.seq_id, n)
            if ahead and need > free:
                return None
            while need > free:
                victim = self.running[-1]
                if victim is r and len(self.running) == 1:
                    raise RuntimeError(f"request {r.seq_id} cannot get {need} pages even alone")
                self._preempt(victim)
                preempted.append(victim)
                # entries already planned for the victim (it was later in the list) cannot exist:
                # victims are taken from the back, planning runs from the front.
                free = self.cache.free_pages() - sum(self.cache.pages_needed(e.request.seq_id, e.count) for e in entries)
                if victim is r:
                    break
            if r not in self.running:
                continue  # r itself was the last one admitted and went back to waiting
            entries.append(PlannedEntry(r, r.num_computed, n, r.num_computed + n == r.cur_len))
            free -= need
            budget -= n
            i += 1

        # 2. admit waiting requests, first come first served (pyre/scheduler.py:49-50)
        # Pages that running prompts will still take in later steps are spoken for.
        promised = None
        while (self.waiting and not preempted and budget > 0 and len(self.running) < self.max_batch
               and self.cache.has_free_slot()):
            if promised is None:  # worked out only when somebody waits and could be let in
                planned = {e.request.seq_id: e.count for e in entries}
                promised = sum(
                    self.cache.pages_needed(r.seq_id, r.cur_len - r.num_computed)
                    - self.cache.pages_needed(r.seq_id, planned.get(r.seq_id, 0)) for r in self.running)
            r = self.waiting[0]
            n = portion(r, budget)
            need_now = self.cache.pages_needed(None, n)
            need_all = self.cache.pages_needed(None, r.cur_len)
            # One page of headroom for every running request, so that an admission
            # is not undone by the very next decoded token.
            if need_all + promised + len(self.running) > free:
                break
            self.waiting.pop(0)
            self.running.append(r)
            self.cache.add_request(r.seq_id)
            admitted.append(r)
            entries.append(PlannedEntry(r, 0, n, n == r.cur_len))
            free -= need_now
            promised += need_all - need_now
            budget -= n
        return StepPlan(entries, preempted, admitted)

    def _preempt(self, r: Request) -> None:
        self.running.remove(r)
        self.engine.finish(r.seq_id)
        r.num_computed = 0
        r.preemptions += 1
        self.waiting.insert(0, r)

    # ------------------------------------------------------------------ running

    def step(self) -> list[tuple[int, int]]:
        """Plan, run and sample one batch; returns (seq_id, new token) pairs."""
        self.last_finished = []
        ahead, self._ahead = self._ahead, None
        if ahead is not None and all(e.request.done for e in ahead[0].entries):
            ahead = None  # every request of the step that ran ahead has ended meanwhile
        if ahead is not None:
            plan, logits = ahead
        else:
            plan = self.plan()
            if not plan.entries:
                if self.has_work:
                    raise RuntimeError("scheduler made no progress (no request fits the pool or the budget)")
                return []
            entries = [Entry(e.request.seq_id, e.request.token_slice(e.start, e.count),
                             [e.count - 1] if e.samples else []) for e in plan.entries]
            logits = self.engine.step(entries)
        self.steps += 1
        for e in plan.entries:
            e.request.num_computed += e.count
        sampling = [e.request for e in plan.entries if e.samples]
        out: list[tuple[int, int]] = []
        if sampling:
            temps = [r.params.temperature for r in sampling]
            us = [uniform(r.params.seed, r.seq_id, len(r.generated)) if r.params.temperature > 0 else 0.0
                  for r in sampling]
            if self.lookahead:
                handle = self.sampler.launch(logits, temps, us)
                self._ahead = self._run_ahead(sampling)
                new = self.sampler.collect(handle)
            else:
                new = self.sampler.sample(logits, temps, us)
            for r, tok in zip(sampling, new):
                if r.done:
                    continue  # a surplus row of a step that ran ahead
                tok = int(tok)
                r.generated.append(tok)
                out.append((r.seq_id, tok))
                p = r.params
                if p.eos_id is not None and tok == p.eos_id and not p.ignore_eos:
                    r.finish_reason = "eos"
                elif len(r.generated) >= p.max_new_tokens:
                    r.finish_reason = "length"
        self.last_finished = [r for r in self.running if r.done]
        for r in self.last_finished:
            self.running.remove(r)
            self.engine.finish(r.seq_id)
            self.finished[r.seq_id] = r
        while len(self.finished) > self.max_finished_kept:
            del self.finished[next(iter(self.finished))]
        return out

    def take_finished(self) -> dict[int, Request]:
        """The requests that have finished since the last call, which the scheduler then forgets."""
        done, self.finished = self.finished, {}
        return done

    def _run_ahead(self, sampling: list[Request]):
        """Plan the next step without this step's tokens and put it on the device. Returns
        (plan, logits) or None. The sampler's ids of this step must already be on the stream."""
        feed = {}
        marked = []
        for i, r in enumerate(sampling):
            if r.done:
                continue  # a surplus row of the step before
            marked.append(r)
            if len(r.generated) + 1 >= r.params.max_new_tokens:
                r.ending = True
            else:
                r.pending = 1
                feed[r.seq_id] = i
        try:
            nxt = self.plan(ahead=True)
            if nxt is None or not nxt.entries:
                return None
            entries = []
            for e in nxt.entries:
                r = e.request
                if r.pending and e.start + e.count == r.cur_len:
                    assert e.count == 1, "a request that was sampled for has all but one token in the cache"
                    entries.append(Entry(r.seq_id, [0], [0], feed=feed[r.seq_id]))
                else:
                    entries.append(Entry(r.seq_id, r.token_slice(e.start, e.count), [e.count - 1] if e.samples else []))
        finally:
            for r in marked:
                r.pending, r.ending = 0, False
        try:
            logits = self.engine.step(entries, fed_ids=self.sampler.ids)
        except (MemoryError, ValueError):
            # The engine's step is all or nothing: the cache is as it was. The step that was to
            # run ahead is given up (its admissions taken back); this step's tokens are
            # collected as usual and the next step is planned with them.
            for r in reversed(nxt.admitted):
                self.running.remove(r)
                if r.seq_id in self.cache:
                    self.engine.finish(r.seq_id)
                self.waiting.insert(0, r)
            return None
        return nxt, logits

    def run(self) -> dict[int, list[int]]:
        """Run until every request is finished: {seq_id: generated tokens} of the requests that
        finished meanwhile (`pyre/scheduler.py:105-114`). They stay in ``finished`` until
        :meth:`take_finished` (or the cap) removes them."""
        results: dict[int, list[int]] = {sid: r.generated for sid, r in self.finished.items()}
        while self.has_work:
            self.step()
            results.update((r.seq_id, r.generated) for r in self.last_finished)
        return dict(sorted(results.items()))
