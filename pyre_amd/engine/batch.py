"""A step's batch as flat arrays.

A step is a list of entries ``(request, its next tokens, which of them want
logits)``: portions of prompts beside single decoded tokens, in any mix
(`pyre/model.py:251-294` runs one request with any number of tokens, `:297-342`
many requests with one token each; here both are one call). The arrays below
are everything the kernels need; they are packed into one int32 buffer so that a
step costs one host-to-device copy.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

#: sizes (requests) at which decode steps are captured in HIP graphs: up to 64 rows the
#: weight-streaming products' own sizes, beyond that the BLAS library's products
DECODE_ROW_BUCKETS = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256)
MIN_TABLE_WIDTH = 8


def round_decode_shape(n_rows: int, n_pages: int) -> tuple[int, int]:
    """The fixed sizes at which a step's single-token requests are run: the number of
    requests rounded up to a bucket (beyond the largest bucket: as it is), the block
    table's width to a power of two of pages. A captured step is replayed at these
    sizes, and whoever chooses a launch shape that changes the order of a sum (how the
    keys of a request are split) chooses it from these, so that an eager step and a
    replayed one give the same bits. This function is the only place that rounds."""
    rows = next((b for b in DECODE_ROW_BUCKETS if b >= n_rows), n_rows)
    width = max(MIN_TABLE_WIDTH, 1 << (max(1, n_pages) - 1).bit_length())
    return rows, width


@dataclass
class Entry:
    rid: object
    tokens: list[int]
    want: list[int] = field(default_factory=list)  #: indices into ``tokens``
    #: the entry's single token is row ``feed`` of the ids that the caller hands to the
    #: step on the device (a result that the host has not waited for); ``tokens`` is then
    #: a placeholder of length one
    feed: int | None = None


@dataclass
class HostBatch:
    """Host-side description of one step (numpy int32 arrays)."""

    n_tokens: int
    n_seqs: int
    rids: list
    tokens: np.ndarray          #: [N]
    positions: np.ndarray       #: [N] absolute position of each token
    seq_of_token: np.ndarray    #: [N] row of the step's block tables
    q_start: np.ndarray         #: [S + 1] first token of each request's run
    ctx_len: np.ndarray         #: [S] keys each request has after this step
    state_slots: np.ndarray     #: [S] the request's state slot
    logit_rows: np.ndarray      #: [M] token indices whose logits are wanted, in entry order
    slots: list[np.ndarray]     #: per page group [N]: cache slot of each token
    tables: list[np.ndarray]    #: per page group [S, P]: block tables (-1: released or unused)
    page_size: int = 0
    max_q_len: int = 0
    n_single: int = 0                  #: requests that bring one token
    max_single_ctx: int = 0            #: longest context among them
    token_src: np.ndarray = None       #: [N] row of the device-side ids that a token comes from, or -1
    #: what the parts asked for beside the above (:class:`~pyre_amd.parts.base.StepArraySpec`)
    arrays: dict = field(default_factory=dict)

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1

    @property
    def feeds(self) -> bool:
        return self.token_src is not None and bool((self.token_src >= 0).any())

    def decode_shape(self) -> tuple[int, int]:
        """(requests, context in tokens) at which the single-token requests are to be
        launched: their number and longest context, rounded by :func:`round_decode_shape`."""
        ps = max(1, self.page_size)
        rows, width = round_decode_shape(self.n_single, -(-self.max_single_ctx // ps))
        return rows, width * ps

    def attach(self, specs) -> "HostBatch":
        """Build the arrays that the parts asked for, in the order given: a later one may
        be made from an earlier one."""
        self.arrays = {}
        for s in specs:
            self.arrays[s.name] = np.ascontiguousarray(s.build(self), dtype=np.int32)
        return self


def build_host_batch(entries: list[Entry], cache, vocab_size: int, table_width: int | None = None) -> HostBatch:
    """Lay the entries out in the order given. ``cache`` is the
    :class:`~pyre_amd.cache.CacheManager`; every request must already have its
    pages reserved for this step."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    n_seqs = len(entries)
    seen = set()
    tokens: list[int] = []
    token_src: list[int] = []
    q_start = [0]
    starts: list[int] = []
    state_slots: list[int] = []
    logit_rows: list[int] = []
    n_groups = len(cache.page_groups)
    ps = cache.page_size
    width = table_width or cache.max_pages_per_seq
    tables = [np.full((n_seqs, width), -1, dtype=np.int32) for _ in range(n_groups)]
    max_q = 0
    for s, e in enumerate(entries):
        if e.rid in seen:
            raise ValueError(f"request {e.rid!r} appears twice in one step")
        seen.add(e.rid)
        n = len(e.tokens)
        if n == 0:
            raise ValueError(f"request {e.rid!r} brings no tokens")
        if e.feed is not None and n != 1:
            raise ValueError(f"request {e.rid!r}: only a single token can come from the device")
        base = len(tokens)
        tokens.extend(e.tokens)
        token_src.extend([-1] * n if e.feed is None else [int(e.feed)])
        q_start.append(base + n)
        starts.append(cache.length(e.rid))
        state_slots.append(cache.slot(e.rid))
        for w in e.want:
            if not (0 <= int(w) < n):
                raise ValueError(f"request {e.rid!r}: wanted place {w} is outside its {n} tokens")
            logit_rows.append(base + int(w))
        for g in range(n_groups):
            have = len(cache.block_table(e.rid, g))
            if have > width:
                raise ValueError(f"request {e.rid!r} has {have} pages, the table holds {width}")
            tables[g][s, :have] = cache.block_table_array(e.rid, g)[:have]
        max_q = max(max_q, n)
    n_tokens = len(tokens)
    i32 = lambda x: np.asarray(x, dtype=np.int32)  # noqa: E731
    tok = np.asarray(tokens, dtype=np.int64)
    if tok.min() < 0 or tok.max() >= vocab_size:
        bad = next((e.rid, t) for e in entries for t in e.tokens if not (0 <= int(t) < vocab_size))
        raise ValueError(f"token id {bad[1]} of request {bad[0]!r} is outside the vocabulary (0..{vocab_size - 1})")
    q_start_a, starts_a = i32(q_start), i32(starts)
    counts = q_start_a[1:] - q_start_a[:-1]
    seq_of_token = np.repeat(np.arange(n_seqs, dtype=np.int32), counts)
    # position of a token = its request's length before the step + its index within the run
    positions = (starts_a - q_start_a[:-1])[seq_of_token] + np.arange(n_tokens, dtype=np.int32)
    ctx_len = starts_a + counts
    slots = []
    for g in range(n_groups):
        pages = tables[g][seq_of_token, positions // ps]
        if (pages < 0).any():
            t = int(np.argmax(pages < 0))
            raise RuntimeError(f"position {int(positions[t])} of request {entries[int(seq_of_token[t])].rid!r} "
                               "lies in a released page")
        slots.append((pages * ps + positions % ps).astype(np.int32))
    single = counts == 1
    return HostBatch(
        page_size=ps, n_single=int(single.sum()), max_single_ctx=int(ctx_len[single].max()) if single.any() else 0,
        n_tokens=n_tokens, n_seqs=n_seqs, rids=[e.rid for e in entries], tokens=tok.astype(np.int32),
        positions=positions.astype(np.int32), seq_of_token=seq_of_token, q_start=q_start_a,
        ctx_len=ctx_len.astype(np.int32), state_slots=i32(state_slots), logit_rows=i32(logit_rows),
        slots=slots, tables=tables, max_q_len=max_q, token_src=i32(token_src))


def prepare_step(entries: list[Entry], cache, vocab_size: int, graph_max_rows: int = 0,
                 has_fed_ids: bool = False) -> tuple[HostBatch, tuple[int, int] | None]:
    """Everything of a step that can fail, all or nothing: admit the requests not seen
    before, reserve pages for every entry's tokens, lay the batch out. If any of it
    fails (no pages, no slot, a token outside the vocabulary, a request named twice, a
    request past the longest length) the error is raised with this call's admissions
    and reservations undone: the cache is as it was.

    Returns the batch and, for a step of single tokens of at most ``graph_max_rows``
    requests that each want their logits, the fixed sizes (rows, table width) at which
    it can be captured and replayed; else None."""
    from pyre_amd.cache.allocator import OutOfPages

    admitted, reserved = [], []
    try:
        seen = set()
        for e in entries:
            if e.rid in seen:
                raise ValueError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
        # all pages or none: checked for the whole step before the first one is taken
        if cache.page_groups:
            need = sum(cache.pages_needed(e.rid if e.rid in cache else None, len(e.tokens)) for e in entries)
            if need > cache.free_pages():
                raise OutOfPages(f"the step needs {need} pages, {cache.free_pages()} are free")
        for e in entries:
            if e.rid not in cache:
                cache.add_request(e.rid)
                admitted.append(e.rid)
        for e in entries:
            cache.reserve(e.rid, len(e.tokens))
            reserved.append(e.rid)
        n_tokens = sum(len(e.tokens) for e in entries)
        # the widest table of the step (the groups share a page size, so their tables are equally long)
        pages = max((len(cache.block_table(e.rid, g)) for e in entries for g in range(len(cache.page_groups))), default=0)
        graphable = (n_tokens == len(entries) and n_tokens <= graph_max_rows and all(len(e.want) == 1 for e in entries))
        if graphable:
            rows, width = round_decode_shape(n_tokens, pages)
        else:
            width = max(MIN_TABLE_WIDTH, -(-pages // 8) * 8)
        hb = build_host_batch(entries, cache, vocab_size, table_width=width)
        if hb.feeds and not has_fed_ids:
            raise ValueError("an entry takes its token from the device, but no ids were given")
        return hb, ((rows, width) if graphable else None)
    except BaseException:
        for rid in admitted:
            cache.free_request(rid)
        for rid in reserved:
            if rid not in admitted:
                cache.unreserve(rid)
        raise


def pad_decode_batch(hb: HostBatch, n_rows: int, scratch_slot: int, max_ctx: int) -> HostBatch:
    """A decode-only batch widened to ``n_rows`` requests with rows that do nothing:
    token 0 at position 0, no cache slot to write to, an empty block table (every key
    hidden), the scratch state slot. A captured step is replayed at a fixed size;
    the rows beyond the live requests are these. ``max_ctx`` is the longest context
    the step's table can hold."""
    pad = n_rows - hb.n_seqs
    if pad < 0 or not hb.decode_only:
        raise ValueError("only decode batches can be padded, and only upwards")
    i32 = lambda x: np.asarray(x, dtype=np.int32)  # noqa: E731
    cat = lambda a, b: np.concatenate([a, i32(b)])  # noqa: E731
    n = hb.n_tokens
    return HostBatch(
        n_tokens=n_rows, n_seqs=n_rows, rids=hb.rids + [None] * pad,
        tokens=cat(hb.tokens, [0] * pad), positions=cat(hb.positions, [0] * pad),
        seq_of_token=cat(hb.seq_of_token, range(hb.n_seqs, n_rows)),
        q_start=i32(range(n_rows + 1)), ctx_len=cat(hb.ctx_len, [1] * pad),
        state_slots=cat(hb.state_slots, [scratch_slot] * pad),
        logit_rows=i32(range(n_rows)),
        slots=[cat(s, [-1] * pad) for s in hb.slots],
        tables=[np.concatenate([t, np.full((pad, t.shape[1]), -1, dtype=np.int32)]) for t in hb.tables],
        max_q_len=1, page_size=hb.page_size, n_single=n_rows, max_single_ctx=max_ctx,
        token_src=cat(hb.token_src, [-1] * pad))
