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


TILE = 32  #: tokens of one request that the prompt-portion attention kernel takes at a time


@dataclass
class Entry:
    rid: object
    tokens: list[int]
    want: list[int] = field(default_factory=list)  #: indices into ``tokens``


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
    max_q_len: int = 0
    decode_tokens: np.ndarray = None   #: token indices of requests that bring one token
    prefill_tiles: np.ndarray = None   #: [T, 2] (first token, count <= TILE) of the others, longest context first
    max_decode_ctx: int = 0            #: longest context among the single-token requests

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1


def build_host_batch(entries: list[Entry], cache, vocab_size: int, table_width: int | None = None) -> HostBatch:
    """Lay the entries out in the order given. ``cache`` is the
    :class:`~pyre_amd.cache.CacheManager`; every request must already have its
    pages reserved for this step."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    seen = set()
    tokens: list[int] = []
    positions: list[int] = []
    seq_of_token: list[int] = []
    q_start = [0]
    ctx_len: list[int] = []
    state_slots: list[int] = []
    logit_rows: list[int] = []
    n_groups = len(cache.page_groups)
    slots: list[list[int]] = [[] for _ in range(n_groups)]
    width = table_width or cache.max_pages_per_seq
    tables = [np.full((len(entries), width), -1, dtype=np.int32) for _ in range(n_groups)]
    max_q = 0
    for s, e in enumerate(entries):
        if e.rid in seen:
            raise ValueError(f"request {e.rid!r} appears twice in one step")
        seen.add(e.rid)
        n = len(e.tokens)
        if n == 0:
            raise ValueError(f"request {e.rid!r} brings no tokens")
        for t in e.tokens:
            if not (0 <= int(t) < vocab_size):
                raise ValueError(f"token id {t} of request {e.rid!r} is outside the vocabulary (0..{vocab_size - 1})")
        start = cache.length(e.rid)
        base = len(tokens)
        tokens.extend(int(t) for t in e.tokens)
        positions.extend(range(start, start + n))
        seq_of_token.extend([s] * n)
        q_start.append(base + n)
        ctx_len.append(start + n)
        state_slots.append(cache.slot(e.rid))
        for w in e.want:
            if not (0 <= int(w) < n):
                raise ValueError(f"request {e.rid!r}: wanted place {w} is outside its {n} tokens")
            logit_rows.append(base + int(w))
        for g in range(n_groups):
            slots[g].extend(cache.slot_mapping(e.rid, g, start, n))
            tbl = cache.block_table(e.rid, g)
            if len(tbl) > width:
                raise ValueError(f"request {e.rid!r} has {len(tbl)} pages, the table holds {width}")
            tables[g][s, :len(tbl)] = tbl
        max_q = max(max_q, n)
    i32 = lambda x: np.asarray(x, dtype=np.int32)  # noqa: E731
    decode_tokens, tiles, max_decode_ctx = [], [], 0
    for s in range(len(entries)):
        a, b = q_start[s], q_start[s + 1]
        if b - a == 1:
            decode_tokens.append(a)
            max_decode_ctx = max(max_decode_ctx, ctx_len[s])
        else:
            tiles.extend((positions[t0] + min(TILE, b - t0), t0, min(TILE, b - t0)) for t0 in range(a, b, TILE))
    tiles.sort(key=lambda t: -t[0])  # the tiles with the most keys start first
    return HostBatch(
        decode_tokens=i32(decode_tokens), prefill_tiles=i32([t[1:] for t in tiles]).reshape(-1, 2),
        max_decode_ctx=max_decode_ctx,
        n_tokens=len(tokens), n_seqs=len(entries), rids=[e.rid for e in entries], tokens=i32(tokens),
        positions=i32(positions), seq_of_token=i32(seq_of_token), q_start=i32(q_start),
        ctx_len=i32(ctx_len), state_slots=i32(state_slots), logit_rows=i32(logit_rows),
        slots=[i32(x) for x in slots], tables=tables, max_q_len=max_q)


def pad_decode_batch(hb: HostBatch, n_rows: int, scratch_slot: int, max_ctx: int) -> HostBatch:
    """A decode-only batch widened to ``n_rows`` requests with rows that do nothing:
    token 0 at position 0, no cache slot to write to, an empty block table (every key
    hidden), the scratch state slot. A captured step is replayed at a fixed size;
    the rows beyond the live requests are these. ``max_ctx`` (the longest context
    the step's table can hold) fixes how the keys are split."""
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
        max_q_len=1, decode_tokens=i32(range(n_rows)), prefill_tiles=i32([]).reshape(-1, 2),
        max_decode_ctx=max_ctx)
