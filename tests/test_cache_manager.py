"""The cache manager's bookkeeping (CPU): allocator vectors of the reference's tests,
block tables, groups, windows, slots, and invariants under random orders."""

from __future__ import annotations

import random

import pytest

from pyre_amd.cache import RELEASED, CacheManager, OutOfPages, PageAllocator
from pyre_amd.parts.base import PagedCacheSpec, PagedTensorSpec, StateCacheSpec


def KVCacheSpec(nkv, hd, window=0):
    return PagedCacheSpec((PagedTensorSpec("k", (nkv, hd), 1), PagedTensorSpec("v", (nkv, hd), 2)), window)


FULL = KVCacheSpec(2, 16)
WIN = KVCacheSpec(2, 16, window=40)


# --- the reference's allocator tests (tests/test_paged_cache.py:23-66) ------------

def test_allocate_and_free_roundtrip():
    a = PageAllocator(4)
    pages = [a.allocate() for _ in range(4)]
    assert a.num_free == 0 and len(set(pages)) == 4
    for p in pages:
        a.free(p)
    assert a.num_free == 4 and a.num_used == 0


def test_exhaustion_raises():
    a = PageAllocator(2)
    a.allocate(), a.allocate()
    with pytest.raises(MemoryError, match="exhausted"):
        a.allocate()
    with pytest.raises(OutOfPages):
        a.allocate_many(1)


def test_freed_pages_are_reused_at_once():
    a = PageAllocator(2)
    p0 = a.allocate()
    a.allocate()
    a.free(p0)
    assert a.allocate() == p0


def test_double_free_raises():
    a = PageAllocator(2)
    p = a.allocate()
    a.free(p)
    with pytest.raises(ValueError, match="double free"):
        a.free(p)
    with pytest.raises(ValueError):
        a.free(1)            # never allocated


def test_allocate_many_is_all_or_nothing():
    a = PageAllocator(3)
    a.allocate()
    with pytest.raises(OutOfPages):
        a.allocate_many(3)
    assert a.num_free == 2


# --- block tables (tests/test_paged_cache.py:69-102) -----------------------------

def manager(specs=(FULL, FULL), pages=8, seqs=4, page_size=16, max_len=256):
    return CacheManager(list(specs), page_size, pages, seqs, max_len)


def test_seventeen_tokens_take_two_pages():
    m = manager()
    m.add_request("a")
    m.reserve("a", 17)
    assert len(m.block_table("a", 0)) == 2 and m.page_groups[0].allocator.num_used == 2
    m.commit("a", 17)
    m.reserve("a", 15)                                   # 32 tokens still fit two pages
    assert len(m.block_table("a", 0)) == 2
    m.commit("a", 15)
    m.reserve("a", 1)
    assert len(m.block_table("a", 0)) == 3


def test_free_returns_everything_and_requests_are_disjoint():
    m = manager()
    m.add_request("a"), m.add_request("b")
    m.reserve("a", 48), m.reserve("b", 16)
    assert set(m.block_table("a", 0)).isdisjoint(m.block_table("b", 0))
    assert m.slot("a") != m.slot("b")
    m.check_invariants()
    m.free_request("a")
    assert "a" not in m and m.page_groups[0].allocator.num_used == 1
    m.free_request("b")
    assert m.page_groups[0].allocator.num_used == 0 and m.slots.num_used == 0
    with pytest.raises(ValueError, match="already exists"):
        m.add_request("c"), m.add_request("c")


def test_slot_mapping_follows_the_table():
    m = manager(page_size=8)
    m.add_request("a")
    m.reserve("a", 20)
    t = m.block_table("a", 0)
    got = m.slot_mapping("a", 0, 5, 6)                   # positions 5..10 cross a page edge
    assert got == [t[0] * 8 + 5, t[0] * 8 + 6, t[0] * 8 + 7, t[1] * 8 + 0, t[1] * 8 + 1, t[1] * 8 + 2]


def test_reserve_takes_all_pages_or_none():
    m = manager(pages=3)
    m.add_request("a"), m.add_request("b")
    m.reserve("a", 32)
    with pytest.raises(OutOfPages):
        m.reserve("b", 33)                               # needs 3, 1 free
    assert m.block_table("b", 0) == [] and m.page_groups[0].allocator.num_free == 1
    m.check_invariants()
    with pytest.raises(ValueError, match="limit"):
        m.reserve("a", 1000)
    with pytest.raises(RuntimeError, match="reservation"):
        m.commit("b", 5)


def test_slots_run_out_separately():
    m = manager(seqs=2)
    m.add_request(1), m.add_request(2)
    assert not m.has_free_slot()
    with pytest.raises(OutOfPages, match="slot"):
        m.add_request(3)


# --- groups -----------------------------------------------------------------------

def test_layers_with_the_same_needs_share_a_group():
    specs = [FULL, WIN, FULL, None, StateCacheSpec((4, 8)), WIN, StateCacheSpec((4, 8))]
    m = CacheManager(specs, 16, 10, 4, 512)
    assert [g.entries for g in m.page_groups] == [[0, 2], [1, 5]]
    assert [g.entries for g in m.state_groups] == [[4, 6]]
    assert m.group_of_entry == {0: ("paged", 0), 2: ("paged", 0), 1: ("paged", 1), 5: ("paged", 1), 4: ("state", 0),
                                6: ("state", 0)}
    assert m.page_groups[1].layer_index(5) == 1
    assert m.bytes_per_page(2) == 2 * (2 * 2 * 16 * 16 * 2) * 2


def test_an_entry_may_keep_several_caches():
    """A layer with two mixers keeps two caches: the entry's description is a list, and a cell
    is (entry, place in that list)."""
    state = StateCacheSpec((4, 8))
    specs = [[FULL, state], [], [WIN], None, [FULL, FULL]]
    m = CacheManager(specs, 16, 10, 4, 512)
    assert [g.cells for g in m.page_groups] == [[(0, 0), (4, 0), (4, 1)], [(2, 0)]]
    assert [g.cells for g in m.state_groups] == [[(0, 1)]]
    assert [m.caches_of_entry(e) for e in range(5)] == [2, 0, 1, 0, 2]
    assert m.group_of_cell[(4, 1)] == ("paged", 0) and m.page_groups[0].layer_index(4, 1) == 2
    assert m.group_of_entry == {0: ("paged", 0), 2: ("paged", 1), 4: ("paged", 0)}
    assert m.bytes_per_page(2) == (3 + 1) * (2 * 2 * 16 * 16 * 2)


def test_a_cache_that_needs_pages_of_another_size_is_refused():
    """All page groups share the engine's page size; a mixer whose kernels need another says so
    in its description and is refused when the manager is made, not at its first step."""
    needs_32 = PagedCacheSpec((PagedTensorSpec("k", (2, 16), token_axis=1),), page_size=32)
    CacheManager([FULL, needs_32], 32, 10, 4, 512)
    with pytest.raises(ValueError, match="pages of 32 tokens.*set to pages of 16"):
        CacheManager([FULL, needs_32], 16, 10, 4, 512)
    with pytest.raises(ValueError, match="positive"):
        PagedCacheSpec((PagedTensorSpec("k", (2, 16)),), page_size=0)


def test_a_window_gives_pages_back_once_passed():
    m = CacheManager([FULL, WIN], 16, 12, 2, 512)
    m.add_request("a")
    m.reserve("a", 100)
    m.commit("a", 100)
    full, win = m.block_table("a", 0), m.block_table("a", 1)
    # next query at 100 sees keys 61..100: keys <= 60 are dead: pages 0..2 (keys 0..47) go, page 3 (48..63) stays
    assert win[:3] == [RELEASED] * 3 and all(p != RELEASED for p in win[3:]) and RELEASED not in full
    assert m.page_groups[1].allocator.num_used == 4 and m.page_groups[0].allocator.num_used == 7
    with pytest.raises(RuntimeError, match="released"):
        m.slot_mapping("a", 1, 40, 1)
    for _ in range(30):                                   # decoding on: the window slides, pages keep coming back
        m.reserve("a", 1)
        m.commit("a", 1)
    m.check_invariants()
    assert m.page_groups[1].allocator.num_used <= 4
    m.free_request("a")
    assert all(g.allocator.num_used == 0 for g in m.page_groups)


def test_window_release_never_hides_a_visible_key():
    """For every way of cutting a request into portions, each query's window
    [p - w + 1, p] lies in pages that are still held when the portion runs."""
    rng = random.Random(4)
    for _ in range(50):
        w, ps = rng.choice([1, 5, 16, 33]), rng.choice([4, 16])
        m = CacheManager([KVCacheSpec(1, 8, window=w)], ps, 64, 1, 400)
        m.add_request(0)
        total = 0
        while total < 300:
            n = rng.choice([1, 1, 2, 7, 40])
            m.reserve(0, n)
            table = m.block_table(0, 0)
            first_query = total
            for key in range(max(0, first_query - w + 1), total + n):
                assert table[key // ps] != RELEASED
            m.commit(0, n)
            total += n
        m.free_request(0)
        assert m.page_groups[0].allocator.num_used == 0


# --- random orders -----------------------------------------------------------------

@pytest.mark.parametrize("seed", range(8))
def test_no_page_lost_held_twice_or_freed_twice(seed):
    rng = random.Random(seed)
    m = CacheManager([FULL, WIN, StateCacheSpec((3,))], rng.choice([4, 16]), 40, 6, 300)
    live, next_id = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.has_free_slot():
            m.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 3, 17, 50])
            try:
                m.reserve(rid, n)
            except OutOfPages:
                victim = rng.choice(list(live))            # what a scheduler would do: give one up
                m.free_request(victim)
                del live[victim]
            except ValueError:
                m.free_request(rid)                        # reached the longest length
                del live[rid]
            else:
                m.commit(rid, n)
                live[rid] += n
                assert m.length(rid) == live[rid]
        elif live:
            rid = rng.choice(list(live))
            m.free_request(rid)
            del live[rid]
        m.check_invariants()
        assert set(m.live_requests) == set(live)
    for rid in list(live):
        m.free_request(rid)
    assert all(g.allocator.num_used == 0 for g in m.page_groups) and m.slots.num_used == 0


# --- what a page holds is the mixer's business ------------------------------------------

def test_a_page_holds_whatever_the_description_says():
    import torch

    latent = PagedCacheSpec((PagedTensorSpec("latent", (24,)), PagedTensorSpec("gate", (3, 2), token_axis=2, dtype="float32")))
    assert PagedTensorSpec("k", (2, 16), 1).page_shape(8) == (2, 8, 16)
    assert PagedTensorSpec("v", (2, 16), 2).page_shape(8) == (2, 16, 8)
    assert PagedTensorSpec("latent", (24,)).page_shape(8) == (8, 24)
    m = CacheManager([latent, FULL, latent], 8, 5, 2, 64)
    assert [g.entries for g in m.page_groups] == [[0, 2], [1]]
    m.materialize("cpu", torch.bfloat16)
    g = m.page_groups[0]
    assert g.tensors["latent"].shape == (2, 5, 8, 24) and g.tensors["latent"].dtype == torch.bfloat16
    assert g.tensors["gate"].shape == (2, 5, 3, 2, 8) and g.tensors["gate"].dtype == torch.float32
    assert set(m.page_groups[1].tensors) == {"k", "v"}
    assert m.bytes_per_page(2) == 2 * 8 * (24 * 2 + 6 * 4) + 2 * (2 * 16 * 8 * 2)
    with pytest.raises(ValueError, match="name of its own"):
        PagedCacheSpec((PagedTensorSpec("x", (4,)), PagedTensorSpec("x", (4,))))
    with pytest.raises(ValueError, match="token_axis"):
        PagedTensorSpec("x", (4,), token_axis=2)


def test_unreserve_gives_back_what_a_step_that_did_not_run_had_taken():
    m = CacheManager([FULL, WIN], 16, 12, 2, 512)
    m.add_request("a")
    m.reserve("a", 20)
    m.commit("a", 20)
    before = [list(m.block_table("a", g)) for g in range(2)]
    m.reserve("a", 70)                 # four more pages in each group
    assert m.page_groups[0].allocator.num_used == 6
    m.unreserve("a")
    assert [list(m.block_table("a", g)) for g in range(2)] == before
    assert m.page_groups[0].allocator.num_used == 2 and m.length("a") == 20
    assert (m.block_table_array("a", 0)[2:] == RELEASED).all()
    m.check_invariants()
    m.reserve("a", 70)
    m.commit("a", 70)                  # and the request goes on as if nothing had happened
    m.check_invariants()
    m.free_request("a")
    assert m.page_groups[0].allocator.num_used == 0 and m.page_groups[1].allocator.num_used == 0


def test_poison_mode_marks_what_nobody_holds():
    """NaN wherever no live request holds the memory and in the slots of a held page that its
    request has not written yet (a page is handed out as it is), under a random sequence of
    requests with a window (on the CPU: torch does the filling)."""
    import torch

    rng = random.Random(5)
    m = CacheManager([FULL, WIN, StateCacheSpec((3,))], 16, 14, 3, 400, poison=True)
    m.materialize("cpu", torch.float32)
    assert all(torch.isnan(t).all() for g in m.page_groups for t in g.tensors.values())
    assert torch.isnan(m.state_groups[0].tensor[:, :3]).all()
    live = {}
    for step in range(300):
        if live and rng.random() < 0.25:
            rid = rng.choice(list(live))
            m.free_request(rid)
            del live[rid]
        elif len(live) < 3 and rng.random() < 0.5:
            rid = step
            slot = m.add_request(rid)
            assert (m.state_groups[0].tensor[:, slot] == 0).all()
            live[rid] = 0
        elif live:
            rid = rng.choice(list(live))
            n = rng.randrange(1, 40)
            try:
                m.reserve(rid, n)
            except (OutOfPages, ValueError):
                continue
            # the request writes its tokens (here: ones) and commits
            for gi, g in enumerate(m.page_groups):
                for pos in range(live[rid], live[rid] + n):
                    page = m.block_table(rid, gi)[pos // 16]
                    g.tensors["k"][:, page, :, pos % 16] = 1.0
            m.commit(rid, n)
            live[rid] += n
        m.check_invariants()
        for gi, g in enumerate(m.page_groups):
            written = {}                                   # page -> slots of it that its request has written
            for r, length in live.items():
                for i, p in enumerate(m.block_table(r, gi)):
                    if p != RELEASED:
                        written[p] = max(0, min(16, length - 16 * i))
            for p in range(g.num_pages):
                nan = torch.isnan(g.tensors["k"][:, p])    # [layers, kv heads, slots, head]
                n = written.get(p, 0)
                assert not nan[:, :, :n].any() and nan[:, :, n:].all(), (step, gi, p)
        free_slots = set(range(3)) - {m.slot(r) for r in live}
        for sl in free_slots:
            assert torch.isnan(m.state_groups[0].tensor[:, sl]).all()


# --- a step is prepared all or nothing ---------------------------------------------------

def _snapshot(m):
    return ({r: (m.slot(r), m.length(r), [list(m.block_table(r, g)) for g in range(len(m.page_groups))])
             for r in m.live_requests},
            [g.allocator.num_free for g in m.page_groups], m.slots.num_free)


def test_a_step_that_cannot_be_prepared_leaves_the_cache_as_it_was():
    from pyre_amd.engine.batch import Entry, prepare_step

    m = CacheManager([FULL, WIN], 16, 8, 3, 256)
    hb, shape = prepare_step([Entry("a", [1] * 40, [39])], m, 100)
    assert shape is None and hb.n_tokens == 40
    m.commit("a", 40)
    before = _snapshot(m)
    # the second entry runs out of pages: "a" keeps no reservation, "b" and "c" are not admitted
    with pytest.raises(OutOfPages):
        prepare_step([Entry("a", [1] * 20, []), Entry("b", [2] * 60, []), Entry("c", [3] * 30, [])], m, 100)
    assert _snapshot(m) == before
    m.check_invariants()
    # reserve itself fails (the longest length) after others were reserved
    roomy = CacheManager([FULL], 16, 40, 3, 100)
    prepare_step([Entry("a", [1] * 40, [])], roomy, 100)
    roomy.commit("a", 40)
    was = _snapshot(roomy)
    with pytest.raises(ValueError, match="limit"):
        prepare_step([Entry("b", [2] * 10, []), Entry("a", [1] * 70, [])], roomy, 100)
    assert _snapshot(roomy) == was
    # laying out fails after everything was reserved: a token outside the vocabulary
    with pytest.raises(ValueError, match="vocabulary"):
        prepare_step([Entry("a", [1, 2], []), Entry("b", [5, 100], [])], m, 100)
    assert _snapshot(m) == before
    with pytest.raises(ValueError, match="twice"):
        prepare_step([Entry("b", [1], []), Entry("b", [2], [])], m, 100)
    with pytest.raises(ValueError, match="wanted place"):
        prepare_step([Entry("b", [1, 2], [2])], m, 100)
    # no slot for a fourth request
    for r in "bc":
        prepare_step([Entry(r, [1], [])], m, 100)
        m.commit(r, 1)
    before = _snapshot(m)
    with pytest.raises(OutOfPages, match="slot"):
        prepare_step([Entry("a", [1], []), Entry("d", [1], [])], m, 100)
    assert _snapshot(m) == before
    m.check_invariants()
    # and a retry with a batch that fits goes through
    hb, shape = prepare_step([Entry("a", [7], [0]), Entry("b", [8], [0])], m, 100, graph_max_rows=64)
    assert shape == (2, 8) and hb.n_single == 2 and hb.decode_shape() == (2, 8 * 16)


def test_rounding_of_decode_steps_is_idempotent():
    from pyre_amd.engine.batch import DECODE_ROW_BUCKETS, round_decode_shape

    for n in range(1, 70):
        for pages in (1, 7, 8, 9, 200, 256, 257):
            rows, width = round_decode_shape(n, pages)
            assert rows >= n and width >= pages and width & (width - 1) == 0
            assert round_decode_shape(rows, width) == (rows, width)
            assert rows in DECODE_ROW_BUCKETS or n > DECODE_ROW_BUCKETS[-1]
