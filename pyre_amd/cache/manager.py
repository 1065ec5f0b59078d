"""The cache manager: page pools, block tables, state slots.

Every entry of a model's layer order declares what it keeps: a list of cache descriptions
(:class:`~pyre_amd.parts.base.PagedCacheSpec`, :class:`~pyre_amd.parts.base.StateCacheSpec`),
one per cache of the entry's layer (none, one for a layer with one mixer, more for a layer with
several). A *cell* is (entry, index in that list). Cells with the same needs form a *group*:

* a **page group** has a pool of pages of its own and, for each request, a block
  table of its own. One page id addresses that page in every layer of the group
  (`pyre/paged_cache.py:96-109` lays the reference's single pool out the same way).
  Which tensors a page holds, and how a page of each is laid out, is what the
  description says (the mixer's choice); the manager allocates
  ``[layers, pages, *page_shape]`` for each and knows nothing of their meaning.
  A group with a window gives a page back as soon as no later query can see it.
  All groups share one page size, the engine's; a description that names another
  (``PagedCacheSpec.page_size``: a mixer whose kernels need pages of a particular size) is
  refused when the manager is made.
* a **state group** has one fixed-size state per (layer, slot).

A request holds one *slot* from admission to its end; the slot indexes the state
tensors. Pages are *reserved* for all tokens of a step before the step runs and
the request's length is *committed* after it, so no kernel ever sees a half-grown
table (`pyre/paged_cache.py:118-122,198-201` has per-layer side effects instead,
and `tests/test_paged_cache.py:203-213` records the bug that came of it).

This module is bookkeeping only and runs without a GPU; ``materialize`` allocates
the pools' tensors.

``fill(tensor, ids, value)`` sets ``tensor[:, id]`` to ``value`` for the listed pages or
slots (the engine passes its fill kernel; without one torch does it). It zeroes a state
slot when a request starts. Debugging aid: with ``poison=True`` every page and every state
slot that goes back to a pool is filled with NaN at once, and the whole pool at the start,
so that a read of memory which no live request owns shows in the results instead of hiding
behind stale, finite data. A page is handed out as it is (NaN in that mode): a mixer whose
kernels read slots of its own pages that it has not written yet has to see to it that they are
harmless (the attention part's writing kernel zeroes the values behind a step's last token).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from pyre_amd.cache.allocator import OutOfPages, PageAllocator
from pyre_amd.parts.base import PagedCacheSpec, StateCacheSpec

RELEASED = -1  #: block-table entry of a page that a window has passed


class _Cells:
    """The cells (entry of the layer order, index among that entry's caches) of a group, in order."""

    cells: list

    @property
    def entries(self) -> list[int]:
        """Positions in the layer order, ascending (an entry with two cells of this group twice)."""
        return [entry for entry, _ in self.cells]

    def layer_index(self, entry: int, k: int = 0) -> int:
        """Where cell (entry, k) lies along the first axis of the group's tensors."""
        return self.cells.index((entry, k))


@dataclass
class PageGroup(_Cells):
    index: int
    spec: PagedCacheSpec
    cells: list[tuple[int, int]]
    page_size: int
    num_pages: int
    allocator: PageAllocator
    #: name -> [len(cells), num_pages, *page_shape] for every tensor of the description
    tensors: dict = field(default_factory=dict)


@dataclass
class StateGroup(_Cells):
    index: int
    spec: StateCacheSpec
    cells: list[tuple[int, int]]
    tensor: object = None            #: [len(cells), num_slots, *shape]


@dataclass
class _Request:
    slot: int
    length: int = 0                  #: tokens committed
    reserved: int = 0                #: tokens that pages exist for
    tables: list[list[int]] = field(default_factory=list)  #: one per page group
    #: the same tables as int32 arrays (filled with RELEASED beyond their ends), kept in
    #: step with the lists so that a step's batch copies rows instead of converting lists
    arrays: list[np.ndarray] = field(default_factory=list)


class CacheManager:
    def __init__(self, cache_specs: list, page_size: int, num_pages: int, max_num_seqs: int,
                 max_model_len: int, fill=None, poison: bool = False):
        """``cache_specs[i]`` is what entry i of the layer order keeps: a list of descriptions
        (a single description or None stand for a list of one or of none)."""
        self.fill = fill
        self.poison = poison
        if page_size <= 0 or num_pages <= 0 or max_num_seqs <= 0:
            raise ValueError("page_size, num_pages and max_num_seqs must be positive")
        self.page_size = page_size
        self.max_num_seqs = max_num_seqs
        self.max_model_len = max_model_len
        self.max_pages_per_seq = -(-max_model_len // page_size)
        self.page_groups: list[PageGroup] = []
        self.state_groups: list[StateGroup] = []
        #: (entry, index among the entry's caches) -> ("paged" | "state", group index)
        self.group_of_cell: dict[tuple[int, int], tuple[str, int]] = {}
        by_spec: dict[object, object] = {}
        for entry, kept in enumerate(cache_specs):
            specs = [] if kept is None else list(kept) if isinstance(kept, (list, tuple)) else [kept]
            for k, spec in enumerate(specs):
                grp = by_spec.get(spec)
                if grp is None:
                    if isinstance(spec, PagedCacheSpec):
                        if spec.page_size not in (None, page_size):
                            raise ValueError(f"entry {entry} of the layer order keeps a cache whose kernels need pages "
                                             f"of {spec.page_size} tokens; the engine is set to pages of {page_size}, "
                                             "and all page groups share one size: set page_size to that")
                        grp = PageGroup(len(self.page_groups), spec, [], page_size, num_pages,
                                        PageAllocator(num_pages))
                        self.page_groups.append(grp)
                    elif isinstance(spec, StateCacheSpec):
                        grp = StateGroup(len(self.state_groups), spec, [])
                        self.state_groups.append(grp)
                    else:
                        raise TypeError(f"entry {entry}: unknown cache description {spec!r}")
                    by_spec[spec] = grp
                grp.cells.append((entry, k))
                self.group_of_cell[(entry, k)] = ("paged" if isinstance(grp, PageGroup) else "state", grp.index)
        self._caches_of_entry: dict[int, int] = {}
        for entry, _ in self.group_of_cell:
            self._caches_of_entry[entry] = self._caches_of_entry.get(entry, 0) + 1
        self.slots = PageAllocator(max_num_seqs, what="slot")
        self._requests: dict[object, _Request] = {}

    @property
    def group_of_entry(self) -> dict[int, tuple[str, int]]:
        """entry -> ("paged" | "state", group index) of the entry's first cache."""
        return {entry: where for (entry, k), where in self.group_of_cell.items() if k == 0}

    def caches_of_entry(self, entry: int) -> int:
        """How many caches entry ``entry`` of the layer order keeps."""
        return self._caches_of_entry.get(entry, 0)

    # ------------------------------------------------------------------ tensors

    def materialize(self, device, dtype) -> None:
        """Allocate the pools on ``device`` ("model" tensors in ``dtype``)."""
        import torch

        for g in self.page_groups:
            n = len(g.cells)
            for t in g.spec.tensors:
                dt = torch.float32 if t.dtype == "float32" else dtype
                g.tensors[t.name] = torch.zeros((n, g.num_pages, *t.page_shape(g.page_size)), device=device, dtype=dt)
            self._poison_pages(g, range(g.num_pages))
        for g in self.state_groups:
            dt = torch.float32 if g.spec.dtype == "float32" else dtype
            # one slot more than requests: padding rows of a captured step write there
            g.tensor = torch.zeros((len(g.cells), self.max_num_seqs + 1, *g.spec.shape), device=device, dtype=dt)
            if self.poison:
                self._fill(g.tensor, list(range(self.max_num_seqs)), float("nan"))

    def _fill(self, tensor, ids: list[int], value: float) -> None:
        if tensor is None or not ids:
            return
        if self.fill is not None:
            self.fill(tensor, ids, value)
        else:
            tensor[:, ids] = value

    def _poison_pages(self, g: PageGroup, pages) -> None:
        if not self.poison:
            return
        pages = list(pages)
        for t in g.tensors.values():
            self._fill(t, pages, float("nan"))

    def bytes_per_page(self, dtype_bytes: int) -> int:
        return sum(len(g.cells) * t.elements_per_token() * g.page_size * (4 if t.dtype == "float32" else dtype_bytes)
                   for g in self.page_groups for t in g.spec.tensors)

    # ------------------------------------------------------------------ requests

    def __contains__(self, rid) -> bool:
        return rid in self._requests

    @property
    def live_requests(self) -> list:
        return list(self._requests)

    def has_free_slot(self) -> bool:
        return self.slots.num_free > 0

    def add_request(self, rid) -> int:
        if rid in self._requests:
            raise ValueError(f"request {rid!r} already exists")
        slot = self.slots.allocate()
        self._requests[rid] = _Request(
            slot, tables=[[] for _ in self.page_groups],
            arrays=[np.full(self.max_pages_per_seq, RELEASED, dtype=np.int32) for _ in self.page_groups])
        for g in self.state_groups:
            self._fill(g.tensor, [slot], 0.0)
        return slot

    def slot(self, rid) -> int:
        return self._requests[rid].slot

    def length(self, rid) -> int:
        return self._requests[rid].length

    def _pages_to_add(self, req: _Request, new_len: int) -> int:
        have = len(req.tables[0]) if self.page_groups else 0
        return max(0, -(-new_len // self.page_size) - have)

    def pages_needed(self, rid, n_new: int) -> int:
        """Pages per group that ``reserve(rid, n_new)`` would take (rid may be new: None)."""
        if not self.page_groups:
            return 0
        if rid is None or rid not in self._requests:
            return -(-n_new // self.page_size)
        req = self._requests[rid]
        return self._pages_to_add(req, req.length + n_new)

    def free_pages(self) -> int:
        """Free pages of the tightest group."""
        return min((g.allocator.num_free for g in self.page_groups), default=1 << 30)

    def reserve(self, rid, n_new: int) -> None:
        """Make room for the next ``n_new`` tokens of ``rid`` in every page group.
        Takes all pages or none (:class:`OutOfPages`)."""
        req = self._requests[rid]
        new_len = req.length + n_new
        if new_len > self.max_model_len:
            raise ValueError(f"request {rid!r} would reach {new_len} tokens; the engine's limit is {self.max_model_len}")
        add = self._pages_to_add(req, new_len)
        if add:
            for g in self.page_groups:
                if g.allocator.num_free < add:
                    raise OutOfPages(f"page pool of group {g.index} exhausted "
                                     f"({add} needed, {g.allocator.num_free} of {g.num_pages} free)")
            for g, table, arr in zip(self.page_groups, req.tables, req.arrays):
                have = len(table)
                table.extend(g.allocator.allocate_many(add))
                arr[have:have + add] = table[have:]
        req.reserved = max(req.reserved, new_len)

    def slot_mapping(self, rid, group: int, start: int, n: int) -> list[int]:
        """Flat cache slot (page * page_size + offset) of positions start .. start+n-1."""
        table = self._requests[rid].tables[group]
        ps = self.page_size
        out = []
        for pos in range(start, start + n):
            page = table[pos // ps]
            if page == RELEASED:
                raise RuntimeError(f"position {pos} of request {rid!r} lies in a released page")
            out.append(page * ps + pos % ps)
        return out

    def block_table(self, rid, group: int) -> list[int]:
        return self._requests[rid].tables[group]

    def block_table_array(self, rid, group: int) -> np.ndarray:
        """The request's block table as int32 ``[max_pages_per_seq]``; entries beyond
        its pages are RELEASED. Do not write to it."""
        return self._requests[rid].arrays[group]

    def commit(self, rid, n_new: int) -> None:
        """The step has run: the request is ``n_new`` tokens longer. Pages of a
        windowed group that no later query can see go back to the pool."""
        req = self._requests[rid]
        req.length += n_new
        if req.length > req.reserved:
            raise RuntimeError(f"request {rid!r}: committed past the reservation")
        for g, table, arr in zip(self.page_groups, req.tables, req.arrays):
            w = g.spec.window
            if w <= 0:
                continue
            # The next query sits at position req.length and sees keys > length - w.
            dead_upto = req.length - w  # keys <= dead_upto are never read again
            last_dead_page = (dead_upto + 1) // self.page_size - 1
            dead = []
            for i in range(min(last_dead_page + 1, len(table))):
                if table[i] != RELEASED:
                    g.allocator.free(table[i])
                    dead.append(table[i])
                    table[i] = RELEASED
                    arr[i] = RELEASED
            self._poison_pages(g, dead)

    def free_request(self, rid) -> None:
        req = self._requests.pop(rid)
        for g, table in zip(self.page_groups, req.tables):
            held = [page for page in table if page != RELEASED]
            for page in reversed(held):
                g.allocator.free(page)
            self._poison_pages(g, held)
        self.slots.free(req.slot)
        if self.poison:
            for g in self.state_groups:
                self._fill(g.tensor, [req.slot], float("nan"))

    def unreserve(self, rid) -> None:
        """Give back the pages that were reserved beyond the request's committed length
        (a step that was prepared and then not run)."""
        req = self._requests[rid]
        keep = -(-req.length // self.page_size)
        for g, table, arr in zip(self.page_groups, req.tables, req.arrays):
            extra = table[keep:]
            for page in reversed(extra):
                if page != RELEASED:
                    g.allocator.free(page)
            self._poison_pages(g, [p for p in extra if p != RELEASED])
            del table[keep:]
            arr[keep:] = RELEASED
        req.reserved = req.length

    # ------------------------------------------------------------------ checks

    def check_invariants(self) -> None:
        """No page lost, held twice or free while held (used by the tests)."""
        for gi, g in enumerate(self.page_groups):
            held = [p for r in self._requests.values() for p in r.tables[gi] if p != RELEASED]
            if len(held) != len(set(held)):
                raise AssertionError(f"group {gi}: a page is held twice")
            if len(held) != g.allocator.num_used:
                raise AssertionError(f"group {gi}: {g.allocator.num_used} pages in use, {len(held)} held")
            for p in held:
                if not g.allocator.is_used(p):
                    raise AssertionError(f"group {gi}: page {p} is held but free")
        slots = [r.slot for r in self._requests.values()]
        if len(slots) != len(set(slots)) or len(slots) != self.slots.num_used:
            raise AssertionError("slot bookkeeping is inconsistent")
