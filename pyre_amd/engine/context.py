"""Per-engine runtime (device, element type, scratch memory) and the per-step
context that every part receives."""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np
import torch

from pyre_amd.engine.batch import HostBatch, round_decode_shape

TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class Workspace:
    """Named scratch buffers that live as long as the engine. A buffer grows when
    a larger one is asked for and is otherwise handed out again, so a step that
    has run once at its largest size allocates nothing afterwards."""

    def __init__(self, device: torch.device):
        self.device = device
        self._bufs: dict[tuple[str, torch.dtype], torch.Tensor] = {}
        self._views: dict[tuple[str, torch.dtype, tuple[int, ...]], torch.Tensor] = {}
        self.frozen = False  #: set while a HIP graph is captured or replayed: growing is an error
        #: set once a step has been captured: a captured step keeps using the memory it was
        #: captured with, so a buffer that grows afterwards leaves its old memory allocated
        self.keep_replaced = False
        self._replaced: list[torch.Tensor] = []

    def get(self, name: str, shape: tuple[int, ...], dtype: torch.dtype, zeroed: bool = False) -> torch.Tensor:
        """``zeroed``: the buffer is zero when it is made (and whoever uses it leaves it so)."""
        shape = tuple(shape)
        view = self._views.get((name, dtype, shape))
        if view is not None:
            return view
        numel = max(1, math.prod(shape))
        key = (name, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < numel:
            if self.frozen:
                raise RuntimeError(f"workspace buffer {name!r} would have to grow inside a captured step")
            if buf is not None and self.keep_replaced:
                self._replaced.append(buf)
            buf = (torch.zeros if zeroed else torch.empty)(numel, device=self.device, dtype=dtype)
            self._bufs[key] = buf
            for k in [k for k in self._views if k[0] == name and k[1] == dtype]:
                del self._views[k]  # views of the buffer that this one replaces
        view = buf[:math.prod(shape)].view(shape)
        if len(self._views) < 4096:
            self._views[(name, dtype, shape)] = view
        return view

    def nbytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in [*self._bufs.values(), *self._replaced])


@dataclass
class Runtime:
    device: torch.device
    dtype: torch.dtype               #: element type of weights' products, activations and caches
    max_positions: int               #: rows of position tables (the longest request)
    workspace: Workspace = None
    options: dict = field(default_factory=dict)
    #: compute units of the device, read once: launch plans whose shape decides the order of a
    #: sum go by this number for as long as the engine lives (None: asked of the device)
    compute_units: int | None = None

    def __post_init__(self) -> None:
        if self.workspace is None:
            self.workspace = Workspace(self.device)
        if self.compute_units is None:
            from pyre_amd.hip import ops

            self.compute_units = ops.compute_units(self.device)

    @property
    def true_fp32(self) -> bool:
        return self.dtype == torch.float32


def meta_layout(n_cap: int, s_cap: int, table_widths: list[int], extra=()) -> tuple[dict, int]:
    """Offsets (in int32 elements) of the step arrays inside the metadata buffer
    for a step of up to ``n_cap`` tokens and ``s_cap`` requests. ``extra``: the arrays
    that parts asked for (:class:`~pyre_amd.parts.base.StepArraySpec`)."""
    off = 0
    lay = {}

    def put(name: str, n: int) -> None:
        nonlocal off
        lay[name] = (off, n)
        off += (n + 3) // 4 * 4

    for name in ("tokens", "positions", "seq_of_token", "logit_rows", "token_src"):
        put(name, n_cap)
    rows = round_decode_shape(s_cap, 1)[0]  # a part may plan single-token requests for the rounded number of them
    for spec in extra:
        put("x:" + spec.name, int(spec.capacity(n_cap, rows)))
    put("q_start", s_cap + 1)
    put("ctx_len", s_cap)
    put("state_slots", s_cap)
    for g, w in enumerate(table_widths):
        put(f"slots{g}", n_cap)
        put(f"table{g}", s_cap * w)
    return lay, off


class MetaBuffers:
    """Pinned host staging and the device copy of a step's int32 arrays."""

    def __init__(self, device: torch.device, max_tokens: int, max_seqs: int, table_widths: list[int], extra=()):
        """``table_widths``: the widest block table of each page group; ``extra``: the
        arrays that parts asked for."""
        self.max_widths = table_widths
        self.extra = list(extra)
        _, size = meta_layout(max_tokens, max_seqs, table_widths, self.extra)
        self.capacity = size
        self.host = torch.empty(size, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(size, dtype=torch.int32, device=device)
        self._copied = torch.cuda.Event()
        self._pending = False

    def upload(self, hb: HostBatch, n_cap: int | None = None, s_cap: int | None = None) -> dict[str, torch.Tensor]:
        n_cap = n_cap or hb.n_tokens
        s_cap = s_cap or hb.n_seqs
        widths = [t.shape[1] for t in hb.tables]
        lay, used = meta_layout(n_cap, s_cap, widths, self.extra)
        if used > self.capacity:
            raise RuntimeError(f"step of {n_cap} tokens / {s_cap} requests exceeds the engine's limits")
        if self._pending:
            self._copied.synchronize()
        h = self.host_np
        h[:used] = 0

        def fill(name: str, arr: np.ndarray) -> None:
            o, _ = lay[name]
            h[o:o + arr.size] = arr.reshape(-1)

        fill("tokens", hb.tokens), fill("positions", hb.positions), fill("seq_of_token", hb.seq_of_token)
        fill("logit_rows", hb.logit_rows), fill("q_start", hb.q_start), fill("ctx_len", hb.ctx_len)
        fill("state_slots", hb.state_slots)
        for spec in self.extra:
            arr = hb.arrays[spec.name]
            if arr.size > lay["x:" + spec.name][1]:
                raise RuntimeError(f"step array {spec.name!r} has {arr.size} entries, its stated capacity is "
                                   f"{lay['x:' + spec.name][1]}")
            fill("x:" + spec.name, arr)
        o, n = lay["token_src"]
        h[o:o + n] = -1
        if hb.token_src is not None:
            fill("token_src", hb.token_src)
        for g, w in enumerate(widths):
            fill(f"slots{g}", hb.slots[g])
            o, _ = lay[f"table{g}"]
            tbl = hb.tables[g]
            h[o:o + tbl.size] = tbl.reshape(-1)
            if s_cap > hb.n_seqs:  # padding rows of a captured step read nothing
                h[o + tbl.size:o + s_cap * w] = -1
        self.dev[:used].copy_(self.host[:used], non_blocking=True)
        self._copied.record()
        self._pending = True
        views = {}
        for name, (o, n) in lay.items():
            views[name] = self.dev[o:o + n]
        for g, w in enumerate(widths):
            views[f"table{g}"] = views[f"table{g}"].view(s_cap, w)
        return views


@dataclass
class PagedLayerView:
    """One layer's paged tensors and the step's addressing for its group."""

    tensors: dict                    #: name -> [pages, *page_shape], as the mixer's description laid them out
    table: torch.Tensor              #: [S, P] int32, this step's block tables
    slots: torch.Tensor              #: [N] int32, where this step's tokens go (page * page_size + offset)
    page_size: int
    window: int
    writes: bool = True              #: False: the layer reads a cache another layer wrote

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.tensors[name]


@dataclass
class StateLayerView:
    """One layer's per-request state: ``tensor[slot]`` belongs to the request in that slot."""

    tensor: torch.Tensor             #: [num_slots, *shape]
    slots: torch.Tensor              #: [S] int32, slot of each request of the step


@dataclass
class StepContext:
    runtime: Runtime
    host: HostBatch
    n_tokens: int
    n_seqs: int
    n_logits: int
    tokens: torch.Tensor
    positions: torch.Tensor
    seq_of_token: torch.Tensor
    logit_rows: torch.Tensor
    q_start: torch.Tensor
    ctx_len: torch.Tensor
    state_slots: torch.Tensor
    arrays: dict = field(default_factory=dict)  #: name -> int32 device array that a part asked for

    @property
    def workspace(self) -> Workspace:
        return self.runtime.workspace

    @property
    def dtype(self) -> torch.dtype:
        return self.runtime.dtype
