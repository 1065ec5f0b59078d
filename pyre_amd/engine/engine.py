"""The engine: a model, its caches and one step function.

``Engine.step(entries)`` runs exactly the tokens it is given, as one batch, against
the cache that earlier steps left, and returns the float32 logits at the wanted
places. The reference has three separate forwards for this (`pyre/model.py:188-201`
contiguous cache and one shared start, `:251-294` one request with any number of
tokens, `:297-342` many requests with one token each) and an empty `pyre/engine.py`.
"""

from __future__ import annotations

from pathlib import Path

import torch

from pyre_amd.cache import CacheManager
from pyre_amd.config.engine import EngineConfig
from pyre_amd.config.model import ModelConfig
from pyre_amd.engine.batch import DECODE_ROW_BUCKETS, Entry, pad_decode_batch, prepare_step, round_decode_shape
from pyre_amd.engine.context import (TORCH_DTYPES, MetaBuffers, PagedLayerView, Runtime, StateLayerView,
                                     StepContext)
from pyre_amd.parts.model import LayeredModel
from pyre_amd.registry import get_architecture, load_config
from pyre_amd.weights.loader import adopt_state, load_weights


#: decode steps of up to this many requests are captured in HIP graphs, at these sizes
GRAPH_ROW_BUCKETS = DECODE_ROW_BUCKETS
GRAPH_MAX_ROWS = GRAPH_ROW_BUCKETS[-1]


class Engine:
    #: ``step`` takes ``fed_ids``: tokens that are results still on the device
    accepts_fed_ids = True

    def __init__(self, model: LayeredModel, config: ModelConfig, engine_config: EngineConfig):
        if not torch.cuda.is_available():
            raise RuntimeError("pyre_amd needs a GPU: there is no CPU execution path")
        from pyre_amd.hip import lib

        lib.lib()  # fail now, and loudly, if the kernel library cannot be built or loaded
        self.model = model
        self.config = config
        self.engine_config = ec = engine_config
        self.device = torch.device(ec.device)
        self.dtype = TORCH_DTYPES[ec.dtype]
        spec = model.spec
        # The model's own limit is the default, not a bound: the reference reads
        # max_position_embeddings and never consults it (`pyre/config.py:60`).
        self.max_model_len = ec.max_model_len or spec.max_positions
        with torch.cuda.device(self.device):
            self.runtime = Runtime(self.device, self.dtype, self.max_model_len)
        specs = model.cache_specs()
        probe = CacheManager(specs, ec.page_size, 1, ec.max_num_seqs, self.max_model_len)
        num_pages = self._choose_num_pages(probe)
        from pyre_amd.hip import ops

        with torch.cuda.device(self.device):
            self.cache = CacheManager(specs, ec.page_size, num_pages, ec.max_num_seqs, self.max_model_len,
                                      fill=ops.fill_rows, poison=ec.debug_poison)
            self.cache.materialize(self.device, self.dtype)
        # A captured step runs at rounded sizes: its rows may exceed max_num_seqs (49 requests
        # run as 64), its tables are a power of two of pages wide.
        seq_cap, width = round_decode_shape(ec.max_num_seqs, self.cache.max_pages_per_seq)
        self.step_arrays = model.step_arrays()
        self.meta = MetaBuffers(self.device, max(ec.max_num_batched_tokens, seq_cap), seq_cap,
                                [width for _ in self.cache.page_groups], self.step_arrays)
        self.steps_run = 0
        #: captured decode steps: (rows, table width) -> "warm" (ran eagerly once) or (graph, logits)
        self._graphs: dict[tuple[int, int], object] = {}
        self.graph_replays = 0
        if ec.tune_gemm_rows and self.dtype == torch.bfloat16:
            self.tune_library_gemms(ec.tune_gemm_rows)

    # ------------------------------------------------------------------ construction

    def _choose_num_pages(self, probe: CacheManager) -> int:
        ec = self.engine_config
        if ec.num_pages is not None:
            return ec.num_pages
        if ec.max_cached_tokens is not None:
            return max(1, -(-ec.max_cached_tokens // ec.page_size))
        per_page = probe.bytes_per_page(torch.empty((), dtype=self.dtype).element_size())
        if per_page == 0:
            return 1
        free, _ = torch.cuda.mem_get_info(self.device)
        want = int(free * ec.memory_fraction) // per_page
        # No request can use more than its longest length; no pool needs more than all of them.
        cap = ec.max_num_seqs * -(-self.max_model_len // ec.page_size)
        return max(1, min(want, cap))

    @classmethod
    def from_folder(cls, folder: str | Path, engine_config: EngineConfig | None = None) -> "Engine":
        """Model folder (config.json + *.safetensors) -> engine."""
        ec = engine_config or EngineConfig()
        config = load_config(folder)
        model = LayeredModel(get_architecture(config.architecture).build(config))
        tensors = load_weights(folder, model.tensor_specs(), torch.device(ec.device), TORCH_DTYPES[ec.dtype])
        return cls._finish(model, config, ec, tensors)

    @classmethod
    def from_state(cls, config: ModelConfig, state: dict[str, torch.Tensor],
                   engine_config: EngineConfig | None = None, consume: bool = False) -> "Engine":
        """Tensors already in memory (random weights made on the device, tests). ``consume``:
        ``state`` is emptied, so that the tensors which the parts copy (fused weights) are free
        as soon as they have been copied and not when the caller lets go of its dictionary."""
        ec = engine_config or EngineConfig()
        model = LayeredModel(get_architecture(config.architecture).build(config))
        tensors = adopt_state(state, model.tensor_specs(), torch.device(ec.device), TORCH_DTYPES[ec.dtype])
        if consume:
            state.clear()
        return cls._finish(model, config, ec, tensors)

    @classmethod
    def _finish(cls, model, config, ec, tensors) -> "Engine":
        with torch.cuda.device(torch.device(ec.device)):
            rt = Runtime(torch.device(ec.device), TORCH_DTYPES[ec.dtype], 0)
            model.bind(tensors, rt)  # takes the tensors out of the dictionary one by one
            return cls(model, config, ec)

    def tune_library_gemms(self, rows) -> int:
        """For steps of exactly ``rows`` tokens (any of them), let the BLAS front end
        time the vendor libraries' kernels for each distinct many-row 16-bit product of
        this model and remember the fastest (torch's TunableOp). Other row counts keep
        the libraries' own choice. Returns the number of products tuned."""
        import os
        import tempfile

        import torch.cuda.tunable as tunable

        from pyre_amd.parts.fast import SKINNY_MAX_ROWS

        shapes = {}
        for lin in self.model.linears():
            if lin.weight is not None and lin.weight.dtype == torch.bfloat16:
                shapes.setdefault((lin.out_features, lin.in_features), lin)
        tunable.enable(True)
        if hasattr(tunable, "write_file_on_exit"):
            tunable.write_file_on_exit(False)
        tunable.set_filename(os.path.join(tempfile.gettempdir(), f"pyre_amd_tunable_{os.getpid()}.csv"))
        tunable.set_max_tuning_duration(30)
        tunable.set_max_tuning_iterations(20)
        tunable.tuning_enable(True)
        tuned = 0
        try:
            with torch.cuda.device(self.device):
                for m in sorted({int(r) for r in rows if int(r) > SKINNY_MAX_ROWS}):
                    for (n_out, k), lin in shapes.items():
                        if n_out == self.vocab_size:
                            continue  # the head's float32 logits do not go through the library
                        x = torch.zeros(m, k, device=self.device, dtype=torch.bfloat16)
                        out = torch.empty(m, n_out, device=self.device, dtype=torch.bfloat16)
                        torch.mm(x, lin.weight.t(), out=out)
                        tuned += 1
                torch.cuda.synchronize()
        finally:
            tunable.tuning_enable(False)
        return tuned

    # ------------------------------------------------------------------ the step

    @property
    def vocab_size(self) -> int:
        return self.model.spec.vocab_size

    def has(self, rid) -> bool:
        return rid in self.cache

    def step(self, entries: list[Entry], fed_ids: torch.Tensor | None = None, tap=None) -> torch.Tensor | None:
        """Run one batch. Requests not seen before are admitted (a slot and empty
        block tables); pages for all the step's tokens are reserved first, lengths
        are committed afterwards. Returns float32 ``[sum(len(want)), vocab]`` on the
        device, rows in the order of the entries and of each ``want`` (None if no
        logits are wanted).

        The step is all or nothing: if it cannot be prepared (no pages, no slot, a token
        outside the vocabulary, a request named twice) the error is raised with every
        admission and reservation of this call undone, so that the caller sees the cache
        it had and may try again with another batch.

        The returned tensor is a view of scratch memory that belongs to the engine: the
        next ``step`` overwrites it (work put on the same stream before that, a sampler's
        kernels or a copy to the host, reads it in order and is safe). Copy it if it has
        to outlive the next step.

        An entry with ``feed = i`` takes its one token from ``fed_ids[i]`` (int32 on
        the device, for instance the ids a sampler has just written) when the step
        runs on the device: the host can put the step on the stream without waiting
        for the previous step's result.

        ``tap(pos, rows)``, a debugging aid, is called after every entry ``pos`` of the layer
        order with a copy of the hidden rows ``[tokens, hidden]`` (float32) as they stand there;
        such a step runs eagerly.
        """
        n_tokens = sum(len(e.tokens) for e in entries)
        ec = self.engine_config
        if n_tokens > ec.max_num_batched_tokens:
            raise ValueError(f"step of {n_tokens} tokens exceeds max_num_batched_tokens={ec.max_num_batched_tokens}")
        if len(entries) > ec.max_num_seqs:
            raise ValueError(f"step of {len(entries)} requests exceeds max_num_seqs={ec.max_num_seqs}")
        hb, graph_shape = prepare_step(entries, self.cache, self.vocab_size,
                                       GRAPH_MAX_ROWS if ec.use_graphs and tap is None else 0, fed_ids is not None)
        with torch.cuda.device(self.device):
            if graph_shape is not None:
                logits = self._step_captured(hb, *graph_shape, fed_ids)
            else:
                logits = self._run(hb, fed_ids, tap)
        for e in entries:
            self.cache.commit(e.rid, len(e.tokens))
        self.steps_run += 1
        return logits

    def _upload(self, hb, fed_ids, n_cap=None, s_cap=None):
        """The step's arrays to the device; tokens that are results still on the
        device are put in place there."""
        views = self.meta.upload(hb, n_cap, s_cap)
        if hb.feeds:
            from pyre_amd.hip import ops

            ops.feed_tokens(views["tokens"], views["token_src"], fed_ids, hb.n_tokens)
        return views

    def _context(self, hb, fed_ids=None, n_cap=None, s_cap=None):
        views = self._upload(hb, fed_ids, n_cap, s_cap)
        ctx = StepContext(
            runtime=self.runtime, host=hb, n_tokens=hb.n_tokens, n_seqs=hb.n_seqs,
            n_logits=len(hb.logit_rows), tokens=views["tokens"], positions=views["positions"],
            seq_of_token=views["seq_of_token"], logit_rows=views["logit_rows"][:len(hb.logit_rows)],
            q_start=views["q_start"], ctx_len=views["ctx_len"], state_slots=views["state_slots"],
            arrays={spec.name: views["x:" + spec.name] for spec in self.step_arrays})
        return ctx, self._layer_views(views)

    def _forward(self, ctx, caches, tap=None):
        """The model's kernels on torch's current stream, asked for once."""
        from pyre_amd.hip import ops

        ops.use_stream(torch.cuda.current_stream().cuda_stream)
        try:
            return self.model.forward(ctx, caches, tap) if tap is not None else self.model.forward(ctx, caches)
        finally:
            ops.use_stream(None)

    def _run(self, hb, fed_ids=None, tap=None):
        ctx, caches = self._context(hb.attach(self.step_arrays), fed_ids)
        return self._forward(ctx, caches, tap)

    def _step_captured(self, hb, rows: int, width: int, fed_ids=None):
        """A decode step at a fixed size (``rows`` requests, tables ``width`` pages
        wide): run eagerly the first time, captured in a HIP graph the second,
        replayed from then on. Only the metadata upload happens outside the graph."""
        live = hb.n_seqs
        key = (rows, width)
        padded = pad_decode_batch(hb, rows, self.cache.max_num_seqs, width * self.cache.page_size)
        padded.attach(self.step_arrays)
        state = self._graphs.get(key)
        if state is None:
            ctx, caches = self._context(padded, fed_ids)
            logits = self._forward(ctx, caches)
            self._graphs[key] = "warm"
            return logits[:live]
        if state == "warm":
            ctx, caches = self._context(padded, fed_ids)
            ws = self.runtime.workspace
            graph = torch.cuda.CUDAGraph()
            ws.frozen = True
            try:
                with torch.cuda.graph(graph):
                    logits = self._forward(ctx, caches)
            finally:
                ws.frozen = False
            ws.keep_replaced = True
            state = self._graphs[key] = (graph, logits)
        else:
            self._upload(padded, fed_ids)
        graph, logits = state
        graph.replay()
        self.graph_replays += 1
        return logits[:live]

    def _layer_views(self, views) -> list[list]:
        """For every entry of the layer order the views of its caches (or of the entry's whose
        caches it reads), in the order of the layer's descriptions."""
        cache = self.cache
        out = []
        for pos, call in enumerate(self.model.schedule):
            src = call.cache_from if call.cache_from is not None else pos
            mine = []
            for k in range(cache.caches_of_entry(src)):
                kind, gi = cache.group_of_cell[(src, k)]
                if kind == "paged":
                    g = cache.page_groups[gi]
                    li = g.layer_index(src, k)
                    mine.append(PagedLayerView({name: t[li] for name, t in g.tensors.items()}, views[f"table{gi}"],
                                               views[f"slots{gi}"], g.page_size, g.spec.window,
                                               writes=call.cache_from is None))
                else:
                    g = cache.state_groups[gi]
                    mine.append(StateLayerView(g.tensor[g.layer_index(src, k)], views["state_slots"]))
            out.append(mine)
        return out

    def finish(self, rid) -> None:
        """The request is over: its pages and its slot go back."""
        self.cache.free_request(rid)
