"""Decode and prefill throughput of a Qwen2.5 shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--model qwen2.5-7b]
    python bench.py --workload serve [--model qwen2.5-1.5b] [--requests 256] [--max-batch 256]

A step is one decode step of the scheduler: every running request gets one new
token (plan, one engine step over the paged cache, greedy sampling, token fed
back). ``value`` is decoded tokens per second at ``--batch`` requests whose
context reaches ``--context`` at the last timed step. The same line carries the
prefill of a 2,048-token prompt, the decode step's memory roofline (of the published
peak and of the streaming-read bandwidth measured at the start), decode
throughput, step time and roofline at batch 1 and 64, the peak device memory
(`bench/harness.py:122`), the page pool's size, and where and when it ran
(device, ROCm and torch versions, git revision, time: `bench/harness.py:49-67`).
Nothing is timed before the engine has passed a check of its output (``gate``:
`bench/bench_pyre.py:69-74` refuses to measure an engine whose cached generation
differs from the naive one): a wrong or non-finite result ends the run with status 3.
Run without options that change the workload, the line also carries, under ``points``,
batch 8 at contexts of 16,384 and 32,768 tokens, a portion of 2,048 tokens after 30,720,
the Qwen2.5-1.5B and -32B shapes at batch 8 and the 1.5B serving workload.
Timing follows the reference's harness (`bench/harness.py:95-120`): fenced by device
synchronisation, warm-up first, the median of three timed blocks of ``--steps`` steps;
decode excludes prefill (`bench/harness.py:10-12`).

``--workload serve`` is continuous batching as in `bench/bench_batch.py:29-46` (one
scheduler run, all tokens over the wall clock): by default 256 requests on the
Qwen2.5-1.5B shape, prompt lengths log-uniform in [16, 2048], outputs uniform in
[16, 512], prompt portions of 512, contexts of at most 4,096, seeded.

Synthetic token ids (uniform over the vocabulary), random weights ~ N(0, 0.02): there is
no tokenizer and no checkpoint here.
"""

from __future__ import annotations

import argparse
import gc
import json
import random
import statistics
import sys
import time

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}  # dense, published
PREFILL_TOKENS = 2048


def model_numbers(cfg, n_layers: int, dtype_bytes: int):
    """Bytes a decode step must read and flops of a prefill, from the sizes alone."""
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    qd, kvd = cfg.q_dim, cfg.kv_dim
    per_layer = (qd + 2 * kvd) * H + (qd + 2 * kvd) + H * qd + 2 * I * H + H * I + 2 * H
    weight_bytes = (n_layers * per_layer + V * H + H) * dtype_bytes
    kv_bytes_per_token = 2 * n_layers * kvd * dtype_bytes

    def prefill_flops(t: int) -> float:
        linear = 2.0 * t * n_layers * ((qd + 2 * kvd) * H + H * qd + 3 * I * H)
        attn = n_layers * 4.0 * cfg.head_dim * cfg.num_attention_heads * t * (t + 1) / 2
        return linear + attn + 2.0 * V * H

    return weight_bytes, kv_bytes_per_token, prefill_flops


def environment() -> dict:
    """Where and when: device, library versions, the revision of this tree (git's, and a hash of
    the sources for trees that travel without their history)."""
    import datetime
    import hashlib
    import os
    import subprocess

    import torch

    root = os.path.dirname(os.path.abspath(__file__))
    try:
        sha = subprocess.run(["git", "rev-parse", "--short", "HEAD"], capture_output=True, text=True, timeout=10,
                             cwd=root).stdout.strip() or None
    except (OSError, subprocess.SubprocessError):
        sha = None
    digest = hashlib.sha1()
    for folder, _, files in sorted(os.walk(os.path.join(root, "pyre_amd"))):
        if "_build" in folder or "__pycache__" in folder:
            continue
        for f in sorted(files):
            if f.endswith((".py", ".hip", ".h")):
                digest.update(open(os.path.join(folder, f), "rb").read())
    digest.update(open(os.path.abspath(__file__), "rb").read())
    props = torch.cuda.get_device_properties(0)
    return {"device": props.name or torch.cuda.get_device_name(0), "arch": getattr(props, "gcnArchName", ""),
            "compute_units": props.multi_processor_count, "memory_gb": round(props.total_memory / 2**30, 1),
            "torch": torch.__version__, "rocm": torch.version.hip, "git": sha, "sources_sha1": digest.hexdigest()[:12],
            "time": datetime.datetime.now(datetime.timezone.utc).strftime("%Y-%m-%dT%H:%M:%SZ")}


def serve(args) -> dict:
    """Continuous batching of many requests of unequal lengths through the scheduler; returns
    the line of the record."""
    import math

    import torch

    from pyre_amd.api import Scheduler
    from pyre_amd.config import EngineConfig, preset
    from pyre_amd.engine.context import TORCH_DTYPES
    from pyre_amd.engine.engine import Engine
    from pyre_amd.weights import model_tensor_specs, random_state

    model = args.model or "qwen2.5-1.5b"
    cfg = preset(model)
    dev, max_context, chunk = "cuda:0", 4096, 512
    rng = random.Random(args.seed)
    prompts, outputs = [], []
    for _ in range(args.requests):
        n = int(round(math.exp(rng.uniform(math.log(16), math.log(2048)))))
        prompts.append([rng.randrange(cfg.vocab_size) for _ in range(n)])
        outputs.append(rng.randint(16, 512))
    t0 = time.perf_counter()
    budget = args.token_budget or 4 * chunk + args.max_batch
    ec = EngineConfig(dtype=args.dtype, device=dev, page_size=16, max_num_seqs=args.max_batch,
                      max_cached_tokens=args.max_batch * max_context, max_model_len=max_context,
                      max_num_batched_tokens=budget, prefill_chunk=chunk, use_graphs=not args.no_graphs,
                      tune_gemm_rows=())
    state = random_state(model_tensor_specs(cfg), 0, 0.02, 0.0, TORCH_DTYPES[ec.dtype], device=dev)
    engine = Engine.from_state(cfg, state, ec, consume=True)
    del state
    print(f"[bench] {model}: engine ready in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    checked = None if getattr(args, "no_gate", False) else gate(engine, cfg.vocab_size, args.dtype, cfg.num_hidden_layers, model)

    def run(n_requests: int) -> dict:
        sched = Scheduler(engine, max_batch=args.max_batch)
        for p, n in zip(prompts[:n_requests], outputs[:n_requests]):
            sched.add_request(p, max_new_tokens=n)
        replays0, captured_s, eager_s, captured, eager = engine.graph_replays, 0.0, 0.0, 0, 0
        torch.cuda.synchronize()
        t_start = t_note = time.perf_counter()
        while sched.has_work:
            before = engine.graph_replays
            t = time.perf_counter()
            sched.step()
            dt = time.perf_counter() - t
            if engine.graph_replays > before:
                captured, captured_s = captured + 1, captured_s + dt
            else:
                eager, eager_s = eager + 1, eager_s + dt
            if time.perf_counter() - t_note > 30:
                t_note = time.perf_counter()
                print(f"[bench] {len(sched.finished)} of {n_requests} requests done ...", file=sys.stderr, flush=True)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t_start
        gen = sum(len(r.generated) for r in sched.finished.values())
        assert len(sched.finished) == n_requests and engine.cache.page_groups[0].allocator.num_used == 0
        pre = sum(len(p) for p in prompts[:n_requests])
        return {"wall_s": round(wall, 3), "prompt_tokens": pre, "generated_tokens": gen,
                "total_tok_s": round((pre + gen) / wall, 1), "decode_tok_s": round(gen / wall, 1),
                "steps": captured + eager, "captured_steps": captured,
                "captured_share": round(captured / max(1, captured + eager), 4),
                "ms_per_captured_step": round(captured_s / max(1, captured) * 1e3, 3),
                "ms_per_uncaptured_step": round(eager_s / max(1, eager) * 1e3, 3),
                "preemptions": sum(r.preemptions for r in sched.finished.values()),
                "graph_replays": engine.graph_replays - replays0}

    run(min(args.requests, 2 * args.max_batch))      # warm-up: buffers grown, decode steps captured
    # What lives now (the interpreter's and torch's objects, the model, the captured steps) lives as
    # long as the process: out of the garbage collector's sight, as a server does after start-up. A
    # full collection in the middle of the run otherwise looks at all of it (46 ms once in 2 s).
    gc.collect()
    gc.freeze()
    res = run(args.requests)
    line = {
        "metric": "serving tok/s (%s shape, %d requests, continuous batching)" % (model, args.requests),
        "value": res["total_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": res["steps"], "warmup": 0,
        "ms_per_step": round(res["wall_s"] / res["steps"] * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic token ids, random weights N(0, 0.02) seed 0; prompts log-uniform [16, 2048], "
                "outputs uniform [16, 512], seed %d" % args.seed,
        "config": {"model": model, "requests": args.requests, "max_batch": args.max_batch, "prefill_chunk": chunk,
                   "max_num_batched_tokens": budget, "max_context": max_context, "page_size": 16,
                   "parallelism": "single GPU", "layers": cfg.num_hidden_layers, "hidden_size": cfg.hidden_size,
                   "intermediate_size": cfg.intermediate_size, "num_attention_heads": cfg.num_attention_heads,
                   "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "vocab_size": cfg.vocab_size, "graphs": bool(ec.use_graphs)},
        "serve": res, "gate": checked, "pool_pages": engine.cache.page_groups[0].num_pages,
        "peak_mem_gb": round(torch.cuda.max_memory_allocated() / 2**30, 2), "env": environment(),
    }
    return line


def gate_bounds(dtype: str, layers: int) -> float:
    """How far the logits of one position may lie apart, as a part of the row's largest logit,
    when the position is computed in two ways by an engine that is in order: rounding noise of
    the precision (1e-5 in 32-bit, 2e-2 in bfloat16 for models of up to three layers), growing
    with the square root of the depth as independent noise does."""
    return {"float32": 1e-5, "bfloat16": 2e-2}[dtype] * max(1.0, (layers / 3) ** 0.5)


def gate(engine, vocab: int, dtype: str, layers: int, tag: str) -> dict:
    """Refuse to time an engine whose output is wrong (`bench/bench_pyre.py:69-74` of the reference
    exits when its cached generation differs from the naive one, before it measures): a prompt
    of 40 tokens whole, then the same prompt as a portion of 24 tokens and 16 single tokens (the
    decode steps that are timed, captured in graphs if the engine captures); the logits must be
    finite and each position's two rows must agree within the precision's bound."""
    import torch

    from pyre_amd.engine.batch import Entry

    rng = random.Random(1234)
    ids = [rng.randrange(vocab) for _ in range(40)]
    whole = engine.step([Entry("gate", ids, list(range(40)))]).clone()
    engine.finish("gate")
    rows = [engine.step([Entry("gate", ids[:24], list(range(24)))]).clone()]
    for i in range(24, 40):
        rows.append(engine.step([Entry("gate", ids[i:i + 1], [0])]).clone())
    engine.finish("gate")
    cut = torch.cat(rows)
    finite = bool(torch.isfinite(whole).all() and torch.isfinite(cut).all())
    scale = whole.abs().amax(dim=1).clamp_min(1e-30)
    worst = float(((whole - cut).abs().amax(dim=1) / scale).max()) if finite else float("nan")
    spread = float(whole.std())
    bound = gate_bounds(dtype, layers)
    res = {"rows": 40, "max_diff": round(worst, 8), "bound": bound, "finite": finite, "logit_std": round(spread, 5)}
    print(f"[bench] gate {tag}: whole against portion + single tokens {res}", file=sys.stderr, flush=True)
    if not finite or not worst <= bound or not spread > 0:
        print(f"bench.py: the engine's logits are wrong ({tag}: {res}); nothing is timed")
        sys.exit(3)
    return res


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--model", default=None, help="preset shape (qwen2.5-7b; for --workload serve qwen2.5-1.5b)")
    ap.add_argument("--workload", default="decode", choices=["decode", "serve"])
    ap.add_argument("--requests", type=int, default=256, help="serve: number of requests")
    ap.add_argument("--max-batch", type=int, default=256, help="serve: requests that run at a time")
    ap.add_argument("--seed", type=int, default=0, help="serve: seed of the lengths and token ids")
    ap.add_argument("--token-budget", type=int, default=0,
                    help="serve: tokens in one step (0: four prompt portions beside a token of every running request)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the shape has")
    ap.add_argument("--points", default="1,64", help="further decode batch sizes ('' for none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--prefill-only", action="store_true", help="time the prefill alone (for profiling): no decode steps")
    ap.add_argument("--portion", type=int, default=0, metavar="TOKENS",
                    help="with --prefill-only: also time the last portion of this many tokens of a prompt of "
                         "--context tokens that is fed in such portions (chunked prefill late in a long context)")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--no-tune", action="store_true", help="keep the BLAS library's default kernels for prefill")
    ap.add_argument("--no-breakdown", action="store_true", help="no per-kernel times of the decode step in the line")
    ap.add_argument("--no-gate", action="store_true", help="skip the check of the engine's output before timing (profiling runs)")
    ap.add_argument("--extras", default="auto", choices=["auto", "on", "off"],
                    help="the further points of the default run: batch 8 at contexts of 16,384 and 32,768 tokens, a "
                         "portion of 2,048 tokens after 30,720, the 1.5B and 32B shapes at batch 8, the 1.5B serving "
                         "workload (auto: only when no other option changes the run)")
    ap.add_argument("--opt", action="append", default=[], metavar="KEY=VALUE",
                    help="engine runtime option (kernel choice ablations), e.g. skinny_gemm=0")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.workload == "serve":
        print(json.dumps(serve(args)))
        return 0
    plain_run = (args.model is None and args.batch == 8 and args.context == 4096 and args.points == "1,64" and args.dtype == "bfloat16"
                 and args.layers is None and not (args.no_prefill or args.prefill_only or args.no_graphs or args.opt))
    extras = args.extras == "on" or (args.extras == "auto" and plain_run)
    args.model = args.model or "qwen2.5-7b"

    import torch

    from pyre_amd.api import Scheduler
    from pyre_amd.config import EngineConfig, preset
    from pyre_amd.engine.batch import Entry
    from pyre_amd.engine.context import TORCH_DTYPES
    from pyre_amd.engine.engine import Engine
    from pyre_amd.hip import ops
    from pyre_amd.weights import model_tensor_specs, random_state

    dev = "cuda:0"
    dtype_bytes = 2 if args.dtype == "bfloat16" else 4
    measured_read = round(ops.read_bandwidth(dev), 1)
    print(f"[bench] streaming reads reach {measured_read} GB/s here (published peak {HBM_PEAK_GBS:.0f})", file=sys.stderr, flush=True)
    rng = random.Random(0)
    BLOCKS = 3

    def sync() -> None:
        torch.cuda.synchronize()

    def build(model: str, layers: int | None, max_batch: int, longest: int, cached_tokens: int, tune: bool):
        """An engine of ``model``'s shape with random weights, checked before anything is timed."""
        full = preset(model)
        n_layers = layers or full.num_hidden_layers
        cfg = preset(model, num_hidden_layers=n_layers)
        t0 = time.perf_counter()
        ec = EngineConfig(dtype=args.dtype, device=dev, page_size=16, max_num_seqs=max_batch,
                          max_cached_tokens=cached_tokens + 64 * 16, max_model_len=longest,
                          max_num_batched_tokens=PREFILL_TOKENS, prefill_chunk=PREFILL_TOKENS,
                          use_graphs=not args.no_graphs, tune_gemm_rows=(PREFILL_TOKENS,) if tune else ())
        state = random_state(model_tensor_specs(cfg), 0, 0.02, 0.0, TORCH_DTYPES[ec.dtype], device=dev)
        engine = Engine.from_state(cfg, state, ec, consume=True)
        for kv in args.opt:
            k, v = kv.split("=", 1)
            engine.runtime.options[k] = int(v)
        sync()
        print(f"[bench] {model}: engine ready in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
        checked = None if args.no_gate else gate(engine, cfg.vocab_size, args.dtype, n_layers, model)
        return engine, cfg, full, n_layers, checked

    PROFILED = 4  # decode steps under the profiler for the per-kernel breakdown

    def kernel_breakdown(sched) -> dict:
        """Microseconds per decode step of each kernel (the longest ten, by the part of their names
        that tells them apart), from the device's own trace of a few more steps of this run."""
        from torch.profiler import ProfilerActivity, profile

        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            for _ in range(PROFILED):
                sched.step()
            sync()
        rows = sorted(((e.key, e.device_time_total) for e in prof.key_averages() if e.device_time_total > 0), key=lambda r: -r[1])
        short = lambda k: k.replace("void ", "").replace("(anonymous namespace)::", "").split("(")[0][:48]  # noqa: E731
        out = {}
        for key, total in rows[:10]:
            out[short(key)] = round(out.get(short(key), 0.0) + total / PROFILED, 1)
        out["all kernels"] = round(sum(t for _, t in rows) / PROFILED, 1)
        return out

    def decode(engine, cfg, n_layers: int, batch: int, context: int, steps: int, warmup: int, breakdown: bool = False) -> dict:
        """Three timed blocks of `steps` decode steps at `batch`; the block of median time counts.
        The last block ends at the full context (`breakdown`: a few steps under the profiler follow)."""
        weight_bytes, kv_per_token, _ = model_numbers(cfg, n_layers, dtype_bytes)
        sched = Scheduler(engine, max_batch=batch)
        # Requests whose prompt is done decode while the others are still being
        # prefilled (one step per portion of a prompt), so leave room for those tokens too.
        portions = -(-context // PREFILL_TOKENS)
        start_ctx = context - (BLOCKS * steps + warmup) - portions * batch - 2 - (PROFILED if breakdown else 0)
        for _ in range(batch):
            sched.add_request([rng.randrange(cfg.vocab_size) for _ in range(start_ctx)], max_new_tokens=context - start_ctx)
        t_fill = time.perf_counter()
        while any(r.num_computed < len(r.prompt_ids) for r in sched.running + sched.waiting):
            sched.step()
            if time.perf_counter() - t_fill > 30:
                t_fill = time.perf_counter()
                print(f"[bench] filling caches for batch {batch} ...", file=sys.stderr, flush=True)
        for _ in range(warmup):
            sched.step()
        blocks = []
        for _ in range(BLOCKS):
            ctx0 = sum(r.num_computed for r in sched.running) / batch
            sync()
            t = time.perf_counter()
            for _ in range(steps):
                out = sched.step()
                assert len(out) == batch
            sync()
            blocks.append((time.perf_counter() - t, ctx0 + steps / 2))
        kernels = None
        if breakdown:
            try:
                kernels = kernel_breakdown(sched)
            except Exception as e:  # noqa: BLE001  (a profiler that is not there costs the run nothing)
                kernels = {"error": repr(e)[:120]}
        for r in list(sched.running):
            engine.finish(r.seq_id)
        dt, mean_ctx = sorted(blocks)[BLOCKS // 2]
        ms = dt / steps * 1e3
        achieved = (weight_bytes + batch * mean_ctx * kv_per_token) / (ms / 1e3) / 1e9
        return {"tok_s": batch * steps / dt, "ms": ms, "gbs": achieved, "frac": achieved / HBM_PEAK_GBS, "kernels": kernels}

    def prefill_of(engine, cfg, n_layers: int) -> dict:
        _, _, prefill_flops = model_numbers(cfg, n_layers, dtype_bytes)
        times = []
        for i in range(4):
            sched = Scheduler(engine, max_batch=1)
            sched.add_request([rng.randrange(cfg.vocab_size) for _ in range(PREFILL_TOKENS)], max_new_tokens=1)
            sync()
            t = time.perf_counter()
            sched.step()
            sync()
            if i:
                times.append(time.perf_counter() - t)
        ms = statistics.median(times) * 1e3
        fl = prefill_flops(PREFILL_TOKENS)
        return {"value": round(PREFILL_TOKENS / (ms / 1e3), 1), "tokens": PREFILL_TOKENS, "ms": round(ms, 3),
                "frac": round(fl / (ms / 1e3) / (MFMA_PEAK_TFLOPS[args.dtype] * 1e12), 4)}

    def portion_of(engine, cfg, context: int, tokens: int) -> dict:
        """A prompt of ``context`` tokens in portions of ``tokens``; the last three portions of the
        third pass are timed, the median counts (chunked prefill late in a long context)."""
        ids = [rng.randrange(cfg.vocab_size) for _ in range(context)]
        times = []
        for trial in range(3):
            cuts = list(range(0, context, tokens))
            for a in cuts:
                last = a + tokens >= context
                timed = trial == 2 and a in cuts[-3:]
                if timed:
                    sync()
                    t = time.perf_counter()
                engine.step([Entry("long", ids[a:a + tokens], [min(tokens, context - a) - 1] if last else [])])
                if timed:
                    sync()
                    times.append(time.perf_counter() - t)
            engine.finish("long")
        ms = statistics.median(times) * 1e3
        return {"context": context, "tokens": tokens, "ms": round(ms, 3), "value": round(tokens / (ms / 1e3), 1)}

    points = [int(p) for p in args.points.split(",") if p.strip()]
    max_batch = max([args.batch, *points])
    long_contexts = [16384, 32768] if extras else []
    longest = max([args.context, *long_contexts])
    cached = max([max_batch * args.context, *[args.batch * c for c in long_contexts]])
    engine, cfg, full, n_layers, checked = build(args.model, args.layers, max_batch, longest, cached, not args.no_tune)
    pool_pages = engine.cache.page_groups[0].num_pages

    prefill = None
    if not args.no_prefill:
        prefill = prefill_of(engine, cfg, n_layers)
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    if args.prefill_only:
        portion = portion_of(engine, cfg, args.context, args.portion) if args.portion else None
        print(json.dumps({"metric": "prefill tok/s (%s shape, %d tokens)" % (args.model, PREFILL_TOKENS),
                          "prefill": prefill, "portion": portion, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32"}))
        return 0
    main_point = decode(engine, cfg, n_layers, args.batch, args.context, args.steps, args.warmup, breakdown=not args.no_breakdown)
    value, ms_per_step, achieved = main_point["tok_s"], main_point["ms"], main_point["gbs"]
    pts, pts_ms, pts_frac = {}, {}, {}

    def note(name: str, pt: dict) -> None:
        pts[name], pts_ms[name], pts_frac[name] = round(pt["tok_s"], 1), round(pt["ms"], 4), round(pt["frac"], 4)
        print(f"[bench] {name} {pts[name]} tok/s, {pts_ms[name]} ms, {pts_frac[name]} of the HBM peak", file=sys.stderr, flush=True)

    for b in points:
        note(f"decode_b{b}", decode(engine, cfg, n_layers, b, args.context, args.steps, args.warmup))
    pts_ms[f"decode_b{args.batch}"], pts_frac[f"decode_b{args.batch}"] = round(ms_per_step, 4), round(achieved / HBM_PEAK_GBS, 4)

    # The further points of the default run. Each is a measurement of its own: one that cannot be
    # made (out of memory, an error) is named in `extras_failed` and costs the others nothing.
    failed, gates = {}, {args.model: checked}
    if extras:
        short = max(5, args.steps // 2)
        for c in long_contexts:
            try:
                note(f"decode_b{args.batch}_ctx{c}", decode(engine, cfg, n_layers, args.batch, c, short, args.warmup))
            except Exception as e:  # noqa: BLE001
                failed[f"decode_b{args.batch}_ctx{c}"] = repr(e)[:200]
        try:
            late = portion_of(engine, cfg, 32768, PREFILL_TOKENS)
            pts["prefill_2048_after_30720"], pts_ms["prefill_2048_after_30720"] = late["value"], late["ms"]
            print(f"[bench] portion late in a long prompt {late}", file=sys.stderr, flush=True)
        except Exception as e:  # noqa: BLE001
            failed["prefill_2048_after_30720"] = repr(e)[:200]
    peak_mem = {args.model: round(torch.cuda.max_memory_allocated() / 2**30, 2)}
    if extras:
        del engine
        gc.collect()
        torch.cuda.empty_cache()
        for other, context in (("qwen2.5-1.5b", 4096), ("qwen2.5-32b", 8192)):
            tag = other.replace("qwen2.5-", "qwen").replace(".", "p")
            try:
                torch.cuda.reset_peak_memory_stats()
                eng2, cfg2, _, layers2, gates[other] = build(other, None, args.batch, context, args.batch * context, False)
                note(f"{tag}_decode_b{args.batch}_ctx{context}", decode(eng2, cfg2, layers2, args.batch, context, args.steps, args.warmup))
                peak_mem[other] = round(torch.cuda.max_memory_allocated() / 2**30, 2)
                del eng2
            except Exception as e:  # noqa: BLE001
                failed[f"{tag}_decode_b{args.batch}"] = repr(e)[:200]
            gc.collect()
            torch.cuda.empty_cache()
        try:
            served = serve(argparse.Namespace(model=None, requests=256, max_batch=256, seed=0, token_budget=0,
                                              dtype=args.dtype, no_graphs=args.no_graphs))
            pts["qwen1p5b_serve_256_requests"] = served["value"]
            pts_ms["qwen1p5b_serve_256_requests_uncaptured_step"] = served["serve"]["ms_per_uncaptured_step"]
            pts_ms["qwen1p5b_serve_256_requests_captured_step"] = served["serve"]["ms_per_captured_step"]
        except Exception as e:  # noqa: BLE001
            failed["qwen1p5b_serve_256_requests"] = repr(e)[:200]

    line = {
        "metric": "decode tok/s (%s shape, batch %d, context %d)" % (args.model, args.batch, args.context),
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic token ids, random weights N(0, 0.02) seed 0",
        "config": {"model": args.model, "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single GPU", "layers": n_layers, "layers_of_shape": full.num_hidden_layers,
                   "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                   "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size, "page_size": 16,
                   "prefill_tokens": PREFILL_TOKENS, "graphs": not args.no_graphs,
                   "blas_tuned_rows": 0 if args.no_tune else PREFILL_TOKENS, "pool_pages": pool_pages,
                   "extra_points": "7B b8 at 16,384 and 32,768; 2,048 after 30,720; 1.5B and 32B b8; 1.5B serving" if extras else "none"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "frac_of_measured": round(achieved / measured_read, 4)},
        "points": pts, "points_ms_per_step": pts_ms, "points_hbm_frac": pts_frac,
        "kernels_us_per_step": main_point["kernels"], "measured_read_gbs": measured_read, "peak_mem_gb": peak_mem, "pool_pages": pool_pages,
        "gate": gates, "extras_failed": failed,
        "timing": "median of %d timed blocks of %d steps" % (BLOCKS, args.steps), "env": environment(),
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
