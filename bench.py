"""Decode and prefill throughput of the Qwen2.5-7B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096]

A step is one decode step of the scheduler: every running request gets one new
token (plan, one engine step over the paged cache, greedy sampling, token fed
back). ``value`` is decoded tokens per second at ``--batch`` requests whose
context reaches ``--context`` at the last timed step. The same line carries the
prefill of a 2,048-token prompt, the decode step's memory roofline, and decode
throughput at batch 1 and 64. Timing follows the reference's harness
(`bench/harness.py:95-120`): fenced by device synchronisation, warm-up first;
decode excludes prefill (`bench/harness.py:10-12`). Synthetic token ids (uniform
over the vocabulary), random weights ~ N(0, 0.02): there is no tokenizer and no
checkpoint here.
"""

from __future__ import annotations

import argparse
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


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--model", default="qwen2.5-7b", help="preset shape")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the shape has")
    ap.add_argument("--points", default="1,64", help="further decode batch sizes ('' for none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--prefill-only", action="store_true", help="time the prefill alone (for profiling): no decode steps")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--no-tune", action="store_true", help="keep the BLAS library's default kernels for prefill")
    ap.add_argument("--opt", action="append", default=[], metavar="KEY=VALUE",
                    help="engine runtime option (kernel choice ablations), e.g. skinny_gemm=0")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    from pyre_amd.api import Scheduler
    from pyre_amd.config import EngineConfig, preset
    from pyre_amd.engine.context import TORCH_DTYPES
    from pyre_amd.engine.engine import Engine
    from pyre_amd.weights import model_tensor_specs, random_state

    full = preset(args.model)
    n_layers = args.layers or full.num_hidden_layers
    cfg = preset(args.model, num_hidden_layers=n_layers)
    points = [int(p) for p in args.points.split(",") if p.strip()]
    max_batch = max([args.batch, *points])
    dev = "cuda:0"
    t0 = time.perf_counter()
    ec = EngineConfig(dtype=args.dtype, device=dev, page_size=16, max_num_seqs=max_batch,
                      max_cached_tokens=max_batch * args.context + 64 * 16, max_model_len=args.context,
                      max_num_batched_tokens=PREFILL_TOKENS, prefill_chunk=PREFILL_TOKENS,
                      use_graphs=not args.no_graphs, tune_gemm_rows=() if args.no_tune else (PREFILL_TOKENS,))
    state = random_state(model_tensor_specs(cfg), 0, 0.02, 0.0, TORCH_DTYPES[ec.dtype], device=dev)
    engine = Engine.from_state(cfg, state, ec)
    del state
    for kv in args.opt:
        k, v = kv.split("=", 1)
        engine.runtime.options[k] = int(v)
    print(f"[bench] engine ready in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    dtype_bytes = 2 if args.dtype == "bfloat16" else 4
    weight_bytes, kv_per_token, prefill_flops = model_numbers(cfg, n_layers, dtype_bytes)
    rng = random.Random(0)

    def prompt(n: int) -> list[int]:
        return [rng.randrange(cfg.vocab_size) for _ in range(n)]

    def sync() -> None:
        torch.cuda.synchronize()

    def decode(batch: int, steps: int, warmup: int) -> tuple[float, float]:
        """(tokens per second, ms per step) of `steps` decode steps at `batch`."""
        sched = Scheduler(engine, max_batch=batch)
        # Requests whose prompt is done decode while the others are still being
        # prefilled (one step per portion of a prompt), so leave room for those tokens too.
        portions = -(-args.context // PREFILL_TOKENS)
        start_ctx = args.context - (steps + warmup) - portions * batch - 2
        for _ in range(batch):
            sched.add_request(prompt(start_ctx), max_new_tokens=args.context - start_ctx)
        t_fill = time.perf_counter()
        while any(r.num_computed < len(r.prompt_ids) for r in sched.running + sched.waiting):
            sched.step()
            if time.perf_counter() - t_fill > 30:
                t_fill = time.perf_counter()
                print(f"[bench] filling caches for batch {batch} ...", file=sys.stderr, flush=True)
        for _ in range(warmup):
            sched.step()
        sync()
        t = time.perf_counter()
        for _ in range(steps):
            out = sched.step()
            assert len(out) == batch
        sync()
        dt = time.perf_counter() - t
        for r in list(sched.running):
            engine.finish(r.seq_id)
        return batch * steps / dt, dt / steps * 1e3

    prefill = None
    if not args.no_prefill:
        times = []
        for i in range(4):
            sched = Scheduler(engine, max_batch=1)
            sched.add_request(prompt(PREFILL_TOKENS), max_new_tokens=1)
            sync()
            t = time.perf_counter()
            sched.step()
            sync()
            if i:
                times.append(time.perf_counter() - t)
        ms = statistics.median(times) * 1e3
        fl = prefill_flops(PREFILL_TOKENS)
        prefill = {"value": round(PREFILL_TOKENS / (ms / 1e3), 1), "tokens": PREFILL_TOKENS, "ms": round(ms, 3),
                   "frac": round(fl / (ms / 1e3) / (MFMA_PEAK_TFLOPS[args.dtype] * 1e12), 4)}
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    if args.prefill_only:
        print(json.dumps({"metric": "prefill tok/s (%s shape, %d tokens)" % (args.model, PREFILL_TOKENS),
                          "prefill": prefill, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32"}))
        return 0
    value, ms_per_step = decode(args.batch, args.steps, args.warmup)
    mean_ctx = args.context - args.steps / 2
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_per_token
    achieved = step_bytes / (ms_per_step / 1e3) / 1e9
    pts = {}
    for b in points:
        pts[f"decode_b{b}"] = round(decode(b, args.steps, args.warmup)[0], 1)
        print(f"[bench] decode_b{b} {pts[f'decode_b{b}']}", file=sys.stderr, flush=True)

    line = {
        "metric": "decode tok/s (Qwen2.5-7B shape, batch %d, context %d)" % (args.batch, args.context),
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic token ids, random weights N(0, 0.02) seed 0",
        "config": {"model": args.model, "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single GPU", "layers": n_layers, "layers_of_shape": full.num_hidden_layers,
                   "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                   "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size, "page_size": 16,
                   "prefill_tokens": PREFILL_TOKENS, "graphs": bool(ec.use_graphs),
                   "blas_tuned_rows": PREFILL_TOKENS if ec.tune_gemm_rows else 0},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": pts,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
