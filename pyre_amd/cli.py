"""Command line: generate from token ids with a model folder or a preset shape with
random weights. Option names follow the reference's scripts where it has them:
``--model --device --dtype`` (`scripts/serve.py:16-21`, `scripts/diagnose_parity.py:77-83`),
``--tokens`` / ``--max-new-tokens`` / ``--gen-len`` for the number of new tokens
(`scripts/diagnose_parity.py:82`, `bench/bench_pyre.py:55`, `bench/bench_batch.py:52`),
``--seed`` (`bench/bench_memory.py:36`), ``--out`` for a JSON result file. There is no
tokenizer: prompts are token ids."""

from __future__ import annotations

import argparse
import json
import random
import sys
import time


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="pyre_generate", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="model folder, or a preset name with --random-seed")
    ap.add_argument("--random-seed", type=int, default=None, help="draw random weights for a preset shape")
    ap.add_argument("--device", default="cuda")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--prompt-ids", action="append", default=[], metavar="I,J,K",
                    help="one prompt as comma-separated token ids (may be repeated)")
    ap.add_argument("--prompt-len", type=int, default=None, help="instead: random prompts of this length")
    ap.add_argument("--num-prompts", type=int, default=1)
    ap.add_argument("--max-new-tokens", "--tokens", "--gen-len", dest="max_new_tokens", type=int, default=16)
    ap.add_argument("--temperature", type=float, default=0.0, help="0: greedy")
    ap.add_argument("--seed", type=int, default=0, help="seed of sampling and of random prompts")
    ap.add_argument("--eos-id", type=int, default=None)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-blocks", type=int, default=None, help="cache pages (default: from free memory)")
    ap.add_argument("--max-batch", type=int, default=64, help="requests running at a time")
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048)
    ap.add_argument("--prefill-chunk", type=int, default=512)
    ap.add_argument("--max-model-len", type=int, default=None)
    ap.add_argument("--tune-gemm-rows", type=int, nargs="*", default=[],
                    help="step sizes for which the BLAS library's kernels are timed at start-up")
    ap.add_argument("--out", default=None, help="write a JSON result file")
    return ap


def main(argv: list[str] | None = None) -> int:
    args = build_parser().parse_args(argv)
    from pyre_amd.api import Scheduler, load_model

    engine, cfg = load_model(
        args.model, device=args.device, dtype=args.dtype, random_seed=args.random_seed,
        num_blocks=args.num_blocks, page_size=args.page_size, max_num_seqs=args.max_batch,
        max_num_batched_tokens=args.max_num_batched_tokens, prefill_chunk=args.prefill_chunk,
        max_model_len=args.max_model_len, tune_gemm_rows=tuple(args.tune_gemm_rows))
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    if args.prompt_len is not None:
        rng = random.Random(args.seed)
        prompts += [[rng.randrange(engine.vocab_size) for _ in range(args.prompt_len)]
                    for _ in range(args.num_prompts)]
    if not prompts:
        print("no prompt: give --prompt-ids or --prompt-len", file=sys.stderr)
        return 2
    sched = Scheduler(engine, max_batch=args.max_batch)
    ids = [sched.add_request(p, args.max_new_tokens, args.eos_id, args.temperature, args.seed) for p in prompts]
    t0 = time.perf_counter()
    results = sched.run()
    dt = time.perf_counter() - t0
    total = sum(len(results[i]) for i in ids)
    for i, p in zip(ids, prompts):
        print(f"request {i}: prompt of {len(p)} tokens -> {','.join(map(str, results[i]))}")
    print(f"{total} tokens in {dt:.3f} s ({total / dt:.1f} tok/s, {sched.steps} steps)", file=sys.stderr)
    if args.out:
        with open(args.out, "w") as f:
            json.dump({"model": args.model, "dtype": args.dtype, "prompts": prompts,
                       "generated": [results[i] for i in ids], "seconds": dt, "steps": sched.steps}, f)
    return 0


if __name__ == "__main__":
    sys.exit(main())
