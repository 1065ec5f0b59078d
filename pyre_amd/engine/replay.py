"""Trace replay: feed given token ids through a model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives
:class:`~pyre_amd.engine.engine.Engine`, the object generation uses. The nearest
things in the reference are ``_chunked_vs_whole`` (`tests/test_cache.py:107-123`)
and `scripts/diagnose_parity.py`.

Input (stdin), one JSON object per line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step that wants logits, ``<out>/<step>.f32`` receives them as little-endian
float32 ``[wanted, vocab]``; after every step ``done <step>`` is printed.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

TOKEN_ROUNDING = 64


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page (a divisor of 64)")
    ap.add_argument("--max-seqs", type=int, default=8, help="most requests that are live at a time")
    ap.add_argument("--poison", action="store_true",
                    help="debugging aid: freed cache pages and state slots are filled with NaN")
    ap.add_argument("--graphs", action="store_true",
                    help="capture steps of single tokens in HIP graphs and replay them, as generation does "
                         "(the same kernels and the same bits either way)")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    if args.page_size <= 0 or TOKEN_ROUNDING % args.page_size:
        ap.error(f"--page-size must divide {TOKEN_ROUNDING}")

    def note(msg: str) -> None:
        print(f"[trace_run] {msg}", file=sys.stderr, flush=True)

    note("loading torch ...")
    import numpy as np
    import torch

    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.batch import Entry
    from pyre_amd.engine.engine import Engine
    from pyre_amd.hip import lib

    if not torch.cuda.is_available():
        note("no GPU visible: there is no CPU path")
        return 1
    note("preparing the kernel library ...")
    lib.lib()
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    max_tokens = -(-max(args.max_tokens, TOKEN_ROUNDING) // TOKEN_ROUNDING) * TOKEN_ROUNDING
    from pyre_amd.registry import get_architecture, load_config

    # the longest request: what the model's description says, or the pool if that is more
    config = load_config(args.model)
    model_limit = get_architecture(config.architecture).build(config).max_positions
    ec = EngineConfig(dtype=args.dtype, device=args.device, page_size=args.page_size,
                      max_cached_tokens=max_tokens, max_num_seqs=args.max_seqs,
                      max_model_len=max(model_limit, max_tokens),
                      max_num_batched_tokens=max(max_tokens, 4096), use_graphs=args.graphs, debug_poison=args.poison)
    note(f"loading {args.model} ({args.dtype}) ...")
    engine = Engine.from_folder(args.model, ec)
    note(f"ready: {engine.cache.page_groups[0].num_pages if engine.cache.page_groups else 0} pages of "
         f"{args.page_size} tokens")

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        step = msg["step"]
        entries = [Entry(e["id"], list(e["tokens"]), list(e.get("want", []))) for e in msg.get("entries", [])]
        if entries:
            logits = engine.step(entries)
            if logits is not None:
                arr = logits.to("cpu").numpy().astype("<f4", copy=False)
                arr.tofile(out_dir / f"{step}.f32")
            else:
                torch.cuda.synchronize(engine.device)
        for rid in msg.get("end", []):
            if engine.has(rid):
                engine.finish(rid)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
