"""bin/trace_run as a user runs it: a subprocess, steps on stdin one at a time (the
next only after ``done <step>``), logits in <out>/<step>.f32."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from helpers import TOL, plain_logits, random_ids

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


def run_trace(model_dir, dtype, out_dir, max_tokens, steps, extra=()):
    proc = subprocess.Popen(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
         "--out", str(out_dir), "--max-tokens", str(max_tokens), *extra],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {st['step']}", line
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


@pytest.mark.parametrize("model,dtype,extra", [("tiny-a", "float32", ()), ("tiny-c", "bfloat16", ()), ("tiny-b", "bfloat16", ()),
                                               ("tiny-b", "float32", ("--page-size", "8", "--max-seqs", "3", "--poison"))])
def test_trace_run(model, dtype, extra, model_dirs, plain_models, tmp_path):
    plain = plain_models[model]
    vocab = plain[0]["vocab_size"]
    reqs = {"a": random_ids(vocab, 70, 1), "b": random_ids(vocab, 40, 2), "c": random_ids(vocab, 64, 3),
            "d": random_ids(vocab, 50, 4), "e": random_ids(vocab, 61, 5)}
    # five requests of <= 128 rounded tokens each, at most three live: 3 * 128 = 384 tokens of cache
    fed = {r: 0 for r in reqs}
    sizes = [13, 2, 30, 1, 7, 64, 3]
    live, waiting, steps, k = [], list(reqs), [], 0
    wanted = {}
    while live or waiting:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            n = min(sizes[k % len(sizes)], len(reqs[r]) - fed[r])
            k += 1
            want = [] if k % 5 == 0 else list(range(0, n, 2))
            entries.append({"id": r, "tokens": reqs[r][fed[r]:fed[r] + n], "want": want})
            wanted.setdefault(len(steps), []).extend((r, fed[r] + w) for w in want)
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [r for r in live if r not in end]
    steps.append({"step": len(steps), "entries": [], "end": []})          # an empty step is allowed
    out = tmp_path / "out"
    run_trace(model_dirs[model], dtype, out, 384, steps, extra)
    ref = {r: plain_logits(plain, ids, torch.bfloat16 if dtype == "bfloat16" else None) for r, ids in reqs.items()}
    checked = 0
    for st, rows in wanted.items():
        f = out / f"{st}.f32"
        if not rows:
            assert not f.exists()
            continue
        got = torch.from_numpy(np.fromfile(f, dtype="<f4").reshape(len(rows), vocab))
        for i, (r, pos) in enumerate(rows):
            scale = ref[r][pos].abs().max().item()
            d = (got[i] - ref[r][pos]).abs().max().item() / scale
            assert d <= TOL[dtype], f"step {st} request {r} position {pos}: {d:.3e}"
            checked += 1
    assert checked > 50
