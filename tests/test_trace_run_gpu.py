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

from helpers import TOL, cut, plain_logits, random_ids

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


def _check(out, wanted, ref, vocab, dtype):
    checked = 0
    for st, rows in wanted.items():
        got = torch.from_numpy(np.fromfile(out / f"{st}.f32", dtype="<f4").reshape(len(rows), vocab))
        for i, (r, pos) in enumerate(rows):
            scale = ref[r][pos].abs().max().item()
            d = (got[i] - ref[r][pos]).abs().max().item() / scale
            assert d <= TOL[dtype], f"step {st} request {r} position {pos}: {d:.3e}"
            checked += 1
    return checked


@pytest.mark.parametrize("mode,extra", [("whole", ()), ("tail", ()), ("tail", ("--graphs",)), ("ragged", ())])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_in_the_replay_modes(mode, extra, dtype, model_dirs, plain_models, tmp_path):
    """The program itself, with its own sizing of the cache from --max-tokens, through the modes
    that the engine is tested in: each request alone and whole; most of it in one step and the
    last 32 tokens one by one (also with those steps captured and replayed); portions of
    changing size down to two tokens. One request is live at a time and the pool holds just
    the longest (150 tokens rounded up to 192), so every request after the first gets pages that
    another one gave back."""
    plain = plain_models["tiny-c"]
    vocab = plain[0]["vocab_size"]
    reqs = {r: random_ids(vocab, n, seed=ord(r) + n) for r, n in (("a", 97), ("b", 64), ("c", 33), ("d", 150))}
    steps, wanted = [], {}

    def add(r, lo, n, want, end):
        wanted[len(steps)] = [(r, lo + w) for w in want]
        steps.append({"step": len(steps), "entries": [{"id": r, "tokens": reqs[r][lo:lo + n], "want": want}],
                      "end": [r] if end else []})

    for r, ids in reqs.items():
        n = len(ids)
        if mode == "whole":
            add(r, 0, n, list(range(n)), True)
        elif mode == "tail":
            add(r, 0, n - 32, [n - 33], False)
            for i in range(n - 32, n):
                add(r, i, 1, [0], i == n - 1)
        else:
            lo = 0
            for k in cut(n, [17, 5, 2, 32, 3, 2, 21]):
                add(r, lo, k, list(range(k)), lo + k == n)
                lo += k
    out = tmp_path / "out"
    run_trace(model_dirs["tiny-c"], dtype, out, 192, steps, extra)
    ref = {r: plain_logits(plain, ids, torch.bfloat16 if dtype == "bfloat16" else None) for r, ids in reqs.items()}
    checked = _check(out, wanted, ref, vocab, dtype)
    assert checked == (sum(len(i) for i in reqs.values()) if mode != "tail" else 33 * len(reqs))
