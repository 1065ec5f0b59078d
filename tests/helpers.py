"""Helpers of the GPU tests: traces, their replay through the engine, comparison."""

from __future__ import annotations

import random

import torch

import plain_qwen2 as P

#: Bounds fixed before any run. float32 noise of the plain implementation itself is
#: ~5e-7 of the logit scale on the tiny shapes, 16-bit storage noise ~5e-3.
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


def random_ids(vocab: int, n: int, seed: int) -> list[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def make_engine(folder, dtype: str, **kw):
    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.engine import Engine

    args = dict(dtype=dtype, page_size=16, max_cached_tokens=1024, max_num_seqs=8,
                max_num_batched_tokens=1024, use_graphs=False)
    args.update(kw)
    return Engine.from_folder(folder, EngineConfig(**args))


def make_engine_from_state(config, state, dtype: str, **kw):
    """The same for tensors that are already on the device (shapes too large for a file)."""
    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.engine import Engine

    args = dict(dtype=dtype, page_size=16, max_cached_tokens=1024, max_num_seqs=8,
                max_num_batched_tokens=1024, use_graphs=False)
    args.update(kw)
    return Engine.from_state(config, dict(state), EngineConfig(**args))


def replay(engine, steps) -> dict:
    """steps: [(entries, end)] with entries = [(rid, tokens, want)].
    Returns {(rid, position): logits row (CPU float32)}."""
    from pyre_amd.engine.batch import Entry

    got = {}
    fed = {}
    for entries, end in steps:
        es = [Entry(r, list(t), list(w)) for r, t, w in entries]
        logits = engine.step(es)
        if logits is not None:
            rows = logits.float().cpu()
            i = 0
            for r, t, w in entries:
                base = fed.get(r, 0)
                for x in w:
                    got[(r, base + x)] = rows[i].clone()
                    i += 1
            assert i == rows.shape[0]
        for r, t, w in entries:
            fed[r] = fed.get(r, 0) + len(t)
        for r in end:
            engine.finish(r)
            fed.pop(r, None)
    return got


def plain_logits(plain, ids, rounding=None) -> torch.Tensor:
    cfg, w = plain
    return P.forward(w, cfg, ids, rounding=rounding).float().cpu()


def first_bad(got: dict, want: dict[object, torch.Tensor], tol: float):
    """Compare every (request, position) row; return a message naming the first
    position that is off (None if all are within ``tol`` of the logit scale)."""
    worst = 0.0
    for (rid, pos) in sorted(got, key=lambda k: (str(k[0]), k[1])):
        ref = want[rid][pos]
        scale = max(ref.abs().max().item(), 1e-6)
        d = (got[(rid, pos)] - ref).abs().max().item() / scale
        worst = max(worst, d)
        if not (d <= tol):
            return f"request {rid!r} position {pos}: max |diff| / scale = {d:.3e} > {tol:.1e}", worst
    return None, worst


def cut(n: int, sizes: list[int]) -> list[int]:
    """Portion lengths that sum to n, cycling through ``sizes``."""
    out, i = [], 0
    while n > 0:
        s = min(sizes[i % len(sizes)], n)
        if n - s == 1 and s > 2:  # leave no single-token rest in the ragged mode
            s -= 1
        out.append(s)
        n -= s
        i += 1
    return out
