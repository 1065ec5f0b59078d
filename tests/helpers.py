"""Helpers of the GPU tests: traces, their replay through the engine, comparison."""

from __future__ import annotations

import random

import torch

import plain_qwen2 as P

#: Bounds fixed before any run. float32 noise of the plain implementation itself is
#: ~5e-7 of the logit scale on the tiny shapes, 16-bit storage noise ~5e-3.
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


def depth_tol(dtype: str, layers: int) -> float:
    """The bound for a model of ``layers`` layers, fixed before any run of such a model: the
    bounds above are those of the tiny models (up to three layers); every layer adds rounding
    noise of its own, independent of the others', so the bound grows with the square root of
    the depth (28 layers: 3.1e-5 and 6.1e-2)."""
    return TOL[dtype] * max(1.0, (layers / 3) ** 0.5)


def layer_report(engine, plain, ids, rounding=None) -> list[tuple[int, float]]:
    """(entry of the layer order, max |hidden - plain hidden| / scale of the plain rows) for one
    request fed whole through ``engine`` (which must not know the request "__layers" yet), the
    way `scripts/diagnose_parity.py:103-120` of the reference walks its layers."""
    from pyre_amd.engine.batch import Entry

    cfg, w = plain
    _, hidden = P.forward(w, cfg, ids, rounding=rounding, return_hidden=True)
    seen = {}
    engine.step([Entry("__layers", list(ids), [])], tap=lambda pos, rows: seen.__setitem__(pos, rows.double().cpu()))
    engine.finish("__layers")
    out = []
    for pos, ref in enumerate(hidden):
        ref = ref.double().cpu()
        out.append((pos, float((seen[pos] - ref).abs().max() / ref.abs().max().clamp_min(1e-30))))
    return out


def first_layer_off(report, tol: float) -> str:
    """One line naming the first layer whose hidden rows leave ``tol``, and every layer's figure."""
    bad = next((f"first layer outside {tol:.1e}: {pos}" for pos, d in report if not d <= tol), f"no layer is outside {tol:.1e}")
    return bad + "; per layer: " + " ".join(f"{pos}:{d:.1e}" for pos, d in report)


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


def check_greedy(plain, prompt: list[int], tokens: list[int], tol: float) -> int:
    """Every generated token against the plain implementation's argmax given the tokens before
    it. A token may differ only where the plain logits leave the choice to rounding (the two
    within ``tol`` of the logit scale); returns how many did."""
    cfg, w = plain
    ids, near = list(prompt), 0
    for k, tok in enumerate(tokens):
        row = P.forward(w, cfg, ids)[-1]
        twin = int(row.argmax())
        if twin != tok:
            margin = float((row[twin] - row[tok]) / row.abs().max())
            assert margin < tol, f"token {k} is {tok}, the plain implementation gives {twin} (margin {margin:.2e})"
            near += 1
        ids.append(tok)
    return near
