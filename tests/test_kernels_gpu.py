"""Each kernel alone against a plain torch reference of the same formula, at sizes
other than the engine's tiny models (odd widths, many heads, long contexts,
scrambled pages)."""

from __future__ import annotations

import math
import random

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _ops():
    from pyre_amd.hip import ops

    return ops


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


# ----------------------------------------------------------------------------- small kernels

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed(dtype):
    ops = _ops()
    table = rnd(301, 70, dtype=DT[dtype])
    ids = i32([5, 300, 0, 17, 5])
    out = torch.empty(5, 70, device=DEV)
    ops.embed(table, ids, out)
    assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [70, 1000, 3584])
def test_add_rmsnorm(dtype, hidden):
    ops = _ops()
    from pyre_amd.hip.ops import Partials

    n, eps = 7, 1e-5
    resid = rnd(n, hidden, seed=1)
    delta = rnd(3, n, hidden, seed=2)                      # three partial sums
    bias = rnd(hidden, seed=3)
    gain = rnd(hidden, seed=4, dtype=DT[dtype]) + 1
    out = torch.empty(n, hidden, device=DEV, dtype=DT[dtype])
    want_resid = resid.double() + delta.double().sum(0) + bias.double()
    want = want_resid * torch.rsqrt(want_resid.pow(2).mean(-1, keepdim=True) + eps) * gain.double()
    r = resid.clone()
    ops.add_rmsnorm(r, Partials(delta, bias), gain, eps, out)
    assert torch.allclose(r.double(), want_resid, atol=1e-5)
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert torch.allclose(out.double(), want, atol=tol, rtol=tol)
    # library special case: no delta, unit gain -> torch's rms_norm
    ones = torch.ones(hidden, device=DEV)
    o32 = torch.empty(n, hidden, device=DEV)
    ops.add_rmsnorm(resid.clone(), None, ones, eps, o32)
    assert torch.allclose(o32, torch.nn.functional.rms_norm(resid, (hidden,), eps=eps), atol=1e-5)
    # rows: only the listed rows, resid untouched
    rows = i32([6, 2])
    r2 = resid.clone()
    o2 = torch.empty(2, hidden, device=DEV, dtype=DT[dtype])
    ops.add_rmsnorm(r2, Partials(delta, bias), gain, eps, o2, rows=rows)
    assert torch.equal(r2, resid)
    assert torch.allclose(o2.double(), want[[6, 2]], atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [1028, 1536, 3584, 5120, 8192])
def test_add_rmsnorm_row_does_not_depend_on_row_count(dtype, hidden):
    """A wide row normed in a step of few rows (the 1024-thread form) and in a step of many
    (the 256-thread form) gives the same bits: the sum of squares is added in one order."""
    ops = _ops()
    from pyre_amd.hip.ops import Partials

    many, few, eps = 200, 5, 1e-6
    resid = rnd(many, hidden, seed=1, scale=3.0)
    delta = rnd(2, many, hidden, seed=2)
    gain = rnd(hidden, seed=4, dtype=DT[dtype]) + 1
    pick = [0, 77, 128, 150, 199][:few]
    out_many = torch.empty(many, hidden, device=DEV, dtype=DT[dtype])
    r_many = resid.clone()
    ops.add_rmsnorm(r_many, Partials(delta), gain, eps, out_many)
    r_few = resid[pick].clone()
    out_few = torch.empty(few, hidden, device=DEV, dtype=DT[dtype])
    ops.add_rmsnorm(r_few, Partials(delta[:, pick].contiguous()), gain, eps, out_few)
    assert torch.equal(r_few, r_many[pick])
    assert torch.equal(out_few, out_many[pick])
    # the final norm's gather form: few listed rows of a long residual, and many of them
    rows_few, rows_many = i32(pick), i32(list(range(many - 1, -1, -1)))
    g_few = torch.empty(few, hidden, device=DEV, dtype=DT[dtype])
    g_many = torch.empty(many, hidden, device=DEV, dtype=DT[dtype])
    ops.add_rmsnorm(resid.clone(), Partials(delta), gain, eps, g_few, rows=rows_few)
    ops.add_rmsnorm(resid.clone(), Partials(delta), gain, eps, g_many, rows=rows_many)
    assert torch.equal(g_few, out_many[pick])
    assert torch.equal(g_many, out_many.flip(0))


@pytest.mark.parametrize("adt,wdt", [("float32", "float32"), ("bfloat16", "bfloat16"), ("bfloat16", "float32")])
@pytest.mark.parametrize("m,n,k", [(1, 37, 50), (5, 130, 257), (77, 200, 64), (130, 65, 1000)])
def test_gemm_generic(adt, wdt, m, n, k):
    ops = _ops()
    a = rnd(m, k, dtype=DT[adt], seed=1)
    w = rnd(n, k, dtype=DT[wdt], seed=2)
    bias = rnd(n, seed=3)
    out = torch.empty(m, n, device=DEV)
    ops.gemm_generic(a, w, bias, out, m)
    want = a.double() @ w.double().T + bias.double()
    assert torch.allclose(out.double(), want, atol=1e-4 * math.sqrt(k), rtol=1e-5)
    # linearity in the input, and bias alone for a zero input
    out0 = torch.empty(m, n, device=DEV)
    ops.gemm_generic(torch.zeros_like(a), w, bias, out0, m)
    assert torch.allclose(out0, bias.expand(m, n))


@pytest.mark.parametrize("m,n,k", [(1, 37, 50), (5, 130, 257), (32, 128, 16), (33, 129, 17), (77, 200, 64), (130, 65, 1000),
                                   (300, 3584, 3584), (8, 1000, 18944), (20, 777, 3584), (64, 4608, 3584), (48, 96, 40),
                                   (33, 1000, 1100), (12, 300, 1024), (16, 4608, 3584), (9, 50, 96), (3, 3584, 3584),
                                   (17, 131, 3584)])
def test_gemm_f32_on_the_matrix_cores(m, n, k):
    """float32 in, float32 products and sums (the result is as close to a float64 product as
    plain float32 FMAs are), and a row's result bit for bit the same whatever rows share
    the call and wherever it lies among them."""
    ops = _ops()
    a = rnd(m, k, seed=1)
    w = rnd(n, k, seed=2)
    bias = rnd(n, seed=3)
    out = torch.full((m, n), float("nan"), device=DEV)
    ops.gemm_f32(a, w, bias, out, m)
    want = a.double() @ w.double().T + bias.double()
    assert torch.allclose(out.double(), want, atol=1e-4 * math.sqrt(k), rtol=1e-5)
    fma = torch.empty(m, n, device=DEV)
    ops.gemm_generic(a, w, bias, fma, m)
    err_mfma, err_fma = (out.double() - want).abs().max().item(), (fma.double() - want).abs().max().item()
    assert err_mfma <= 4 * err_fma + 1e-6, (err_mfma, err_fma)      # no reduced-precision mode
    # rows alone, in another order, in a strided view, without a bias: the same bits
    for rows in ([0], [m - 1], list(range(m - 1, -1, -1)), list(range(0, m, 3))):
        sub = a[rows].contiguous()
        o = torch.empty(len(rows), n, device=DEV)
        ops.gemm_f32(sub, w, bias, o, len(rows))
        assert torch.equal(o, out[rows]), rows
    wide = torch.zeros(m, k + 5, device=DEV)
    wide[:, 1:k + 1] = a                                            # rows that do not start on 16 bytes
    o = torch.empty(m, n, device=DEV)
    ops.gemm_f32(wide[:, 1:k + 1], w, None, o, m)
    assert torch.allclose(o + bias, out, atol=1e-6, rtol=1e-6)
    # linearity: a zero input gives the bias
    ops.gemm_f32(torch.zeros_like(a), w, bias, o, m)
    assert torch.equal(o, bias.expand(m, n))
    # k in parts: the parts add up to the product, the bias is in the first, no part is empty
    for ks in {2, 3, ops.gemm_f32_ksplit(n, k)}:
        kper = -(-(-(-k // ks)) // 16) * 16      # a part's length, as the kernel rounds it
        if (ks - 1) * kper >= k:
            continue
        parts = torch.full((ks, m, n), float("nan"), device=DEV)
        ops.gemm_f32(a, w, bias, parts if ks > 1 else parts[0], m, ks)
        assert torch.allclose(parts.double().sum(0), want, atol=1e-4 * math.sqrt(k), rtol=1e-5)
        one = torch.empty(ks, 1, n, device=DEV)
        ops.gemm_f32(a[m // 2:m // 2 + 1], w, bias, one if ks > 1 else one[0], 1, ks)
        assert torch.equal(one[:, 0], parts[:, m // 2])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_silu_mul(dtype):
    ops = _ops()
    from pyre_amd.hip.ops import Partials

    n, inter = 5, 176
    gu = rnd(2, n, 2 * inter, seed=5, scale=3.0)
    out = torch.empty(n, inter, device=DEV, dtype=DT[dtype])
    ops.silu_mul(Partials(gu), out, n)
    s = gu.double().sum(0)
    want = torch.nn.functional.silu(s[:, :inter]) * s[:, inter:]
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert torch.allclose(out.double(), want, atol=tol, rtol=tol)


@pytest.mark.parametrize("n,inter", [(129, 24), (300, 1544), (130, 20)])
def test_silu_mul_of_a_prompt_portion(n, inter):
    """bfloat16 in and out, one partial, many rows: the kernel with eight features per
    thread where the width allows it (24, 1544), the ordinary one where it does not (20)."""
    ops = _ops()
    from pyre_amd.hip.ops import Partials

    gu = rnd(1, n, 2 * inter, seed=6, scale=3.0).to(torch.bfloat16)
    out = torch.full((n, inter), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops.silu_mul(Partials(gu), out, n)
    s = gu[0].double()
    want = torch.nn.functional.silu(s[:, :inter]) * s[:, inter:]
    assert torch.allclose(out.double(), want, atol=2e-2, rtol=2e-2)


# ----------------------------------------------------------------------------- rotary + cache write

def rope_plain(x, pos, theta, rot):
    """x [n, heads, hd]; half-split rotation of the first `rot` elements (pyre/model.py:41-63)."""
    inv = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
    ang = torch.outer(pos.float(), inv)
    cos, sin = ang.cos().double()[:, None, :], ang.sin().double()[:, None, :]
    x = x.double().clone()
    a, b = x[..., :rot // 2].clone(), x[..., rot // 2:rot].clone()
    x[..., :rot // 2] = a * cos - b * sin
    x[..., rot // 2:rot] = b * cos + a * sin
    return x


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq,nkv,hd,rot,page", [(4, 2, 16, 16, 16), (6, 3, 12, 12, 8), (5, 1, 40, 24, 4), (28, 4, 128, 128, 16)])
def test_rope_kv_write(dtype, nq, nkv, hd, rot, page):
    ops = _ops()
    from pyre_amd.hip.ops import Partials
    from pyre_amd.parts.rotary import rotary_tables

    n, theta, npages = 9, 1e4, 12
    width = (nq + 2 * nkv) * hd
    qkv = rnd(2, n, width, seed=7)
    bias = rnd(width, seed=8)
    pos = torch.tensor([0, 1, 2, 40, 41, 7, 100, 3, 64])
    cos, sin = rotary_tables(rot, theta, 128)
    rng = random.Random(1)
    # every token in a page of its own (the tokens that a call writes into one page are a run of
    # consecutive slots: the run's last token zeroes the values behind it)
    slots = torch.tensor([p * page + rng.randrange(page) for p in rng.sample(range(npages), n)])
    slots[4] = -1                                           # this token is not stored
    q = torch.empty(n, nq * hd, device=DEV, dtype=DT[dtype])
    kc = torch.zeros(npages, nkv, page, hd, device=DEV, dtype=DT[dtype])
    vc = torch.zeros(npages, nkv, hd, page, device=DEV, dtype=DT[dtype])
    ops.rope_kv_write(Partials(qkv, bias), q, kc, vc, cos.to(DEV), sin.to(DEV), rot, i32(pos.tolist()),
                      i32(slots.tolist()), n, nq, nkv, hd, page)
    full = (qkv.double().sum(0) + bias.double()).cpu()
    wq = rope_plain(full[:, :nq * hd].view(n, nq, hd), pos, theta, rot)
    wk = rope_plain(full[:, nq * hd:(nq + nkv) * hd].view(n, nkv, hd), pos, theta, rot)
    wv = full[:, (nq + nkv) * hd:].view(n, nkv, hd)
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert torch.allclose(q.double().cpu().view(n, nq, hd), wq, atol=tol, rtol=tol)
    for t in range(n):
        s = int(slots[t])
        if s < 0:
            continue
        p, o = divmod(s, page)
        assert torch.allclose(kc[p, :, o, :].double().cpu(), wk[t], atol=tol, rtol=tol)
        assert torch.allclose(vc[p, :, :, o].double().cpu(), wv[t], atol=tol, rtol=tol)
    # nothing else was written: everything outside the used slots is still zero
    used = {int(s) for s in slots if s >= 0}
    for s in range(npages * page):
        if s not in used:
            p, o = divmod(s, page)
            assert not kc[p, :, o, :].any() and not vc[p, :, :, o].any()
    # position 0 is the identity
    assert torch.allclose(q.double().cpu().view(n, nq, hd)[0], full[0, :nq * hd].view(nq, hd), atol=tol, rtol=tol)


# ----------------------------------------------------------------------------- attention

def paged_case(ctx_lens, q_lens, nq, nkv, hd, page, dtype, seed=0, table_extra=2):
    """Random requests whose keys and values lie in scrambled pages.
    Returns the kernel's inputs and, per request, dense K/V and queries."""
    rng = random.Random(seed)
    S = len(ctx_lens)
    npages_each = [-(-c // page) for c in ctx_lens]
    total = sum(npages_each) + 5
    order = list(range(total))
    rng.shuffle(order)
    width = max(8, -(-max(npages_each) // 8) * 8) + table_extra
    table = torch.full((S, width), -1, dtype=torch.int32)

    def cpu(*shape, seed):
        return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)).to(dtype)

    kc = cpu(total, nkv, page, hd, seed=seed + 1)                 # stale values everywhere
    vc = cpu(total, nkv, hd, page, seed=seed + 2)
    dense, qs, positions, seq_of = [], [], [], []
    it = iter(order)
    for s in range(S):
        pages = [next(it) for _ in range(npages_each[s])]
        table[s, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
        K = cpu(ctx_lens[s], nkv, hd, seed=seed + 10 + s)
        V = cpu(ctx_lens[s], nkv, hd, seed=seed + 50 + s)
        for t in range(ctx_lens[s]):
            kc[pages[t // page], :, t % page, :] = K[t]
            vc[pages[t // page], :, :, t % page] = V[t]
        dense.append((K, V))
        ql = q_lens[s]
        qs.append(cpu(ql, nq, hd, seed=seed + 90 + s))
        positions += list(range(ctx_lens[s] - ql, ctx_lens[s]))
        seq_of += [s] * ql
    q = torch.cat(qs).contiguous().to(DEV)
    return q, kc.to(DEV), vc.to(DEV), table.to(DEV), i32(positions), i32(seq_of), dense, qs


def attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window=0):
    """softmax(q k^T scale) v per request and head in float64 (pyre/model.py:109-123)."""
    outs = []
    for s, (K, V) in enumerate(dense):
        ql, T = q_lens[s], ctx_lens[s]
        q = qs[s].double().transpose(0, 1)                        # nq, ql, hd
        k = K.double().transpose(0, 1).repeat_interleave(nq // nkv, 0)
        v = V.double().transpose(0, 1).repeat_interleave(nq // nkv, 0)
        sc = q @ k.transpose(-1, -2) * scale
        qpos = torch.arange(T - ql, T, device=sc.device)[:, None]
        kpos = torch.arange(T, device=sc.device)[None, :]
        hide = kpos > qpos
        if window:
            hide = hide | (kpos < qpos - window + 1)
        sc = sc.masked_fill(hide, -math.inf)
        outs.append((torch.softmax(sc, -1) @ v).transpose(0, 1))   # ql, nq, hd
    return torch.cat(outs)


GENERIC_SHAPES = [(4, 2, 16, 16), (8, 2, 12, 8), (4, 2, 10, 6), (3, 1, 20, 5), (6, 6, 40, 4), (28, 4, 128, 16), (5, 1, 256, 32)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq,nkv,hd,page", GENERIC_SHAPES)
@pytest.mark.parametrize("window", [0, 37])
def test_attn_generic(dtype, nq, nkv, hd, page, window):
    ops = _ops()
    ctx_lens, q_lens = [1, 33, 300, 1500, 64], [1, 5, 1, 40, 64]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, DT[dtype])
    out = torch.empty_like(q)
    scale = hd ** -0.5
    ops.attn_generic(q, out, kc, vc, pos, seq_of, table, q.shape[0], nq, nkv, hd, page, scale, window)
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window)
    tol = 2e-5 if dtype == "float32" else 2e-2
    assert torch.allclose(out.double().cpu(), want, atol=tol, rtol=tol)
    if window == 0:
        # one visible key: the output is exactly that key's value (request 0)
        assert torch.allclose(out[0].double().cpu(), dense[0][1][0].double().repeat_interleave(nq // nkv, 0), atol=tol)
    if dtype == "float32":
        # one block per head, with plain multiply-adds, whatever the sizes
        alone = torch.empty_like(q)
        ops.attn_generic(q, alone, kc, vc, pos, seq_of, table, q.shape[0], nq, nkv, hd, page, scale, window,
                         matrix_cores=False)
        assert torch.allclose(alone.double().cpu(), want, atol=tol, rtol=tol)


@pytest.mark.parametrize("nq,nkv,hd,page", [(28, 4, 128, 16), (40, 8, 128, 64), (12, 2, 128, 32), (9, 1, 64, 48), (18, 1, 48, 16),
                                            (5, 5, 80, 16), (7, 7, 16, 32), (8, 2, 112, 16), (3, 3, 32, 4), (6, 2, 12, 8),
                                            (20, 2, 256, 16)])
@pytest.mark.parametrize("window", [0, 300, 77])
def test_attn_of_single_tokens_by_groups_of_heads_in_float32(nq, nkv, hd, page, window):
    """The 32-bit path's attention of single tokens: one block serves the query heads that share
    a key/value head (up to 16; 18 heads take two blocks) from one read of its keys and values, on
    the matrix cores' float32 instruction where the sizes allow (head sizes 16 to 128 in steps of 16,
    pages of a multiple of 16), for contexts of one span and of many, with and without a list of
    tokens, with released pages of a window, with spans that start anywhere (a window of 77). The
    result for a token does not depend on what else the call holds, bit for bit."""
    ops = _ops()
    ctx_lens = [1, 127, 128, 129, 700, 2049, 33, 16, 17]
    q_lens = [1] * len(ctx_lens)
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.float32, seed=31)
    if window:                                              # pages that the window has passed are released
        for s, c in enumerate(ctx_lens):
            table[s, :max(0, (c - window) // page)] = -1
    n, scale = q.shape[0], hd ** -0.5
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window)
    out = torch.full_like(q, float("nan"))
    ops.attn_generic(q, out, kc, vc, pos, seq_of, table, n, nq, nkv, hd, page, scale, window)
    assert torch.allclose(out.double().cpu(), want, atol=2e-5, rtol=2e-5)
    some = [6, 0, 4]
    part = torch.full_like(q, float("nan"))
    ops.attn_generic(q, part, kc, vc, pos, seq_of, table, len(some), nq, nkv, hd, page, scale, window, tokens=i32(some))
    assert torch.equal(part[some], out[some]) and torch.isnan(part[1]).all()


def test_attn_of_single_tokens_in_float32_finds_one_key_among_thousands():
    """One key of 3,000 fits the query, at a place that is no multiple of anything; its value is the
    output. Then that key lies just outside a window, and the output is far from its value."""
    ops = _ops()
    nq, nkv, hd, page = 14, 2, 128, 16
    ctx_lens, q_lens = [3000], [1]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.float32, seed=3)
    K, V = dense[0]                                          # [T, nkv, hd]
    at = 1717
    for h in range(nkv):                                     # make key `at` of every key/value head point along its queries
        for rep in range(nq // nkv):
            qs[0][0, h * (nq // nkv) + rep] = K[at, h] * 40.0
    q = qs[0].to(DEV).contiguous()                           # [1, nq, hd]
    out = torch.full_like(q, float("nan"))
    ops.attn_generic(q, out, kc, vc, pos, seq_of, table, 1, nq, nkv, hd, page, 1.0)
    near = V[at].repeat_interleave(nq // nkv, 0)
    assert torch.allclose(out[0].cpu(), near, atol=1e-4)
    window = 3000 - 1 - at                                   # the keys at + 1 .. 2999
    ops.attn_generic(q, out, kc, vc, pos, seq_of, table, 1, nq, nkv, hd, page, 1.0, window)
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, 1.0, window)
    assert torch.allclose(out.double().cpu(), want, atol=2e-5, rtol=2e-5)
    assert (out[0].cpu() - near).abs().max() > 0.1


@pytest.mark.parametrize("listed", [False, True])
def test_attn_generic_in_several_launches_and_with_given_scratch(monkeypatch, listed):
    """Spans of keys leave partial results in scratch memory; a call whose scratch would pass the
    limit of one launch goes out in several, with the same bits."""
    ops = _ops()
    nq, nkv, hd, page, window = 6, 2, 40, 8, 0
    ctx_lens, q_lens = [700, 1300, 30], [9, 1, 30]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.float32, seed=5)
    n, scale = q.shape[0], hd ** -0.5
    some = list(range(0, n, 3)) if listed else None
    count = len(some) if listed else n
    tokens = i32(some) if listed else None
    ref = torch.zeros_like(q)
    ops.attn_generic(q, ref, kc, vc, pos, seq_of, table, count, nq, nkv, hd, page, scale, window, tokens=tokens)
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window)
    rows = some if listed else list(range(n))
    assert torch.allclose(ref.double().cpu()[rows], want[rows], atol=2e-5, rtol=2e-5)
    from pyre_amd.hip.lib import lib

    spans = lib().pyre_attn_generic_spans(table.shape[1] * page)
    assert spans > 1
    monkeypatch.setattr(ops, "ATTN_GENERIC_SCRATCH", 7 * nq * spans * (hd + 2))   # seven tokens a launch
    need = ops.attn_generic_scratch(count, nq, hd, table.shape[1], page, window)
    assert need == 7 * nq * spans * (hd + 2)
    out = torch.zeros_like(q)
    scratch = torch.full((need + 3,), float("nan"), device=DEV)
    ops.attn_generic(q, out, kc, vc, pos, seq_of, table, count, nq, nkv, hd, page, scale, window, tokens=tokens,
                     scratch=scratch)
    assert torch.equal(out, ref)
    assert torch.isnan(scratch[need:]).all()
    with pytest.raises(Exception, match="scratch"):
        ops.attn_generic(q, out, kc, vc, pos, seq_of, table, count, nq, nkv, hd, page, scale, window, tokens=tokens,
                         scratch=scratch[:need - 1])


MFMA_SHAPES = [(28, 4, 128, 16), (8, 8, 64, 16), (6, 1, 32, 32), (40, 2, 96, 16), (3, 1, 256, 48), (4, 2, 64, 48)]


@pytest.mark.parametrize("nq,nkv,hd,page", MFMA_SHAPES)
@pytest.mark.parametrize("window", [0, 50])
@pytest.mark.parametrize("size", [None, 5, 100])
def test_attn_decode_mfma(nq, nkv, hd, page, window, size):
    ops = _ops()
    assert ops.attn_mfma_supports(hd, page, nq, nkv)
    ctx_lens = [1, 31, 32, 33, 700, 2049]
    q_lens = [1] * len(ctx_lens)
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.bfloat16, seed=3)
    n = q.shape[0]
    out = torch.full_like(q, float("nan"))
    scale = hd ** -0.5
    decode_attention(ops, q, out, kc, vc, range(n), pos, seq_of, table, nq, nkv, hd, page, scale, window, size=size)
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window)
    assert torch.allclose(out.double().cpu(), want, atol=2e-2, rtol=2e-2)


def decode_attention(ops, q, out, kc, vc, tokens, pos, seq_of, table, nq, nkv, hd, page, scale, window=0, size=None,
                     rows=None, alone=None):
    """The decode kernel on the single tokens ``tokens`` with a list planned as the engine plans it."""
    from pyre_amd.parts.attention_work import decode_alone, decode_capacity, decode_items, decode_work

    tokens = np.asarray(tokens, dtype=np.int32)
    rows = rows or len(tokens)
    work = decode_work(tokens, pos.cpu().numpy(), rows, window, nq, nkv, size=size)
    cap, items = max(decode_capacity(rows, nq, nkv), int(work[0, 0])), decode_items(nq, nkv)
    acc = torch.full((cap * items * 16 * hd,), float("nan"), device=DEV)
    ml = torch.full((cap * items * 32,), float("nan"), device=DEV)
    counters = torch.zeros(cap * items, dtype=torch.int32, device=DEV)
    alone = decode_alone(rows, nq, nkv) if alone is None else alone
    ops.attn_decode_work_bf16(q, out, kc, vc, work_on_device(work, cap, pos, seq_of), cap, pos, seq_of, table, acc, ml, counters,
                              alone, nq, nkv, hd, page, scale, window)
    assert int(counters.abs().sum()) == 0
    return work


def work_on_device(work, cap, pos, seq_of, fill=0):
    """The list as the kernel reads it (each row with its token's position and table row behind
    it), in a buffer as large as the launch: the rows past its end are never read."""
    from pyre_amd.parts.attention_work import decode_work_with_places

    wide = decode_work_with_places(work, pos.cpu().numpy(), seq_of.cpu().numpy())
    flat = np.full(8 * (1 + cap), fill, dtype=np.int32)
    flat[:wide.size] = wide.reshape(-1)
    return i32(flat.tolist())


@pytest.mark.parametrize("nq,nkv,hd,page", [(28, 4, 128, 16), (12, 2, 128, 64), (8, 2, 64, 16), (6, 3, 32, 32), (16, 1, 96, 48)])
@pytest.mark.parametrize("ks,bias,window,size,alone", [(7, True, 0, None, True), (1, False, 0, 4, False), (3, True, 50, None, False)])
def test_attn_decode_finishes_the_qkv_product_itself(nq, nkv, hd, page, ks, bias, window, size, alone):
    """A step of single tokens: the decode kernel given the q/k/v product's partial sums (sum, bias,
    rotation, the cache write and the zeroes behind the new value are its own work) against the
    kernel that does these and the decode kernel after it: the same bits in the result and in both
    caches. Requests of very different lengths, one of them not stored (no slot), pages that hold
    NaN where nothing was written, contexts that end anywhere in a page."""
    ops = _ops()
    from pyre_amd.hip.ops import Partials
    from pyre_amd.parts.attention_work import decode_alone, decode_capacity, decode_items, decode_work
    from pyre_amd.parts.rotary import rotary_tables

    ctx_lens = [1, 31, 32, 33, 700, 2049, 129, 5, 64]
    q_lens = [1] * len(ctx_lens)
    _, kc, vc, table, pos, seq_of, dense, _ = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.bfloat16, seed=9)
    n, scale, width = len(ctx_lens), hd ** -0.5, (nq + 2 * nkv) * hd
    tab = table.cpu()
    slots = [int(tab[s, (c - 1) // page]) * page + (c - 1) % page for s, c in enumerate(ctx_lens)]
    slots[3] = -1                                            # a token that is not stored
    for s, c in enumerate(ctx_lens):                         # the last key's place and what follows it: not written yet
        last = int(tab[s, (c - 1) // page])
        kc[last, :, (c - 1) % page:, :] = float("nan")
        vc[last, :, :, (c - 1) % page:] = float("nan")
    if slots[3] < 0:                                         # its key is read all the same: leave it finite
        last = int(tab[3, (ctx_lens[3] - 1) // page])
        kc[last, :, (ctx_lens[3] - 1) % page, :] = 0.25
        vc[last, :, :, (ctx_lens[3] - 1) % page:] = 0.5
    parts = Partials(rnd(ks, n, width, seed=12, scale=0.7), rnd(width, seed=13) if bias else None)
    cos, sin = (t.to(DEV).contiguous() for t in rotary_tables(hd, 1e4, max(ctx_lens) + 1))
    slots_d = i32(slots)
    # the two kernels
    k1, v1 = kc.clone(), vc.clone()
    q = torch.empty(n, nq * hd, device=DEV, dtype=torch.bfloat16)
    ops.rope_kv_write(parts, q, k1, v1, cos, sin, hd, pos, slots_d, n, nq, nkv, hd, page)
    want = torch.full((n, nq, hd), float("nan"), device=DEV, dtype=torch.bfloat16)
    decode_attention(ops, q.view(n, nq, hd), want, k1, v1, list(range(n)), pos, seq_of, table, nq, nkv, hd, page, scale,
                     window, size=size, alone=alone)
    assert torch.isfinite(want.float()).all()
    # the one
    k2, v2 = kc.clone(), vc.clone()
    work = decode_work(np.arange(n, dtype=np.int32), pos.cpu().numpy(), n, window, nq, nkv, size=size)
    cap, items = max(decode_capacity(n, nq, nkv), int(work[0, 0])), decode_items(nq, nkv)
    acc = torch.full((cap * items * 16 * hd,), float("nan"), device=DEV)
    ml = torch.full((cap * items * 32,), float("nan"), device=DEV)
    counters = torch.zeros(cap * items, dtype=torch.int32, device=DEV)
    got = torch.full((n, nq, hd), float("nan"), device=DEV, dtype=torch.bfloat16)
    for _ in range(2):                                       # the second call writes what is there already
        ops.attn_decode_work_rope_bf16(parts, cos, sin, slots_d, got, k2, v2, True, work_on_device(work, cap, pos, seq_of), cap, pos,
                                       seq_of, table, acc, ml, counters, decode_alone(n, nq, nkv) if alone is None else alone,
                                       nq, nkv, hd, page, scale, window)
        assert int(counters.abs().sum()) == 0
        assert torch.equal(got, want)
        assert torch.equal(k1.view(torch.int16), k2.view(torch.int16)) and torch.equal(v1.view(torch.int16), v2.view(torch.int16))
    # a layer that keeps no keys and values of its own: the caches stay as they are
    k3, v3 = k1.clone(), v1.clone()
    ops.attn_decode_work_rope_bf16(parts, cos, sin, slots_d, got, k3, v3, False, work_on_device(work, cap, pos, seq_of), cap, pos,
                                   seq_of, table, acc, ml, counters, True, nq, nkv, hd, page, scale, window)
    assert torch.equal(got, want) and torch.equal(k3.view(torch.int16), k1.view(torch.int16))


@pytest.mark.parametrize("nq,nkv,hd,page", MFMA_SHAPES)
@pytest.mark.parametrize("window", [0, 50])
@pytest.mark.parametrize("size,alone", [(None, True), (4, False), (12, True), (None, False)])
def test_attn_decode_from_a_work_list(nq, nkv, hd, page, window, size, alone):
    """Requests of very different lengths, their keys dealt to blocks by the planner (or
    4 or 12 chunks per block: the longest requests then span many blocks that join
    through memory). The second call finds the counters as the first left them; the third
    plans for a larger step, as a captured one would, and must give the same bits."""
    ops = _ops()
    from pyre_amd.parts.attention_work import decode_capacity, decode_items, decode_work

    ctx_lens = [1, 31, 32, 33, 700, 2049, 129, 5]
    q_lens = [1] * len(ctx_lens)
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.bfloat16, seed=3)
    n, scale = q.shape[0], hd ** -0.5
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window)
    rows = 8
    cap, items = decode_capacity(rows, nq, nkv), decode_items(nq, nkv)
    if size is not None:
        cap = 600
    acc = torch.full((cap * items * 16 * hd,), float("nan"), device=DEV)
    ml = torch.full((cap * items * 32,), float("nan"), device=DEV)
    counters = torch.zeros(cap * items, dtype=torch.int32, device=DEV)
    tokens = np.arange(n, dtype=np.int32)
    work = decode_work(tokens, pos.cpu().numpy(), rows, window, nq, nkv, size=size)
    assert work[0, 0] <= cap
    if size is not None and window == 0:
        assert work[1, 1] // 65536 > 4                            # the longest request spans many blocks
    outs = []
    for _ in range(2):
        out = torch.full_like(q, float("nan"))
        ops.attn_decode_work_bf16(q, out, kc, vc, work_on_device(work, cap, pos, seq_of), cap, pos, seq_of, table, acc, ml,
                                  counters, alone, nq, nkv, hd, page, scale, window)
        assert torch.allclose(out.double().cpu(), want, atol=2e-2, rtol=2e-2)
        assert int(counters.abs().sum()) == 0
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    # what lies past the list's end is not followed
    out = torch.full_like(q, float("nan"))
    ops.attn_decode_work_bf16(q, out, kc, vc, work_on_device(work, cap, pos, seq_of, fill=-7), cap, pos, seq_of, table, acc, ml,
                              counters, alone, nq, nkv, hd, page, scale, window)
    assert torch.equal(out, outs[0])


def test_attn_decode_work_list_in_a_mixed_batch():
    """Single tokens between the tokens of prompt portions: the list names them by their
    place in the flat batch, and nothing else is written."""
    ops = _ops()
    from pyre_amd.parts.attention_work import decode_capacity, decode_items, decode_work

    nq, nkv, hd, page = 28, 4, 128, 16
    ctx_lens, q_lens = [300, 40, 1500, 64, 9], [1, 7, 1, 33, 1]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.bfloat16, seed=8)
    scale = hd ** -0.5
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale)
    singles = np.asarray([0, 8, 42], dtype=np.int32)
    cap, items = decode_capacity(4, nq, nkv), decode_items(nq, nkv)
    work = decode_work(singles, pos.cpu().numpy(), 4, 0, nq, nkv)
    acc = torch.empty(cap * items * 16 * hd, device=DEV)
    ml = torch.empty(cap * items * 32, device=DEV)
    counters = torch.zeros(cap * items, dtype=torch.int32, device=DEV)
    out = torch.full_like(q, 7.0)
    ops.attn_decode_work_bf16(q, out, kc, vc, work_on_device(work, cap, pos, seq_of), cap, pos, seq_of, table, acc, ml, counters,
                              True, nq, nkv, hd, page, scale)
    got = out.double().cpu()
    assert torch.allclose(got[singles.tolist()], want[singles.tolist()], atol=2e-2, rtol=2e-2)
    others = [i for i in range(q.shape[0]) if i not in singles.tolist()]
    assert (got[others] == 7.0).all()


def prefill_attention(ops, q, out, kc, vc, tiles, pos, seq_of, table, nq, nkv, hd, page, scale, window=0, size=None):
    """Prompt portions through the kernel for the head size: from a work list planned as the
    engine plans it (or with blocks of ``size`` chunks of 64 keys) for heads of up to 128
    elements, from the tiles themselves for larger ones. Returns the work list, if any."""
    from pyre_amd.parts.attention_work import prefill_items, prefill_slots, prefill_work

    tiles = np.asarray(tiles, dtype=np.int32).reshape(-1, 2)
    if hd > 128:
        ops.attn_prefill_bf16(q, out, kc, vc, i32(tiles.reshape(-1).tolist()), len(tiles), pos, seq_of, table,
                              nq, nkv, hd, page, scale, window)
        return None
    items = prefill_items(nq, nkv)
    work = prefill_work(tiles, pos.cpu().numpy(), window, items, size=size)
    n_slots = prefill_slots(work)
    per_slot = items * ops.attn_prefill_waves(nq, nkv)
    partials = torch.full((max(1, n_slots) * per_slot * (hd // 32 * 1024 + 128),), float("nan"), device=DEV)
    counters = torch.zeros(max(1, n_slots) * per_slot, dtype=torch.int32, device=DEV)
    ops.attn_prefill_work_bf16(q, out, kc, vc, i32(work.reshape(-1).tolist()), len(work), partials, counters, n_slots,
                               pos, seq_of, table, nq, nkv, hd, page, scale, window)
    assert int(counters.abs().sum()) == 0
    return work


# heads of more than 128 elements have one form, without a work list
PREFILL_CASES = [(*shape, size) for shape in MFMA_SHAPES for size in (None, 3, 1) if size is None or shape[2] <= 128]


@pytest.mark.parametrize("nq,nkv,hd,page,size", PREFILL_CASES)
@pytest.mark.parametrize("window", [0, 50, 300])
def test_attn_prefill_mfma(nq, nkv, hd, page, window, size):
    """Prompt portions of several requests. Blocks of one or three chunks of 64 keys deal the
    tiles of the longer requests to many blocks, whose partial results join through memory."""
    ops = _ops()
    from pyre_amd.parts.attention import TILE

    ctx_lens, q_lens = [2, 40, 97, 700, 1100], [2, 40, 33, 3, 600]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.bfloat16, seed=4)
    tiles, base = [], 0
    for ql in q_lens:
        tiles += [(t0, min(TILE, base + ql - t0)) for t0 in range(base, base + ql, TILE)]
        base += ql
    scale = hd ** -0.5
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window)
    outs = []
    for _ in range(2):                                              # the second call finds the counters as the first left them
        out = torch.full_like(q, float("nan"))
        work = prefill_attention(ops, q, out, kc, vc, tiles, pos, seq_of, table, nq, nkv, hd, page, scale, window, size)
        assert torch.allclose(out.double().cpu(), want, atol=2e-2, rtol=2e-2)
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    if size is not None and window == 0:
        assert work[:, 6].max() >= 6                                # the long request's tiles span many blocks


@pytest.mark.parametrize("seed", range(6))
def test_attention_work_lists_on_random_batches(seed):
    """Random numbers of requests with random contexts, windows and head counts, some with a
    portion of their prompt and some with a single token, through both MFMA kernels with the
    lists the planner makes for them: every row against the plain attention."""
    ops = _ops()
    rng = random.Random(100 + seed)
    nkv = rng.choice([1, 2, 4])
    nq = nkv * rng.choice([1, 3, 7, 8])
    hd, page = rng.choice([(64, 16), (128, 16), (128, 32), (32, 48), (96, 16)])
    window = rng.choice([0, 0, 200])
    n_req = rng.randrange(1, 24)
    ctx_lens, q_lens = [], []
    for _ in range(n_req):
        ctx = int(math.exp(rng.uniform(0, math.log(2500)))) + 1
        ql = 1 if rng.random() < 0.6 else rng.randrange(2, min(ctx, 130) + 1)
        ctx_lens.append(max(ctx, ql))
        q_lens.append(ql)
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.bfloat16, seed=seed)
    scale = hd ** -0.5
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window)
    out = torch.full_like(q, float("nan"))
    singles, tiles, base = [], [], 0
    for ql in q_lens:
        if ql == 1:
            singles.append(base)
        else:
            tiles += [(t0, min(32, base + ql - t0)) for t0 in range(base, base + ql, 32)]
        base += ql
    if singles:
        decode_attention(ops, q, out, kc, vc, singles, pos, seq_of, table, nq, nkv, hd, page, scale, window,
                         rows=len(singles) + rng.randrange(0, 5))
    if tiles:
        prefill_attention(ops, q, out, kc, vc, tiles, pos, seq_of, table, nq, nkv, hd, page, scale, window)
    assert torch.allclose(out.double().cpu(), want, atol=2e-2, rtol=2e-2), (nq, nkv, hd, page, window, ctx_lens, q_lens)


def test_attn_prefill_of_a_portion_late_in_a_long_context():
    """64 tokens at the end of 6,000: two tiles, which the planner deals to as many blocks as
    the chip has units; the result is that of undivided tiles up to rounding."""
    ops = _ops()
    nq, nkv, hd, page = 28, 4, 128, 16
    ctx_lens, q_lens = [6000], [64]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.bfloat16, seed=21)
    scale = hd ** -0.5
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale)
    out = torch.full_like(q, float("nan"))
    work = prefill_attention(ops, q, out, kc, vc, [(0, 32), (32, 32)], pos, seq_of, table, nq, nkv, hd, page, scale)
    assert len(work) >= 8 and work[:, 6].min() > 1
    assert torch.allclose(out.double().cpu(), want, atol=2e-2, rtol=2e-2)
    whole = torch.full_like(q, float("nan"))
    prefill_attention(ops, q, whole, kc, vc, [(0, 32), (32, 32)], pos, seq_of, table, nq, nkv, hd, page, scale, size=10 ** 6)
    assert torch.allclose(out.float(), whole.float(), atol=1e-2, rtol=2e-2)


@pytest.mark.parametrize("nq,nkv,hd,page", GENERIC_SHAPES + [(3, 1, 10, 8), (7, 1, 72, 16), (12, 2, 128, 48)])
@pytest.mark.parametrize("window", [0, 37])
def test_attn_prefill_f32_on_the_matrix_cores(nq, nkv, hd, page, window):
    """Prompt portions in true float32: any head size and page size, scrambled pages, windows;
    as close to a float64 result as the one-block-per-token kernel is; a token's result bit for
    bit the same however its request's tokens are cut into tiles; NaN in pages that the
    request does not hold changes nothing; generic kernel for listed single tokens."""
    ops = _ops()
    ctx_lens, q_lens = [2, 40, 97, 700, 1100], [2, 40, 33, 3, 600]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, torch.float32, seed=6)
    held = set(table[table >= 0].tolist())
    for p in range(kc.shape[0]):
        if p not in held:
            kc[p], vc[p] = float("nan"), float("nan")
    scale = hd ** -0.5
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale, window)
    ref = torch.empty_like(q)
    ops.attn_generic(q, ref, kc, vc, pos, seq_of, table, q.shape[0], nq, nkv, hd, page, scale, window)
    outs = []
    for width in (32, 7, 19):                                    # tiles of up to `width` tokens
        tiles, base = [], 0
        for ql in q_lens:
            tiles += [(t0, min(width, base + ql - t0)) for t0 in range(base, base + ql, width)]
            base += ql
        tiles.append((0, 0))                                     # an empty tile does nothing
        out = torch.full_like(q, float("nan"))
        ops.attn_prefill_f32(q, out, kc, vc, i32(tiles).view(-1), len(tiles), pos, seq_of, table, nq, nkv, hd, page, scale, window)
        assert torch.allclose(out.double().cpu(), want, atol=2e-5, rtol=2e-5)
        outs.append(out)
    err, err_ref = (outs[0].double().cpu() - want).abs().max().item(), (ref.double().cpu() - want).abs().max().item()
    assert err <= 4 * err_ref + 1e-6, (err, err_ref)              # no reduced-precision mode
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    # a list of tokens for the one-by-one kernel: only those rows are written
    some = [0, 5, 41, q.shape[0] - 1]
    part = torch.full_like(q, float("nan"))
    ops.attn_generic(q, part, kc, vc, pos, seq_of, table, len(some), nq, nkv, hd, page, scale, window, tokens=i32(some))
    assert torch.equal(part[some], ref[some]) and torch.isnan(part[1]).all()


@pytest.mark.parametrize("kernel", ["generic32", "generic16", "decode", "prefill", "prefill32"])
def test_attention_finds_a_far_key(kernel):
    """Random scores would hide a key that is skipped or misplaced: make one far
    key (at a page's first slot, deep in a long context) dominate and check that
    the output is its value."""
    ops = _ops()
    nq, nkv, hd, page = 8, 2, 64, 16
    dt = torch.float32 if kernel in ("generic32", "plain32", "prefill32") else torch.bfloat16
    ctx_lens, q_lens = [900], [1 if not kernel.startswith("prefill") else 34]
    for target in (0, 16 * 20, 16 * 20 + 15, 899 - 34):
        q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, dt, seed=9)
        K, V = dense[0]
        # all queries point along e0; the target key has a large e0 component
        q.zero_()
        q[:, :, 0] = 8.0
        pages = table[0].tolist()
        kc[pages[target // page], :, target % page, :] = 0
        kc[pages[target // page], :, target % page, 0] = 60.0
        out = torch.empty_like(q)
        n = q.shape[0]
        scale = hd ** -0.5
        if kernel.startswith("generic"):
            ops.attn_generic(q, out, kc, vc, pos, seq_of, table, n, nq, nkv, hd, page, scale, 0)
        elif kernel == "decode":
            decode_attention(ops, q, out, kc, vc, [0], pos, seq_of, table, nq, nkv, hd, page, scale)
        elif kernel == "prefill32":
            ops.attn_prefill_f32(q, out, kc, vc, i32([0, 32, 32, 2]), 2, pos, seq_of, table, nq, nkv, hd, page, scale, 0)
        else:
            prefill_attention(ops, q, out, kc, vc, [(0, 32), (32, 2)], pos, seq_of, table, nq, nkv, hd, page, scale)
        want = V[target].double().repeat_interleave(nq // nkv, 0)      # nq, hd
        assert torch.allclose(out.double().cpu(), want.expand(n, nq, hd), atol=3e-2), (kernel, target)


@pytest.mark.parametrize("kernel", ["generic32", "generic16", "decode", "prefill", "prefill32"])
def test_attention_at_a_windows_edge(kernel):
    """A window of 100 keys: the oldest key that a query still sees dominates its scores, so
    the output is that key's value; the key just before it dominates even more and must not
    be seen at all (an off-by-one at the window's edge would return its value instead)."""
    ops = _ops()
    nq, nkv, hd, page, window = 8, 2, 64, 16, 100
    dt = torch.float32 if kernel in ("generic32", "plain32", "prefill32") else torch.bfloat16
    ql = 34 if kernel.startswith("prefill") else 1
    ctx_lens, q_lens = [700], [ql]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, dt, seed=13)
    K, V = dense[0]
    q.zero_()
    q[:, :, 0] = 8.0
    pages = table[0].tolist()
    last = 699
    edge = last - window + 1            # the oldest key the last query sees; the queries before it see it too
    for key, weight in ((edge, 40.0), (edge - ql, 90.0)):      # the second one lies before every query's window
        kc[pages[key // page], :, key % page, :] = 0
        kc[pages[key // page], :, key % page, 0] = weight
    out = torch.empty_like(q)
    n, scale = q.shape[0], hd ** -0.5
    if kernel.startswith("generic"):
        ops.attn_generic(q, out, kc, vc, pos, seq_of, table, n, nq, nkv, hd, page, scale, window)
    elif kernel == "decode":
        decode_attention(ops, q, out, kc, vc, [0], pos, seq_of, table, nq, nkv, hd, page, scale, window)
    elif kernel == "prefill32":
        ops.attn_prefill_f32(q, out, kc, vc, i32([0, 32, 32, 2]), 2, pos, seq_of, table, nq, nkv, hd, page, scale, window)
    else:
        prefill_attention(ops, q, out, kc, vc, [(0, 32), (32, 2)], pos, seq_of, table, nq, nkv, hd, page, scale, window)
    want = V[edge].double().repeat_interleave(nq // nkv, 0)
    assert torch.allclose(out.double().cpu(), want.expand(n, nq, hd), atol=3e-2), kernel
    # one position on, the edge key itself has left the last query's window: the output is a mixture again
    if ql == 1:
        pos2 = pos + 1
        full = torch.cat([K, torch.zeros(1, nkv, hd, dtype=K.dtype)])
        kc[pages[(last + 1) // page], :, (last + 1) % page, :] = 0
        out2 = torch.empty_like(q)
        if kernel.startswith("generic"):
            ops.attn_generic(q, out2, kc, vc, pos2, seq_of, table, n, nq, nkv, hd, page, scale, window)
        else:
            decode_attention(ops, q, out2, kc, vc, [0], pos2, seq_of, table, nq, nkv, hd, page, scale, window)
        assert not torch.allclose(out2.double().cpu(), want.expand(n, nq, hd), atol=0.2)


@pytest.mark.parametrize("kernel", ["generic32", "plain32", "generic16", "decode", "decode256", "prefill", "prefill256", "prefill32"])
@pytest.mark.parametrize("ctx_len", [700, 689, 655])
def test_attention_ignores_what_a_page_held_before(kernel, ctx_len):
    """A request's last page is only partly its own: the slots past its last key still hold what
    the page's previous owner wrote, which may be NaN or Inf (a request that diverged). The
    kernels on the matrix cores load whole chunks and weight the hidden keys with 0, and 0 * NaN
    is NaN: so the kernel that writes a step's keys and values zeroes the values behind the last
    token it writes into a page. Every page starts as NaN (keys) and Inf (values) here; the
    requests' keys and values go in through that kernel in two steps (all but the last tokens,
    then the last tokens of both requests side by side); then attention. Contexts that end 4,
    15 and 1 keys before the end of a 16-key page."""
    ops = _ops()
    from pyre_amd.hip.ops import Partials

    big = kernel.endswith("256")
    nq, nkv, hd, page = (4, 2, 256, 16) if big else (8, 2, 64, 16)
    dt = torch.float32 if kernel in ("generic32", "plain32", "prefill32") else torch.bfloat16
    ql = 34 if kernel.startswith("prefill") else 1
    ctx_lens, q_lens = [ctx_len, 40], [ql, min(ql, 3)]
    q, kc, vc, table, pos, seq_of, dense, qs = paged_case(ctx_lens, q_lens, nq, nkv, hd, page, dt, seed=17)
    kc.fill_(float("nan"))
    vc.fill_(float("inf"))
    tab = table.cpu()

    def write(spans):
        """The tokens [a, b) of each request (request, a, b), in one call of the writing kernel."""
        rows, positions, slots = [], [], []
        for s, a, b in spans:
            K, V = dense[s]
            rows.append(torch.cat([torch.zeros(b - a, nq * hd), K[a:b].reshape(b - a, -1).float(),
                                   V[a:b].reshape(b - a, -1).float()], dim=1))
            positions += list(range(a, b))
            slots += [int(tab[s, t // page]) * page + t % page for t in range(a, b)]
        qkv = Partials(torch.cat(rows).to(DEV).unsqueeze(0).contiguous())
        n = len(positions)
        ops.rope_kv_write(qkv, torch.empty(n, nq * hd, device=DEV, dtype=dt), kc, vc, None, None, 0, i32(positions),
                          i32(slots), n, nq, nkv, hd, page)

    write([(0, 0, ctx_lens[0] - q_lens[0])])
    write([(1, 0, ctx_lens[1] - q_lens[1])])
    write([(0, ctx_lens[0] - q_lens[0], ctx_lens[0]), (1, ctx_lens[1] - q_lens[1], ctx_lens[1])])
    for s, c in enumerate(ctx_lens):                        # what the writer left: its values, then zeros; keys untouched
        last = int(tab[s, (c - 1) // page])
        if c % page:
            assert (vc[last, :, :, c % page:] == 0).all() and torch.isnan(kc[last, :, c % page:, :]).all()
        assert torch.equal(vc[last, :, :, (c - 1) % page].cpu(), dense[s][1][c - 1].to(dt))
    scale = hd ** -0.5
    want = attention_plain(qs, dense, ctx_lens, q_lens, nq, nkv, scale)
    out = torch.zeros_like(q)
    n = q.shape[0]
    tiles = [(0, 32), (32, 2), (34, 3)]
    if kernel.startswith("generic") or kernel == "plain32":   # float32: on the matrix cores, or one block per head
        ops.attn_generic(q, out, kc, vc, pos, seq_of, table, n, nq, nkv, hd, page, scale, 0,
                         matrix_cores=kernel != "plain32")
    elif kernel.startswith("decode"):
        decode_attention(ops, q, out, kc, vc, [0, 1], pos, seq_of, table, nq, nkv, hd, page, scale)
    elif kernel == "prefill32":
        ops.attn_prefill_f32(q, out, kc, vc, i32([t for tile in tiles for t in tile]), 3, pos, seq_of, table, nq, nkv, hd, page, scale, 0)
    else:
        prefill_attention(ops, q, out, kc, vc, tiles, pos, seq_of, table, nq, nkv, hd, page, scale)
    assert torch.isfinite(out.float()).all(), kernel
    tol = 2e-5 if dt == torch.float32 else 2e-2
    assert torch.allclose(out.double().cpu(), want, atol=tol, rtol=tol), kernel


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page,hd", [(16, 128), (8, 12), (5, 40), (6, 10), (32, 64)])
def test_the_writer_zeroes_the_values_behind_a_steps_last_token(dtype, page, hd):
    """Page sizes and head sizes of the vectorised and of the general writing kernel: three
    requests in one step (one run that ends mid-page, one that ends exactly at a page's end, one
    single token that starts a page); of every page only the slots after the run's last token
    are zeroed, nothing that an earlier step wrote and nothing of other pages."""
    ops = _ops()
    from pyre_amd.hip.ops import Partials

    nq, nkv, dt = 2, 2, DT[dtype]
    pages = 6
    kc = torch.full((pages, nkv, page, hd), 7.0, device=DEV, dtype=dt)
    vc = torch.full((pages, nkv, hd, page), 7.0, device=DEV, dtype=dt)
    # request a: slots 2 .. page + 1 of pages (0, 1): its run ends at slot 1 of page 1; request b: the
    # whole of page 2; request c: slot 0 of page 3; page 4 belongs to nobody
    runs = [[2 + i for i in range(page)], [2 * page + i for i in range(page)], [3 * page]]
    slots = [s for r in runs for s in r]
    n = len(slots)
    vals = rnd(n, (nq + 2 * nkv) * hd, seed=3)
    ops.rope_kv_write(Partials(vals.to(DEV).unsqueeze(0).contiguous()), torch.empty(n, nq * hd, device=DEV, dtype=dt), kc, vc,
                      None, None, 0, i32(list(range(n))), i32(slots), n, nq, nkv, hd, page)
    v = vals.cpu()[:, (nq + nkv) * hd:].view(n, nkv, hd).to(dt)
    got = vc.cpu()
    for i, s in enumerate(slots):
        assert torch.equal(got[s // page, :, :, s % page], v[i]), (i, s)
    assert (got[0, :, :, :2] == 7.0).all()                              # before the run: as it was
    assert (got[1, :, :, 2:] == 0).all()                                # behind the run's end in its last page
    assert (got[3, :, :, 1:] == 0).all() and (got[4] == 7.0).all() and (got[5] == 7.0).all()
    assert (kc.cpu()[1, :, 2:, :] == 7.0).all()                         # keys need no zeroing: their scores are masked


# ----------------------------------------------------------------------------- sampling

def test_argmax_first_of_equals():
    ops = _ops()
    logits = rnd(6, 1001, seed=11)
    logits[2, 700] = 50.0
    logits[2, 30] = 50.0        # tie: the lower index wins, as torch.argmax
    logits[3, 1000] = 99.0
    out = torch.zeros(6, dtype=torch.int32, device=DEV)
    ops.argmax(logits, out)
    assert out.tolist() == logits.argmax(-1).tolist()
    assert out[2] == 30 and out[3] == 1000


def test_sample_inverse_cdf():
    ops = _ops()
    m, v = 64, 1537
    logits = rnd(m, v, seed=12, scale=2.0)
    temps = [0.0 if i % 8 == 0 else 0.5 + 0.01 * i for i in range(m)]
    us = [random.Random(i).random() for i in range(m)]
    out = torch.full((m,), -1, dtype=torch.int32, device=DEV)
    ops.argmax(logits, out)
    ops.sample(logits, torch.tensor(temps, device=DEV), torch.tensor(us, device=DEV), out)
    got = out.tolist()
    for i in range(m):
        if temps[i] == 0:
            assert got[i] == int(logits[i].argmax())
            continue
        c = torch.cumsum(torch.softmax(logits[i].double() / temps[i], -1), -1).cpu()
        lo = c[got[i] - 1].item() if got[i] > 0 else 0.0
        # the drawn number lies in the chosen token's interval (up to float32 rounding of the sums)
        assert lo - 1e-5 <= us[i] <= c[got[i]].item() + 1e-5, (i, got[i], us[i])
    # u = 0 picks the first token with non-zero probability; large T is near uniform: u maps linearly
    out2 = torch.zeros(1, dtype=torch.int32, device=DEV)
    flat = torch.zeros(1, v, device=DEV)
    ops.sample(flat, torch.tensor([1.0], device=DEV), torch.tensor([0.5], device=DEV), out2)
    assert abs(int(out2[0]) - v // 2) <= 1


def test_sample_at_slice_edges_and_against_the_plain_sampler():
    """Targets on and beside the edges of the threads' slices (all sums exact: equal logits,
    2 tokens per slice), then many random rows against the float64 twin wherever the drawn
    number is not within rounding of an edge of the chosen token's interval."""
    import plain_qwen2 as P

    ops = _ops()
    v = 2048
    us = [0.5, (1024 - 0.5) / v, (1024 + 0.5) / v, 0.0, (v - 0.25) / v, 1 / v, 63.5 / v, 64 / v, 128 / v]
    want = [1024, 1023, 1024, 0, v - 1, 1, 63, 64, 128]
    flat = torch.zeros(len(us), v, device=DEV)
    out = torch.zeros(len(us), dtype=torch.int32, device=DEV)
    ops.sample(flat, torch.ones(len(us), device=DEV), torch.tensor(us, device=DEV), out)
    assert out.tolist() == want
    assert [P.sample_inverse_cdf(flat[0].cpu(), 1.0, u) for u in us] == want
    # only a few tokens can be drawn at all, the rest underflow to zero probability
    spiky = torch.full((3, 5000), -1e4, device=DEV)
    spiky[:, 17] = spiky[:, 3000] = spiky[:, 4999] = 0.0
    out3 = torch.zeros(3, dtype=torch.int32, device=DEV)
    ops.sample(spiky, torch.ones(3, device=DEV), torch.tensor([0.2, 0.5, 0.99], device=DEV), out3)
    assert out3.tolist() == [17, 3000, 4999]
    m, v = 256, 15013
    logits = rnd(m, v, seed=21, scale=3.0)
    temps = [0.3 + 0.005 * i for i in range(m)]
    draws = [random.Random(1000 + i).random() for i in range(m)]
    out = torch.zeros(m, dtype=torch.int32, device=DEV)
    ops.sample(logits, torch.tensor(temps, device=DEV), torch.tensor(draws, device=DEV), out)
    got, rows, close = out.tolist(), logits.cpu(), 0
    for i in range(m):
        c = torch.cumsum(torch.softmax(rows[i].double() / temps[i], -1), -1)
        twin = P.sample_inverse_cdf(rows[i], temps[i], draws[i])
        if got[i] != twin:
            edge = c[min(got[i], twin)].item()
            assert abs(got[i] - twin) == 1 and abs(edge - draws[i]) < 1e-5, (i, got[i], twin, draws[i], edge)
            close += 1
    assert close <= 3


# ----------------------------------------------------------------------------- weight-streaming products

@pytest.mark.parametrize("m", [1, 7, 16, 33, 64])
@pytest.mark.parametrize("n,k,ksplit", [(48, 64, 1), (3584, 3584, 3), (1000, 136, 2), (131, 8, 1), (70000, 96, 1),
                                        (3584, 18944, 8)])
def test_gemm_skinny(m, n, k, ksplit):
    ops = _ops()
    assert ops.gemm_skinny_supports(m, n, k, k, k)
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd(n, k, dtype=torch.bfloat16, seed=2)
    out = torch.full((ksplit, m, n), float("nan"), device=DEV)
    ops.gemm_skinny_bf16(x, w, out, m, ksplit)
    want = x.double() @ w.double().T
    assert torch.allclose(out.double().sum(0), want, atol=1e-3 * math.sqrt(k), rtol=1e-4)


@pytest.mark.parametrize("m", [1, 32, 33, 64, 65, 100, 128, 129, 192, 193, 256])
@pytest.mark.parametrize("n,k,ksplit", [(48, 64, 1), (1536, 1536, 6), (1000, 136, 2), (131, 8, 1), (3584, 18944, 4),
                                        (2048, 1000, 3), (70, 4096, 10)])
def test_gemm_mid(m, n, k, ksplit):
    """The products of a decode step of up to 256 rows: sizes that are no multiple of the tiles
    (64 rows of the weights, 32 of the input, stages of 64 k), k in parts; and a row's result is
    bit for bit the same whatever rows share the step and however many they are."""
    ops = _ops()
    assert ops.gemm_mid_supports(m, n, k, k, k)
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd(n, k, dtype=torch.bfloat16, seed=2)
    out = torch.full((ksplit, m, n), float("nan"), device=DEV)
    ops.gemm_mid_bf16(x, w, out, m, ksplit)
    want = x.double() @ w.double().T
    assert torch.allclose(out.double().sum(0), want, atol=1e-3 * math.sqrt(k), rtol=1e-4)
    rows = sorted({0, m // 2, m - 1})
    few = torch.full((ksplit, len(rows), n), float("nan"), device=DEV)
    ops.gemm_mid_bf16(x[rows].contiguous(), w, few, len(rows), ksplit)
    assert torch.equal(few, out[:, rows])
    wide = torch.zeros(m, k + 16, dtype=torch.bfloat16, device=DEV)      # rows that are further apart
    wide[:, 8:k + 8] = x
    again = torch.full_like(out, float("nan"))
    ops.gemm_mid_bf16(wide[:, 8:k + 8], w, again, m, ksplit)
    assert torch.equal(again, out)


@pytest.mark.parametrize("m", [1, 8, 32, 33, 64, 65, 96, 97, 128, 129, 192, 193, 256])
@pytest.mark.parametrize("inter,k", [(176, 64), (8960, 1536), (250, 96), (70, 520), (18944, 136), (16401, 64), (24600, 72)])
def test_gemm_mid_silu(m, inter, k):
    """Blocks of 64 features, and of 96 for up to 128 rows where 64 would make more than 256
    blocks (or of 128 for 25 to 64 rows where 96 still would: the last size), whose loads do not
    divide evenly over the block's waves; the
    row counts lie on both sides of every size of block (64, 96, 128, 192, 256 rows)."""
    ops = _ops()
    features = 64 if m > 128 or inter <= 256 * 64 else 128 if 25 <= m <= 64 and inter > 256 * 96 else 96
    assert ops.gemm_mid_silu_blocks(m, 2 * inter) == -(-inter // features)
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * inter, k, dtype=torch.bfloat16, seed=2, scale=0.1)
    out = torch.full((m, inter), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops.gemm_mid_silu_bf16(x, w, out, m)
    gu = x.double() @ w.double().T
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    assert torch.allclose(out.double(), want, atol=2e-2, rtol=2e-2)
    rows = sorted({0, m // 2, m - 1})
    few = torch.full((len(rows), inter), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops.gemm_mid_silu_bf16(x[rows].contiguous(), w, few, len(rows))
    assert torch.equal(few, out[rows])


@pytest.mark.parametrize("m", [1, 8, 32, 33, 64, 65, 128, 129, 192, 193, 256])
@pytest.mark.parametrize("n,k,ksplit", [(48, 64, 1), (1536, 1536, 4), (1000, 136, 2), (131, 8, 1), (3584, 18944, 9),
                                        (200, 4096, 10)])
def test_gemm_mid_with_128_rows_of_the_weights_a_block(m, n, k, ksplit):
    """The same partial sums, bit for bit, as with 64 rows of the weights a block (the order of an
    element's sums is a function of k alone)."""
    ops = _ops()
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd(n, k, dtype=torch.bfloat16, seed=2)
    out = torch.full((ksplit, m, n), float("nan"), device=DEV)
    ops.gemm_mid_bf16(x, w, out, m, ksplit, wide=True)
    want = x.double() @ w.double().T
    assert torch.allclose(out.double().sum(0), want, atol=1e-3 * math.sqrt(k), rtol=1e-4)
    narrow = torch.full_like(out, float("nan"))
    ops.gemm_mid_bf16(x, w, narrow, m, ksplit)
    assert torch.equal(narrow, out)


def test_gemm_mid_refuses_what_it_cannot_take():
    ops = _ops()
    x, w = rnd(300, 64, dtype=torch.bfloat16), rnd(48, 64, dtype=torch.bfloat16)
    assert not ops.gemm_mid_supports(300, 48, 64, 64, 64) and not ops.gemm_mid_supports(100, 48, 60, 60, 60)
    with pytest.raises(Exception, match="not supported"):
        ops.gemm_mid_bf16(x, w, torch.empty(1, 300, 48, device=DEV), 300, 1)
    with pytest.raises(Exception, match="empty"):
        ops.gemm_mid_bf16(x[:100], w, torch.empty(3, 100, 48, device=DEV), 100, 3)


@pytest.mark.parametrize("m", [1, 8, 40])
@pytest.mark.parametrize("inter,k", [(176, 64), (18944, 3584), (250, 96)])
def test_gemm_skinny_silu(m, inter, k):
    ops = _ops()
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * inter, k, dtype=torch.bfloat16, seed=2, scale=0.1)
    out = torch.full((m, inter), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops.gemm_skinny_silu_bf16(x, w, out, m)
    gu = x.double() @ w.double().T
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    assert torch.allclose(out.double(), want, atol=2e-2, rtol=2e-2)
