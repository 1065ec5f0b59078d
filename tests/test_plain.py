"""The plain implementation pinned by what fixes it beside the reference's text:
special cases that reduce to a library routine, invariants, and the vectors the
reference's own tests hold. Each is chosen so that a plausible mistake fails it."""

from __future__ import annotations

import math

import pytest
import torch

import plain_qwen2 as P

torch.manual_seed(0)


def test_repeat_kv_head_mapping():
    """tests/test_parity.py:111-126 of the reference: n_kv=2, n_rep=6, head i reads i // 6
    (repeat() instead of repeat_interleave() fails this)."""
    x = torch.arange(2, dtype=torch.float64).view(2, 1, 1)
    out = P.repeat_kv(x, 6)
    assert out.shape == (12, 1, 1)
    assert [out[i, 0, 0].item() for i in range(12)] == [i // 6 for i in range(12)]
    assert P.repeat_kv(x, 1) is x


def test_rms_norm_is_the_library_routine():
    x = torch.randn(5, 96, dtype=torch.float64) * 3
    w = torch.randn(96, dtype=torch.float64)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), torch.nn.functional.rms_norm(x, (96,), w, 1e-5), atol=1e-12)
    # scale invariance (a mean subtraction or a gain of 1+w would break one of these)
    one = torch.ones(96, dtype=torch.float64)
    assert torch.allclose(P.rms_norm(7.0 * x, one, 1e-12), P.rms_norm(x, one, 1e-12), atol=1e-9)
    assert torch.allclose(P.rms_norm(x, one, 1e-12).pow(2).mean(-1), torch.ones(5, dtype=torch.float64))
    assert torch.allclose(P.rms_norm(x + 100.0, one, 1e-6).mean(-1), (x + 100).mean(-1) / (x + 100).pow(2).mean(-1).sqrt(), atol=1e-6)


def test_rope_table_and_rotation():
    cos, sin = P.rope_tables(50, 16, 1e4)
    assert cos.shape == (50, 16)
    # row p is cos/sin(p * theta^(-2j/d)), both halves equal (pyre/model.py:41-51)
    j = torch.arange(8, dtype=torch.float64)
    ang = 7 * (1e4 ** (-2 * j / 16))
    assert torch.allclose(cos[7, :8], ang.cos(), atol=1e-6) and torch.allclose(cos[7, 8:], ang.cos(), atol=1e-6)
    assert torch.allclose(sin[7, :8], ang.sin(), atol=1e-6)
    q = torch.randn(3, 50, 16, dtype=torch.float64)
    k = torch.randn(3, 50, 16, dtype=torch.float64)
    qr, kr = P.apply_rope(q, k, cos, sin)
    # position 0 is the identity; norms of the pairs (j, j + d/2) are kept
    assert torch.allclose(qr[:, 0], q[:, 0])
    assert torch.allclose(qr[..., :8] ** 2 + qr[..., 8:] ** 2, q[..., :8] ** 2 + q[..., 8:] ** 2)
    # the pairing is half-split, not interleaved: rotating (1,0,...) at position 1 moves weight to index 8
    e0 = torch.zeros(1, 2, 16, dtype=torch.float64)
    e0[..., 0] = 1
    r0, _ = P.apply_rope(e0, e0, cos[:2], sin[:2])
    assert abs(r0[0, 1, 8].item() - math.sin(1.0)) < 1e-6 and abs(r0[0, 1, 1].item()) < 1e-12
    # only distances count: <rot(q, m), rot(k, n)> depends on m - n
    a, b = torch.randn(16, dtype=torch.float64), torch.randn(16, dtype=torch.float64)
    def dot(m, n):
        x, _ = P.apply_rope(a.view(1, 1, 16), a.view(1, 1, 16), cos[m:m + 1], sin[m:m + 1])
        y, _ = P.apply_rope(b.view(1, 1, 16), b.view(1, 1, 16), cos[n:n + 1], sin[n:n + 1])
        return (x * y).sum().item()
    assert abs(dot(30, 10) - dot(25, 5)) < 1e-4 and abs(dot(30, 10) - dot(40, 20)) < 1e-4   # float32 table
    assert abs(dot(30, 10) - dot(10, 30)) > 1e-3                                            # a sign error in sin fails this


def test_attention_is_the_library_routine():
    q, k, v = (torch.randn(4, 33, 16, dtype=torch.float64) for _ in range(3))
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert torch.allclose(P.causal_attention(q, k, v, 16 ** -0.5), want, atol=1e-12)
    # one visible key: exactly its value; q = 0: running mean of v
    assert torch.allclose(P.causal_attention(q, k, v, 0.25)[:, 0], v[:, 0])
    z = P.causal_attention(torch.zeros_like(q), k, v, 0.25)
    assert torch.allclose(z[:, 9], v[:, :10].mean(1))
    # later tokens never matter to earlier ones
    k2, v2 = k.clone(), v.clone()
    k2[:, 20:] += 5
    v2[:, 20:] -= 3
    assert torch.allclose(P.causal_attention(q, k2, v2, 0.25)[:, :20], P.causal_attention(q, k, v, 0.25)[:, :20])
    # a window of w keeps exactly the last w keys
    w = P.causal_attention(torch.zeros_like(q), k, v, 0.25, window=4)
    assert torch.allclose(w[:, 10], v[:, 7:11].mean(1)) and torch.allclose(w[:, 1], v[:, :2].mean(1))


def test_attention_block_scale_biases_and_head_layout():
    """The block around the attention, pinned where the formulas alone do not: with identity
    projections it is the library's attention at its default scale head_dim ** -0.5
    (`pyre/model.py:82,109`: a scale of 1 / head_dim, or one applied before the rotation's
    table, fails this); q, k and v have biases, the output projection has none
    (`pyre/model.py:83-87`); head n owns columns n * hd .. (n + 1) * hd - 1 of the projections
    (`pyre/model.py:92-94`); V is not rotated."""
    nq, nkv, hd, S = 4, 2, 8, 9
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": hd}
    H = nq * hd
    eye = torch.eye(H, dtype=torch.float64)
    pick = torch.zeros(nkv * hd, H, dtype=torch.float64)      # k and v heads read the columns of q heads 0 and 2
    for g, src in enumerate((0, 2)):
        pick[g * hd:(g + 1) * hd, src * hd:(src + 1) * hd] = torch.eye(hd, dtype=torch.float64)
    w = {"a.q_proj.weight": eye, "a.q_proj.bias": torch.zeros(H, dtype=torch.float64),
         "a.k_proj.weight": pick, "a.k_proj.bias": torch.zeros(nkv * hd, dtype=torch.float64),
         "a.v_proj.weight": pick, "a.v_proj.bias": torch.zeros(nkv * hd, dtype=torch.float64),
         "a.o_proj.weight": eye}
    h = torch.randn(S, H, dtype=torch.float64)
    one, zero = torch.ones(S, hd, dtype=torch.float64), torch.zeros(S, hd, dtype=torch.float64)
    out = P.attention_block(h, w, "a", cfg, one, zero, lambda t: t)           # cos = 1, sin = 0: no rotation
    q = h.view(S, nq, hd).transpose(0, 1)
    kv = q[[0, 0, 2, 2]]                                                      # query head i reads kv head i // 2
    want = torch.nn.functional.scaled_dot_product_attention(q, kv, kv, is_causal=True).transpose(0, 1).reshape(S, H)
    assert torch.allclose(out, want, atol=1e-12)
    # the rotation reaches q and k only: with q = k = 0 (zero weights) any table gives the running mean of v
    cos, sin = P.rope_tables(S, hd, 1e4)
    w0 = dict(w)
    w0["a.q_proj.weight"], w0["a.k_proj.weight"] = torch.zeros_like(eye), torch.zeros_like(pick)
    mean = torch.cumsum(h, 0) / torch.arange(1, S + 1, dtype=torch.float64)[:, None]
    got = P.attention_block(h, w0, "a", cfg, cos, sin, lambda t: t)
    assert torch.allclose(got.view(S, nq, hd)[:, 1], mean.view(S, nq, hd)[:, 0], atol=1e-12)   # head 1 reads kv head 0 = columns of q head 0
    # biases: a v bias passes straight through (the weights of attention sum to 1); an o bias does not exist
    wb = dict(w0)
    wb["a.v_proj.bias"] = torch.arange(nkv * hd, dtype=torch.float64)
    shifted = P.attention_block(h, wb, "a", cfg, cos, sin, lambda t: t)
    assert torch.allclose((shifted - got).view(S, nq, hd)[:, 3], torch.arange(hd, 2 * hd, dtype=torch.float64).expand(S, hd))
    wb["a.o_proj.bias"] = torch.full((H,), 7.0, dtype=torch.float64)
    assert torch.equal(P.attention_block(h, wb, "a", cfg, cos, sin, lambda t: t), shifted)
    wq = dict(w)
    wq["a.q_proj.bias"] = torch.randn(H, dtype=torch.float64)
    assert not torch.allclose(P.attention_block(h, wq, "a", cfg, one, zero, lambda t: t), out)


def test_swiglu_is_the_library_routine():
    h = torch.randn(6, 32, dtype=torch.float64)
    w = {"m.gate_proj.weight": torch.randn(40, 32, dtype=torch.float64),
         "m.up_proj.weight": torch.randn(40, 32, dtype=torch.float64),
         "m.down_proj.weight": torch.randn(32, 40, dtype=torch.float64)}
    want = (torch.nn.functional.silu(h @ w["m.gate_proj.weight"].T) * (h @ w["m.up_proj.weight"].T)) @ w["m.down_proj.weight"].T
    assert torch.allclose(P.swiglu(h, w, "m", lambda x: x), want, atol=1e-12)
    w0 = dict(w)
    w0["m.up_proj.weight"] = torch.zeros(40, 32, dtype=torch.float64)
    assert torch.all(P.swiglu(h, w0, "m", lambda x: x) == 0)          # gate and up swapped would not give zero


def test_whole_model_invariants(plain_models):
    for name, (cfg, w) in plain_models.items():
        ids = torch.randint(0, cfg["vocab_size"], (40,))
        full = P.forward(w, cfg, ids)
        assert full.shape == (40, cfg["vocab_size"])
        # logits at position i do not depend on tokens after i
        assert torch.allclose(P.forward(w, cfg, ids[:17]), full[:17], atol=1e-10)
        # a length-1 prompt: attention returns v0, so the result is position-free
        one = P.forward(w, cfg, ids[:1])
        assert torch.allclose(one[0], full[0], atol=1e-10)
        if cfg["tie_word_embeddings"]:
            assert w["lm_head.weight"] is w["model.embed_tokens.weight"]


def test_norm_sits_before_the_mixer_not_after(plain_models):
    """With all linear weights of a layer's attention zero the layer adds nothing
    from attention: x + 0. A post-norm arrangement would change x."""
    cfg, w = plain_models["tiny-a"]
    w = dict(w)
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"] = torch.zeros_like(w[f"model.layers.{i}.self_attn.o_proj.weight"])
        w[f"model.layers.{i}.mlp.down_proj.weight"] = torch.zeros_like(w[f"model.layers.{i}.mlp.down_proj.weight"])
    ids = torch.tensor([5, 9, 11])
    logits, hidden = P.forward(w, cfg, ids, return_hidden=True)
    emb = w["model.embed_tokens.weight"][ids]
    assert torch.allclose(hidden[-1], emb)
    assert torch.allclose(logits, P.rms_norm(emb, w["model.norm.weight"], cfg["rms_norm_eps"]) @ w["lm_head.weight"].T)


def test_greedy_and_sampling_twin(plain_models):
    cfg, w = plain_models["tiny-b"]
    out = P.greedy(w, cfg, [1, 2, 3], 5)
    assert len(out) == 5 and out[0] == int(P.forward(w, cfg, [1, 2, 3])[-1].argmax())
    assert P.greedy(w, cfg, [1, 2, 3], 5, eos_id=out[1]) == out[:2]      # the stop token is kept (pyre/scheduler.py:82-83)
    logits = torch.tensor([0.0, math.log(2.0), math.log(1.0)])            # p = .25, .5, .25
    assert [P.sample_inverse_cdf(logits, 1.0, u) for u in (0.0, 0.24, 0.26, 0.74, 0.76, 0.999)] == [0, 0, 1, 1, 2, 2]
    assert P.sample_inverse_cdf(logits, 0.0, 0.9) == 1
    assert P.sample_inverse_cdf(logits, 1e-4, 0.999) == 1                # T -> 0 is greedy
