"""Each part alone (norm, position encoding, attention mixer, feed-forward, block,
embedding, head) against the plain implementation's function for it, built through
the part registry with its own random tensors and a hand-made step context."""

from __future__ import annotations

import pytest
import torch

import plain_qwen2 as P

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


class Rig:
    """A cache manager, metadata buffers and a runtime: what the engine gives a part."""

    def __init__(self, cache_specs, dtype, page_size=8, pages=64, seqs=4, max_len=256):
        from pyre_amd.cache import CacheManager
        from pyre_amd.engine.context import MetaBuffers, Runtime

        self.dtype = DT[dtype]
        from pyre_amd.parts.attention import STEP_ARRAYS

        self.cache = CacheManager(cache_specs, page_size, pages, seqs, max_len)
        self.cache.materialize(DEV, self.dtype)
        self.arrays = list(STEP_ARRAYS)
        self.meta = MetaBuffers(DEV, 512, seqs, [32 for _ in self.cache.page_groups], self.arrays)
        self.runtime = Runtime(DEV, self.dtype, max_len)

    def context(self, entries, vocab=1000):
        from pyre_amd.engine.batch import Entry, build_host_batch
        from pyre_amd.engine.context import PagedLayerView, StepContext

        es = [Entry(r, list(t), list(w)) for r, t, w in entries]
        for e in es:
            if e.rid not in self.cache:
                self.cache.add_request(e.rid)
            self.cache.reserve(e.rid, len(e.tokens))
        hb = build_host_batch(es, self.cache, vocab, table_width=32).attach(self.arrays)
        v = self.meta.upload(hb)
        ctx = StepContext(self.runtime, hb, hb.n_tokens, hb.n_seqs, len(hb.logit_rows), v["tokens"], v["positions"],
                          v["seq_of_token"], v["logit_rows"][:len(hb.logit_rows)], v["q_start"], v["ctx_len"],
                          v["state_slots"], {a.name: v["x:" + a.name] for a in self.arrays})
        views = [PagedLayerView({n: t[0] for n, t in g.tensors.items()}, v[f"table{i}"], v[f"slots{i}"], g.page_size,
                                g.spec.window)
                 for i, g in enumerate(self.cache.page_groups)]
        return ctx, views, es

    def commit(self, es):
        for e in es:
            self.cache.commit(e.rid, len(e.tokens))


def dev(t, dtype):
    return t.to(DEV, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rmsnorm_part(dtype):
    from pyre_amd.hip.ops import Partials
    from pyre_amd.parts.base import RMSNormSpec, make_part

    H, n, eps = 72, 11, 1e-5
    part = make_part("norm", RMSNormSpec(H, eps, "n"))
    assert [(s.name, s.shape, s.init) for s in part.tensor_specs()] == [("n.weight", (H,), "gain")]
    gain = rnd(H, seed=1).to(DT[dtype]) + 1
    part.bind({"n.weight": dev(gain, DT[dtype])}, None)
    rig = Rig([], dtype)
    ctx, _, _ = rig.context([("a", list(range(n)), [])])
    resid, delta = rnd(n, H, seed=2), rnd(1, n, H, seed=3)
    r = dev(resid, torch.float32)
    out = torch.empty(n, H, device=DEV, dtype=DT[dtype])
    part.forward(ctx, r, Partials(dev(delta, torch.float32)), out)
    want = P.rms_norm((resid + delta[0]).double(), gain.double(), eps)
    assert torch.allclose(r.cpu().double(), (resid + delta[0]).double(), atol=1e-6)
    assert torch.allclose(out.cpu().double(), want, atol=TOL[dtype], rtol=TOL[dtype])


def test_rotary_part_tables():
    from pyre_amd.engine.context import Runtime
    from pyre_amd.parts.base import NoPositionSpec, RotarySpec, make_part

    part = make_part("position", RotarySpec(24, 1e6, 4096, rotary_dim=16))
    cos, sin, rot = part.rotary(Runtime(DEV, torch.float32, 300))
    assert rot == 16 and cos.shape == (300, 8) and cos.dtype == torch.float32
    pc, ps = P.rope_tables(300, 16, 1e6, torch.float32)          # the reference's table, both halves equal
    assert torch.equal(cos.cpu(), pc[:, :8]) and torch.equal(sin.cpu(), ps[:, 8:])
    assert make_part("position", NoPositionSpec()).rotary(None) == (None, None, 0)
    with pytest.raises(ValueError):
        make_part("position", RotarySpec(24, 1e4, 64, rotary_dim=30))


def attention_weights(H, nq, nkv, hd, seed):
    names = {"q": nq * hd, "k": nkv * hd, "v": nkv * hd}
    w = {f"a.{n}_proj.weight": rnd(o, H, seed=seed + i, scale=0.2) for i, (n, o) in enumerate(names.items())}
    w.update({f"a.{n}_proj.bias": rnd(o, seed=seed + 10 + i, scale=0.2) for i, (n, o) in enumerate(names.items())})
    w["a.o_proj.weight"] = rnd(H, nq * hd, seed=seed + 20, scale=0.2)
    return w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq,nkv,hd,window", [(6, 2, 12, 0), (4, 4, 32, 0), (8, 2, 64, 21), (3, 1, 20, 9)])
def test_attention_part(dtype, nq, nkv, hd, window):
    """Two requests, each fed in two portions and a single token, against the plain
    attention block over the whole sequences."""
    from pyre_amd.parts.attention import KVCacheSpec
    from pyre_amd.parts.base import AttentionSpec, RotarySpec, make_part

    H, theta = 56, 1e4
    spec = AttentionSpec(H, nq, nkv, hd, RotarySpec(hd, theta, 256), "a", window=window)
    part = make_part("mixer", spec)
    assert part.cache_spec() == KVCacheSpec(nkv, hd, window)
    w = attention_weights(H, nq, nkv, hd, seed=nq)
    wt = DT[dtype]
    part.bind({k: dev(v.to(wt), wt) for k, v in w.items()}, None)
    w = {k: v.to(wt).double() for k, v in w.items()}
    rig = Rig([part.cache_spec()], dtype)
    lens = {"a": 37, "b": 22}
    hs = {r: rnd(n, H, seed=n).to(wt) for r, n in lens.items()}
    got = {r: [] for r in lens}
    fed = {r: 0 for r in lens}
    for cuts in ({"a": 20, "b": 9}, {"a": 16, "b": 12}, {"a": 1, "b": 1}):
        entries = [(r, [0] * n, []) for r, n in cuts.items()]
        ctx, views, es = rig.context(entries)
        h = torch.cat([hs[r][fed[r]:fed[r] + n] for r, n in cuts.items()]).to(DEV)
        out = part.forward(ctx, h, views[0])
        rows = (out.data.float().sum(0) + (out.bias.float() if out.bias is not None else 0)).cpu()
        i = 0
        for r, n in cuts.items():
            got[r].append(rows[i:i + n])
            i += n
            fed[r] += n
        rig.commit(es)
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": hd}
    rndf = (lambda x: x.to(torch.bfloat16).to(x.dtype)) if dtype == "bfloat16" else (lambda x: x)
    for r, n in lens.items():
        cos, sin = P.rope_tables(n, hd, theta)
        want = P.attention_block(hs[r].double(), w, "a", cfg, cos, sin, rndf, window=window)
        assert torch.allclose(torch.cat(got[r]).double(), want, atol=TOL[dtype] * 3, rtol=TOL[dtype]), r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n", [3, 70])
def test_swiglu_part(dtype, n):
    from pyre_amd.parts.base import SwiGLUSpec, make_part

    H, I = 40, 136
    part = make_part("feed_forward", SwiGLUSpec(H, I, "m"))
    assert {s.name: s.shape for s in part.tensor_specs()} == {
        "m.gate_proj.weight": (I, H), "m.up_proj.weight": (I, H), "m.down_proj.weight": (H, I)}
    wt = DT[dtype]
    w = {"m.gate_proj.weight": rnd(I, H, seed=1, scale=0.3), "m.up_proj.weight": rnd(I, H, seed=2, scale=0.3),
         "m.down_proj.weight": rnd(H, I, seed=3, scale=0.3)}
    part.bind({k: dev(v, wt) for k, v in w.items()}, None)
    rig = Rig([], dtype)
    ctx, _, _ = rig.context([("a", [0] * n, [])])
    h = rnd(n, H, seed=4).to(wt)
    out = part.forward(ctx, h.to(DEV))
    rndf = (lambda x: x.to(torch.bfloat16).to(x.dtype)) if dtype == "bfloat16" else (lambda x: x)
    want = P.swiglu(h.double(), {k: v.to(wt).double() for k, v in w.items()}, "m", rndf)
    assert torch.allclose(out.data.float().sum(0).cpu().double(), want, atol=TOL[dtype] * 3, rtol=TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_and_head_parts(dtype):
    from pyre_amd.parts.base import EmbeddingSpec, LMHeadSpec, make_part

    V, H = 333, 40
    emb = make_part("embedding", EmbeddingSpec(V, H))
    head = make_part("head", LMHeadSpec(V, H, tied_to="model.embed_tokens.weight"))
    assert head.tensor_specs()[0].alias_of == "model.embed_tokens.weight"
    wt = DT[dtype]
    table = dev(rnd(V, H, seed=5), wt)
    emb.bind({"model.embed_tokens.weight": table}, None)
    head.bind({"lm_head.weight": table}, None)                         # tied: the same memory
    assert head.linear.weight.data_ptr() == table.data_ptr()
    rig = Rig([], dtype)
    ids = [5, 332, 0, 77]
    ctx, _, _ = rig.context([("a", ids, [1, 3])], vocab=V)
    resid = torch.empty(4, H, device=DEV)
    emb.forward(ctx, resid)
    assert torch.equal(resid.cpu(), table.float().cpu()[ids])
    h = dev(rnd(2, H, seed=6), wt)
    logits = head.forward(ctx, h, 2)
    assert logits.dtype == torch.float32 and logits.shape == (2, V)
    want = h.double().cpu() @ table.double().cpu().T
    assert torch.allclose(logits.cpu().double(), want, atol=1e-3 if dtype == "bfloat16" else 1e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_block_part(dtype):
    """The pre-norm arrangement: x + mixer(norm(x)), then x + ffn(norm(x)); the
    block leaves its last term pending for the next norm."""
    from pyre_amd.parts.base import AttentionSpec, BlockSpec, RMSNormSpec, RotarySpec, SwiGLUSpec, make_part
    from pyre_amd.parts.block import Hidden

    H, nq, nkv, hd, I, eps, n = 48, 4, 2, 16, 96, 1e-6, 19
    p = "model.layers.0"
    spec = BlockSpec(AttentionSpec(H, nq, nkv, hd, RotarySpec(hd, 1e4, 128), f"{p}.self_attn"),
                     RMSNormSpec(H, eps, f"{p}.input_layernorm"), SwiGLUSpec(H, I, f"{p}.mlp"),
                     RMSNormSpec(H, eps, f"{p}.post_attention_layernorm"))
    block = make_part("block", spec)
    wt = DT[dtype]
    w = {s.name: rnd(*s.shape, seed=i, scale=0.2) + (1 if s.init == "gain" else 0) for i, s in enumerate(block.tensor_specs())}
    assert len(w) == 12
    block.bind({k: dev(v, wt) for k, v in w.items()}, None)
    rig = Rig([block.cache_specs()], dtype)
    ctx, views, _ = rig.context([("a", [0] * n, [])])
    x = rnd(n, H, seed=99)
    state = Hidden(x.to(DEV))
    block.forward(ctx, state, views)
    got = state.resid.cpu().double() + state.pending.data.float().sum(0).cpu().double()
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": hd, "rms_norm_eps": eps}
    cos, sin = P.rope_tables(n, hd, 1e4)
    rndf = (lambda t: t.to(torch.bfloat16).to(t.dtype)) if dtype == "bfloat16" else (lambda t: t)
    want = P.decoder_layer(x.double(), {k: v.to(wt).double() for k, v in w.items()}, 0, cfg, cos, sin, rndf)
    assert torch.allclose(got, want, atol=TOL[dtype] * 3, rtol=TOL[dtype])
