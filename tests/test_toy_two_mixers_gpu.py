"""A kind of layer that exists only in this file: a block with two mixers, each with a cache
of its own (attention over pages, a running mean with per-request state), and a layer with no
mixer at all. The model asks a block what it keeps and what its parts want of a step
(``cache_specs()``, ``step_arrays()``) and hands it the views in that order; it never looks
inside. One layer is named twice in the order, with caches of its own for each call. Nothing
under pyre_amd/ is changed to run it."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

import pytest
import torch

import plain_qwen2 as P
from helpers import cut, first_bad, random_ids, replay
from pyre_amd.config.model import ModelConfig
from pyre_amd.parts.base import (AttentionSpec, Block, EmbeddingSpec, LayerCall, LMHeadSpec, ModelSpec, RMSNormSpec,
                                 RotarySpec, SwiGLUSpec, make_part, register_part)
from pyre_amd.registry import register_architecture, unregister_architecture
from test_toy_parts_gpu import RunningMean, RunningMeanSpec

pytestmark = pytest.mark.gpu


@dataclass(frozen=True)
class TwoMixerSpec:
    """x += first(norm1(x)); x += second(norm2(x)); x += feed_forward(norm3(x))."""

    first: Any
    first_norm: Any
    second: Any
    second_norm: Any
    feed_forward: Any
    feed_forward_norm: Any
    kind: ClassVar[str] = "two_mixers"


@dataclass(frozen=True)
class OnlyFeedForwardSpec:
    """x += feed_forward(norm(x)): a layer that keeps nothing."""

    feed_forward: Any
    norm: Any
    kind: ClassVar[str] = "only_feed_forward"


class _Arranged(Block):
    """What both toy blocks share: their parts in a tuple, tensors and products of all of them."""

    def tensor_specs(self):
        return [s for p in self.parts for s in p.tensor_specs()]

    def bind(self, tensors, runtime):
        for p in self.parts:
            p.bind(tensors, runtime)

    def linears(self):
        return [lin for p in self.parts for lin in p.linears()]


class TwoMixerBlock(_Arranged):
    def __init__(self, spec):
        self.mixers = [make_part("mixer", spec.first), make_part("mixer", spec.second)]
        self.norms = [make_part("norm", n) for n in (spec.first_norm, spec.second_norm, spec.feed_forward_norm)]
        self.feed_forward = make_part("feed_forward", spec.feed_forward)
        self.parts = (*self.mixers, *self.norms, self.feed_forward)

    def cache_specs(self):
        return [m.cache_spec() for m in self.mixers]              # both keep something here

    def step_arrays(self):
        return [a for m in self.mixers for a in m.step_arrays()]

    def forward(self, ctx, state, caches):
        h = ctx.workspace.get("block.h", (ctx.n_tokens, state.resid.shape[1]), ctx.dtype)
        for mixer, norm, cache in zip(self.mixers, self.norms, caches):
            norm.forward(ctx, state.resid, state.pending, h)
            state.pending = mixer.forward(ctx, h, cache)
        self.norms[2].forward(ctx, state.resid, state.pending, h)
        state.pending = self.feed_forward.forward(ctx, h)


class OnlyFeedForwardBlock(_Arranged):
    def __init__(self, spec):
        self.norm = make_part("norm", spec.norm)
        self.feed_forward = make_part("feed_forward", spec.feed_forward)
        self.parts = (self.norm, self.feed_forward)

    def forward(self, ctx, state, caches):
        assert caches == []
        h = ctx.workspace.get("block.h", (ctx.n_tokens, state.resid.shape[1]), ctx.dtype)
        self.norm.forward(ctx, state.resid, state.pending, h)
        state.pending = self.feed_forward.forward(ctx, h)


@dataclass(frozen=True)
class TwoMixerConfig(ModelConfig):
    architecture: ClassVar[str] = "ToyTwoMixersForCausalLM"
    hidden_size: int = 40
    vocab_size: int = 173

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["hidden_size"], raw["vocab_size"])

    def to_dict(self):
        return {"architectures": [self.architecture], "hidden_size": self.hidden_size, "vocab_size": self.vocab_size}


NQ, NKV, HD, INTER, EPS, THETA = 4, 2, 12, 72, 1e-5, 3e3
#: layer 0 (attention, then running mean), layer 1 (feed-forward only), layer 2 (the same two kinds
#: of mixer), layer 0 again
ORDER = [LayerCall(0), LayerCall(1), LayerCall(2), LayerCall(0)]


def build(cfg) -> ModelSpec:
    H = cfg.hidden_size
    rot = RotarySpec(HD, THETA, 512)

    def two(i):
        p = f"model.layers.{i}"
        return TwoMixerSpec(AttentionSpec(H, NQ, NKV, HD, rot, f"{p}.self_attn"), RMSNormSpec(H, EPS, f"{p}.norm1"),
                            RunningMeanSpec(H, p), RMSNormSpec(H, EPS, f"{p}.norm2"),
                            SwiGLUSpec(H, INTER, f"{p}.mlp"), RMSNormSpec(H, EPS, f"{p}.norm3"))

    layers = (two(0), OnlyFeedForwardSpec(SwiGLUSpec(H, INTER, "model.layers.1.mlp"), RMSNormSpec(H, EPS, "model.layers.1.norm")),
              two(2))
    return ModelSpec(H, cfg.vocab_size, 512, EmbeddingSpec(cfg.vocab_size, H), layers, tuple(ORDER),
                     RMSNormSpec(H, EPS, "model.norm"), LMHeadSpec(cfg.vocab_size, H))


def plain(w, ids):
    """The model by the plain implementation's parts, whole sequence, float64."""
    c = {"num_attention_heads": NQ, "num_key_value_heads": NKV, "head_dim": HD}
    ids = torch.as_tensor(ids)
    x = P.embed(ids, w["model.embed_tokens.weight"])
    cos, sin = P.rope_tables(len(ids), HD, THETA)
    ident = lambda t: t  # noqa: E731
    count = torch.arange(1, len(ids) + 1, dtype=x.dtype)[:, None]
    for call in ORDER:
        p = f"model.layers.{call.layer}"
        if call.layer == 1:
            x = x + P.swiglu(P.rms_norm(x, w[f"{p}.norm.weight"], EPS), w, f"{p}.mlp", ident)
            continue
        x = x + P.attention_block(P.rms_norm(x, w[f"{p}.norm1.weight"], EPS), w, f"{p}.self_attn", c, cos, sin, ident)
        mean = torch.cumsum(P.rms_norm(x, w[f"{p}.norm2.weight"], EPS), 0) / count
        x = x + mean @ w[f"{p}.mix.weight"].T
        x = x + P.swiglu(P.rms_norm(x, w[f"{p}.norm3.weight"], EPS), w, f"{p}.mlp", ident)
    return (P.rms_norm(x, w["model.norm.weight"], EPS) @ w["lm_head.weight"].T).float()


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from pyre_amd.weights import write_random_model

    register_part("mixer", "running_mean", RunningMean)
    register_part("block", TwoMixerSpec.kind, TwoMixerBlock)
    register_part("block", OnlyFeedForwardSpec.kind, OnlyFeedForwardBlock)
    register_architecture(TwoMixerConfig.architecture, TwoMixerConfig, build)
    cfg = TwoMixerConfig()
    folder = tmp_path_factory.mktemp("two_mixers")
    write_random_model(folder, cfg, seed=11, std=0.08, gain_std=0.1)
    yield cfg, folder, P.read_weights(folder)
    unregister_architecture(TwoMixerConfig.architecture)


def _engine(folder, dtype, **kw):
    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.engine import Engine

    args = dict(dtype=dtype, page_size=8, max_cached_tokens=512, max_num_seqs=3, max_num_batched_tokens=256,
                use_graphs=False)
    args.update(kw)
    return Engine.from_folder(folder, EngineConfig(**args))


def test_the_block_says_what_it_keeps(toy):
    cfg, folder, w = toy
    eng = _engine(folder, "float32")
    m = eng.cache
    # entries 0, 2 and 3 keep pages (their first cache) and a state (their second); entry 1 keeps nothing
    assert eng.model.cache_specs()[1] == [] and [len(c) for c in eng.model.cache_specs()] == [2, 0, 2, 2]
    assert [g.cells for g in m.page_groups] == [[(0, 0), (2, 0), (3, 0)]]
    assert [g.cells for g in m.state_groups] == [[(0, 1), (2, 1), (3, 1)]]
    assert m.caches_of_entry(1) == 0 and 1 not in m.group_of_entry
    assert m.page_groups[0].tensors["k"].shape[0] == 3 and m.state_groups[0].tensor.shape[0] == 3
    assert "model.layers.2.mix.weight" in w and "model.layers.1.self_attn.q_proj.weight" not in w


@pytest.mark.parametrize("dtype,tol,poison", [("float32", 1e-5, False), ("float32", 1e-5, True), ("bfloat16", 3e-2, False)])
def test_two_mixers_whole_portions_and_mixed(toy, dtype, tol, poison):
    cfg, folder, w = toy
    reqs = {r: random_ids(cfg.vocab_size, n, seed=n) for r, n in (("a", 57), ("b", 41), ("c", 83), ("d", 30))}
    want = {r: plain(w, ids) for r, ids in reqs.items()}
    eng = _engine(folder, dtype, debug_poison=poison)
    got = replay(eng, [([(r, ids, list(range(len(ids))))], [r]) for r, ids in reqs.items()])
    bad, _ = first_bad(got, want, tol)
    assert bad is None, bad
    # portions of changing size: pages and state both carry across steps
    steps = []
    for r, ids in reqs.items():
        pos = 0
        parts = cut(len(ids), [7, 2, 19, 3, 1, 30])
        for k, n in enumerate(parts):
            steps.append(([(r, ids[pos:pos + n], list(range(n)))], [r] if k == len(parts) - 1 else []))
            pos += n
    got = replay(eng, steps)
    bad, _ = first_bad(got, want, tol)
    assert bad is None, bad
    # mixed: three live at a time, slots and pages used again by the fourth
    fed = {r: 0 for r in reqs}
    live, waiting, steps, k = [], list(reqs), [], 0
    while live or waiting:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            n = min([5, 1, 13, 2][k % 4], len(reqs[r]) - fed[r])
            k += 1
            entries.append((r, reqs[r][fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    got = replay(eng, steps)
    bad, _ = first_bad(got, want, tol)
    assert bad is None, bad
    eng.cache.check_invariants()
    assert all(g.allocator.num_used == 0 for g in eng.cache.page_groups) and eng.cache.slots.num_used == 0
