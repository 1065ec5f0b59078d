"""The framework's generality, shown with parts and an architecture that exist
only in this file: a mixer with state of its own (a running mean, one vector and a
count per request), layers with different mixers and a windowed attention, an
order of layers that names a layer twice and lets a call read another call's
cache. Nothing under pyre_amd/ is changed to run them."""

from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch

import plain_qwen2 as P
from helpers import cut, first_bad, random_ids, replay
from pyre_amd.config.model import ModelConfig
from pyre_amd.hip.ops import Partials
from pyre_amd.parts.base import (AttentionSpec, BlockSpec, EmbeddingSpec, LayerCall, LMHeadSpec, Mixer,
                                 ModelSpec, RMSNormSpec, RotarySpec, StateCacheSpec, SwiGLUSpec, TensorSpec,
                                 register_part)
from pyre_amd.registry import register_architecture, unregister_architecture

pytestmark = pytest.mark.gpu


# ----------------------------------------------------------------------------- a toy mixer

@dataclass(frozen=True)
class RunningMeanSpec:
    hidden_size: int
    prefix: str
    kind: ClassVar[str] = "running_mean"


class RunningMean(Mixer):
    """out[t] = W mean(h[0..t]). Per request it keeps sum(h) (H floats) and the count."""

    def __init__(self, spec):
        self.spec = spec

    def cache_spec(self):
        return StateCacheSpec((self.spec.hidden_size + 1,), "float32")

    def tensor_specs(self):
        h = self.spec.hidden_size
        return [TensorSpec(f"{self.spec.prefix}.mix.weight", (h, h))]

    def bind(self, tensors, runtime):
        self.w = tensors[f"{self.spec.prefix}.mix.weight"].float()

    def forward(self, ctx, h, cache):
        hb, H = ctx.host, self.spec.hidden_size
        out = torch.empty(ctx.n_tokens, H, device=h.device, dtype=torch.float32)
        for s in range(hb.n_seqs):
            a, b = int(hb.q_start[s]), int(hb.q_start[s + 1])
            state = cache.tensor[int(hb.state_slots[s])]
            sums = state[:H] + torch.cumsum(h[a:b].float(), 0)
            counts = state[H] + torch.arange(1, b - a + 1, device=h.device)
            out[a:b] = (sums / counts[:, None]) @ self.w.T
            state[:H] = sums[-1]
            state[H] = counts[-1]
        return Partials(out.view(1, ctx.n_tokens, H))


# ----------------------------------------------------------------------------- a toy architecture

@dataclass(frozen=True)
class ToyConfig(ModelConfig):
    architecture: ClassVar[str] = "ToyMixForCausalLM"
    hidden_size: int = 48
    vocab_size: int = 211
    window: int = 20

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["hidden_size"], raw["vocab_size"], raw["window"])

    def to_dict(self):
        return {"architectures": [self.architecture], "hidden_size": self.hidden_size,
                "vocab_size": self.vocab_size, "window": self.window}


NQ, NKV, HD, INTER, EPS, THETA = 4, 2, 16, 80, 1e-5, 1e4
#: order of layers: 0 (attention), 1 (running mean), 2 (windowed attention), 0 again
#: (a second cache of its own), 3 (attention that reads the keys and values entry 0 wrote)
ORDER = [LayerCall(0), LayerCall(1), LayerCall(2), LayerCall(0), LayerCall(3, cache_from=0)]


def build_toy(cfg: ToyConfig) -> ModelSpec:
    H = cfg.hidden_size
    rot = RotarySpec(HD, THETA, 512)

    def block(i, mixer):
        p = f"model.layers.{i}"
        return BlockSpec(mixer, RMSNormSpec(H, EPS, f"{p}.input_layernorm"),
                         SwiGLUSpec(H, INTER, f"{p}.mlp"), RMSNormSpec(H, EPS, f"{p}.post_attention_layernorm"))

    def attn(i, window=0):
        return AttentionSpec(H, NQ, NKV, HD, rot, f"model.layers.{i}.self_attn", window=window)

    layers = (block(0, attn(0)), block(1, RunningMeanSpec(H, "model.layers.1")),
              block(2, attn(2, cfg.window)), block(3, attn(3)))
    return ModelSpec(H, cfg.vocab_size, 512, EmbeddingSpec(cfg.vocab_size, H), layers, tuple(ORDER),
                     RMSNormSpec(H, EPS, "model.norm"), LMHeadSpec(cfg.vocab_size, H))


def plain_toy(w, cfg: ToyConfig, ids):
    """The toy model by the plain implementation's parts, whole sequence, float64."""
    c = {"num_attention_heads": NQ, "num_key_value_heads": NKV, "head_dim": HD}
    ids = torch.as_tensor(ids)
    x = P.embed(ids, w["model.embed_tokens.weight"])
    cos, sin = P.rope_tables(len(ids), HD, THETA)
    ident = lambda t: t  # noqa: E731
    kept = {}
    for pos, call in enumerate(ORDER):
        i = call.layer
        p = f"model.layers.{i}"
        h = P.rms_norm(x, w[f"{p}.input_layernorm.weight"], EPS)
        if i == 1:
            mean = torch.cumsum(h, 0) / torch.arange(1, len(ids) + 1, dtype=h.dtype)[:, None]
            x = x + mean @ w[f"{p}.mix.weight"].T
        else:
            keep = []
            kv = kept[call.cache_from] if call.cache_from is not None else None
            x = x + P.attention_block(h, w, f"{p}.self_attn", c, cos, sin, ident,
                                      window=cfg.window if i == 2 else 0, kv=kv, keep=keep)
            kept[pos] = keep[0]
        x = x + P.swiglu(P.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], EPS), w, f"{p}.mlp", ident)
    return (P.rms_norm(x, w["model.norm.weight"], EPS) @ w["lm_head.weight"].T).float()


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from pyre_amd.weights import write_random_model

    register_part("mixer", "running_mean", RunningMean)
    register_architecture(ToyConfig.architecture, ToyConfig, build_toy)
    cfg = ToyConfig()
    folder = tmp_path_factory.mktemp("toy")
    write_random_model(folder, cfg, seed=7, std=0.08, gain_std=0.1)
    yield cfg, folder, P.read_weights(folder)
    unregister_architecture(ToyConfig.architecture)


def _engine(folder, dtype, **kw):
    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.engine import Engine

    args = dict(dtype=dtype, page_size=8, max_cached_tokens=512, max_num_seqs=3, max_num_batched_tokens=256,
                use_graphs=False)
    args.update(kw)
    return Engine.from_folder(folder, EngineConfig(**args))


def test_toy_model_is_built_from_the_registry(toy):
    cfg, folder, w = toy
    eng = _engine(folder, "float32")
    m = eng.cache
    # entries 0 and 3 (full attention, own caches) share a group, entry 2 (window) has its own,
    # entry 1 keeps state, entry 4 reads entry 0's cache and keeps nothing
    assert [g.entries for g in m.page_groups] == [[0, 3], [2]]
    assert m.page_groups[1].spec.window == cfg.window
    assert [g.entries for g in m.state_groups] == [[1]] and 4 not in m.group_of_entry
    assert "model.layers.1.mix.weight" in w and "model.layers.1.self_attn.q_proj.weight" not in w


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 3e-2)])
def test_toy_model_whole_portions_and_mixed(toy, dtype, tol):
    cfg, folder, w = toy
    reqs = {r: random_ids(cfg.vocab_size, n, seed=n) for r, n in (("a", 61), ("b", 45), ("c", 90), ("d", 33))}
    want = {r: plain_toy(w, cfg, ids) for r, ids in reqs.items()}
    eng = _engine(folder, dtype)
    # whole
    got = replay(eng, [([(r, ids, list(range(len(ids))))], [r]) for r, ids in reqs.items()])
    bad, _ = first_bad(got, want, tol)
    assert bad is None, bad
    # portions of changing size: the state and the window's released pages carry across steps
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


def test_window_pages_come_back_while_a_request_runs(toy):
    cfg, folder, w = toy
    eng = _engine(folder, "float32")
    ids = random_ids(cfg.vocab_size, 200, seed=3)
    want = {"x": plain_toy(w, cfg, ids)}
    steps = [([("x", ids[:150], [149])], [])] + [([("x", ids[i:i + 1], [0])], []) for i in range(150, 200)]
    got = replay(eng, steps)
    bad, _ = first_bad(got, want, 1e-5)
    assert bad is None, bad
    full, win = eng.cache.page_groups
    assert full.allocator.num_used == 25 and win.allocator.num_used <= 4      # 200 tokens / 8; window 20 -> at most 4 pages
    eng.finish("x")
