"""A toy mixer whose per-token record is not keys and values: one compressed vector per
token, kept as ``[page, token, r]``, and a pair of float32 weights per token kept transposed,
``[page, 2, token]``. It is defined, registered, built and stepped here without a change to
the framework's files: the cache manager allocates whatever a mixer's description says, and
the mixer alone knows what its pages mean. The toy stands for no model of anyone's.

    z_t = h_t Wc^T                    (r numbers, stored in the engine's element type)
    a_t = sigmoid(h_t . wa), b_t = 1  (stored as float32 [2])
    out_t = Wo (sum_{j <= t} a_j z_j / sum_{j <= t} a_j b_j)
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch

import plain_qwen2 as P
from helpers import cut, first_bad, random_ids, replay
from pyre_amd.config.model import ModelConfig
from pyre_amd.hip.ops import Partials
from pyre_amd.parts.base import (BlockSpec, EmbeddingSpec, LayerCall, LMHeadSpec, Mixer, ModelSpec, PagedCacheSpec,
                                 PagedTensorSpec, RMSNormSpec, SwiGLUSpec, TensorSpec, register_part)
from pyre_amd.registry import register_architecture, unregister_architecture

pytestmark = pytest.mark.gpu

R, INTER, EPS = 12, 40, 1e-5


@dataclass(frozen=True)
class LatentSpec:
    hidden_size: int
    rank: int
    prefix: str
    kind: ClassVar[str] = "toy_latent"


class LatentMemory(Mixer):
    def __init__(self, spec):
        self.spec = spec

    def cache_spec(self):
        return PagedCacheSpec((PagedTensorSpec("latent", (self.spec.rank,), token_axis=0),
                               PagedTensorSpec("weights", (2,), token_axis=1, dtype="float32")))

    def tensor_specs(self):
        h, r, p = self.spec.hidden_size, self.spec.rank, self.spec.prefix
        return [TensorSpec(f"{p}.compress.weight", (r, h)), TensorSpec(f"{p}.score.weight", (1, h)),
                TensorSpec(f"{p}.expand.weight", (h, r))]

    def bind(self, tensors, runtime):
        p = self.spec.prefix
        self.wc, self.wa, self.wo = (tensors[f"{p}.{n}.weight"].float() for n in ("compress", "score", "expand"))

    def forward(self, ctx, h, cache):
        hb, r = ctx.host, self.spec.rank
        ps = cache.page_size
        latent, weights = cache["latent"], cache["weights"]          # [pages, ps, r], [pages, 2, ps]
        assert latent.shape[1:] == (ps, r) and weights.shape[1:] == (2, ps) and weights.dtype == torch.float32
        x = h[:ctx.n_tokens].float()
        z = (x @ self.wc.T).to(latent.dtype)
        a = torch.sigmoid(x @ self.wa.T)[:, 0]
        slots = cache.slots[:ctx.n_tokens].long()
        page, off = slots // ps, slots % ps
        latent[page, off] = z                                        # this step's records, then read everything back
        weights[page, 0, off] = a
        weights[page, 1, off] = 1.0
        out = torch.empty(ctx.n_tokens, self.spec.hidden_size, device=h.device, dtype=torch.float32)
        for s in range(hb.n_seqs):
            q0, q1, n_ctx = int(hb.q_start[s]), int(hb.q_start[s + 1]), int(hb.ctx_len[s])
            pages = cache.table[s, :-(-n_ctx // ps)].long()
            zs = latent[pages].reshape(-1, r)[:n_ctx].float()
            ws = weights[pages].permute(0, 2, 1).reshape(-1, 2)[:n_ctx]
            num = torch.cumsum(ws[:, :1] * zs, 0)[n_ctx - (q1 - q0):]
            den = torch.cumsum(ws[:, 0] * ws[:, 1], 0)[n_ctx - (q1 - q0):]
            out[q0:q1] = (num / den[:, None]) @ self.wo.T
        return Partials(out.view(1, ctx.n_tokens, -1))


@dataclass(frozen=True)
class LatentToyConfig(ModelConfig):
    architecture: ClassVar[str] = "ToyLatentForCausalLM"
    hidden_size: int = 40
    vocab_size: int = 97

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["hidden_size"], raw["vocab_size"])

    def to_dict(self):
        return {"architectures": [self.architecture], "hidden_size": self.hidden_size, "vocab_size": self.vocab_size}


def build(cfg) -> ModelSpec:
    H = cfg.hidden_size

    def block(i):
        p = f"model.layers.{i}"
        return BlockSpec(LatentSpec(H, R, f"{p}.memory"), RMSNormSpec(H, EPS, f"{p}.input_layernorm"),
                         SwiGLUSpec(H, INTER, f"{p}.mlp"), RMSNormSpec(H, EPS, f"{p}.post_attention_layernorm"))

    return ModelSpec(H, cfg.vocab_size, 256, EmbeddingSpec(cfg.vocab_size, H), (block(0), block(1)),
                     (LayerCall(0), LayerCall(1)), RMSNormSpec(H, EPS, "model.norm"), LMHeadSpec(cfg.vocab_size, H))


def plain(w, ids, rounding=None):
    """Whole sequence, float64; ``rounding`` rounds what a 16-bit engine stores."""
    rnd = (lambda t: t.to(rounding).to(t.dtype)) if rounding is not None else (lambda t: t)
    x = P.embed(torch.as_tensor(ids), w["model.embed_tokens.weight"])
    for i in range(2):
        p = f"model.layers.{i}"
        h = rnd(P.rms_norm(x, w[f"{p}.input_layernorm.weight"], EPS))
        z = rnd(h @ w[f"{p}.memory.compress.weight"].T)
        a = torch.sigmoid(h @ w[f"{p}.memory.score.weight"].T)
        mix = torch.cumsum(a * z, 0) / torch.cumsum(a, 0)
        x = x + mix @ w[f"{p}.memory.expand.weight"].T
        x = x + P.swiglu(rnd(P.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], EPS)), w, f"{p}.mlp", rnd)
    return (rnd(P.rms_norm(x, w["model.norm.weight"], EPS)) @ w["lm_head.weight"].T).float()


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from pyre_amd.weights import write_random_model

    register_part("mixer", "toy_latent", LatentMemory)
    register_architecture(LatentToyConfig.architecture, LatentToyConfig, build)
    cfg = LatentToyConfig()
    folder = tmp_path_factory.mktemp("toy_latent")
    write_random_model(folder, cfg, seed=4, std=0.2, gain_std=0.1)
    yield cfg, folder, P.read_weights(folder)
    unregister_architecture(LatentToyConfig.architecture)


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 3e-2)])
@pytest.mark.parametrize("poison", [False, True])
def test_a_mixer_with_a_page_layout_of_its_own(toy, dtype, tol, poison):
    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.engine import Engine

    cfg, folder, w = toy
    eng = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=8, num_pages=24, max_num_seqs=3,
                                                  max_num_batched_tokens=256, use_graphs=False, debug_poison=poison))
    g, = eng.cache.page_groups
    assert g.entries == [0, 1] and set(g.tensors) == {"latent", "weights"}
    assert g.tensors["latent"].shape == (2, 24, 8, R) and g.tensors["weights"].shape == (2, 24, 2, 8)
    if poison:
        assert all(torch.isnan(t).all() for t in g.tensors.values())
    reqs = {r: random_ids(cfg.vocab_size, n, seed=n) for r, n in (("a", 61), ("b", 45), ("c", 70), ("d", 33))}
    want = {r: plain(w, ids, torch.bfloat16 if dtype == "bfloat16" else None) for r, ids in reqs.items()}
    # three live at a time in portions of changing size (pages and slots are used again by the fourth)
    fed = {r: 0 for r in reqs}
    portions = {r: cut(len(ids), [7, 2, 19, 3, 1, 30]) for r, ids in reqs.items()}
    live, waiting, steps = [], list(reqs), []
    while live or waiting:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            n = portions[r].pop(0)
            entries.append((r, reqs[r][fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
            if not portions[r]:
                end.append(r)
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    got = replay(eng, steps)
    assert len(got) == sum(len(i) for i in reqs.values())
    bad, _ = first_bad(got, want, tol)
    assert bad is None, bad
    eng.cache.check_invariants()
    assert g.allocator.num_used == 0
    if poison:
        assert all(torch.isnan(t).all() for t in g.tensors.values())   # everything went back, and was marked
