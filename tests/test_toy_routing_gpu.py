"""More of the framework's generality, with parts that exist only in this file: a
feed-forward that routes every token to one of three small experts (router logits
and their softmax in 32 bits), a position encoding of another kind (rotation of half
of each head, angles of half the position) and a layer without any position
encoding, put together into an architecture of their own. Nothing under pyre_amd/
is changed to run them."""

from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch

import plain_qwen2 as P
from helpers import cut, first_bad, random_ids, replay
from pyre_amd.config.model import ModelConfig
from pyre_amd.hip.ops import Partials
from pyre_amd.parts.base import (AttentionSpec, BlockSpec, EmbeddingSpec, FeedForward, LayerCall, LMHeadSpec,
                                 ModelSpec, NoPositionSpec, PositionEncoding, RMSNormSpec, SwiGLUSpec,
                                 TensorSpec, register_part)
from pyre_amd.registry import register_architecture, unregister_architecture

pytestmark = pytest.mark.gpu

H, NQ, NKV, HD, INTER, EXPERTS, EXPERT_INTER, EPS, THETA, VOCAB = 40, 4, 1, 16, 56, 3, 24, 1e-5, 500.0, 97
ROT, POSITION_SCALE = 8, 0.5


# ----------------------------------------------------------------------------- a routed feed-forward

@dataclass(frozen=True)
class Top1ExpertsSpec:
    hidden_size: int
    expert_size: int
    num_experts: int
    prefix: str
    kind: ClassVar[str] = "toy_top1_experts"


class Top1Experts(FeedForward):
    """out = p_e * W2_e relu(W1_e h) with e = argmax of the router's logits and p = their softmax."""

    def __init__(self, spec):
        self.spec = spec

    def tensor_specs(self):
        s, p = self.spec, self.spec.prefix
        specs = [TensorSpec(f"{p}.router.weight", (s.num_experts, s.hidden_size))]
        for e in range(s.num_experts):
            specs += [TensorSpec(f"{p}.experts.{e}.w1.weight", (s.expert_size, s.hidden_size)),
                      TensorSpec(f"{p}.experts.{e}.w2.weight", (s.hidden_size, s.expert_size))]
        return specs

    def bind(self, tensors, runtime):
        p = self.spec.prefix
        self.router = tensors[f"{p}.router.weight"].float()
        self.w1 = [tensors[f"{p}.experts.{e}.w1.weight"].float() for e in range(self.spec.num_experts)]
        self.w2 = [tensors[f"{p}.experts.{e}.w2.weight"].float() for e in range(self.spec.num_experts)]

    def forward(self, ctx, h):
        n = ctx.n_tokens
        x = h[:n].float()
        probs = torch.softmax(x @ self.router.T, dim=-1)
        choice = probs.argmax(-1)
        out = torch.zeros(n, self.spec.hidden_size, device=h.device, dtype=torch.float32)
        for e in range(self.spec.num_experts):  # tokens of one expert together, whatever request they are of
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                y = torch.relu(x[rows] @ self.w1[e].T) @ self.w2[e].T
                out[rows] = probs[rows, e, None] * y
        return Partials(out.view(1, n, self.spec.hidden_size))


# ----------------------------------------------------------------------------- another position encoding

@dataclass(frozen=True)
class HalfSpeedRotarySpec:
    rotary_dim: int
    theta: float
    scale: float
    kind: ClassVar[str] = "toy_half_speed_rotary"


class HalfSpeedRotary(PositionEncoding):
    """Rotates the first ``rotary_dim`` elements of a head by angles of ``scale`` * position."""

    def __init__(self, spec):
        self.spec = spec
        self._tables = None

    def rotary(self, runtime):
        if self._tables is None:
            s = self.spec
            inv_freq = 1.0 / (s.theta ** (torch.arange(0, s.rotary_dim, 2, dtype=torch.float32) / s.rotary_dim))
            ang = torch.outer(torch.arange(runtime.max_positions, dtype=torch.float32) * s.scale, inv_freq)
            self._tables = (ang.cos().to(runtime.device).contiguous(), ang.sin().to(runtime.device).contiguous())
        return self._tables[0], self._tables[1], self.spec.rotary_dim


# ----------------------------------------------------------------------------- the architecture

@dataclass(frozen=True)
class RoutedConfig(ModelConfig):
    architecture: ClassVar[str] = "ToyRoutedForCausalLM"
    num_experts: int = EXPERTS

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["num_experts"])

    def to_dict(self):
        return {"architectures": [self.architecture], "num_experts": self.num_experts}


def build_routed(cfg: RoutedConfig) -> ModelSpec:
    def norms(i):
        p = f"model.layers.{i}"
        return RMSNormSpec(H, EPS, f"{p}.input_layernorm"), RMSNormSpec(H, EPS, f"{p}.post_attention_layernorm")

    n0, n1 = norms(0), norms(1)
    layers = (
        BlockSpec(AttentionSpec(H, NQ, NKV, HD, HalfSpeedRotarySpec(ROT, THETA, POSITION_SCALE), "model.layers.0.self_attn"),
                  n0[0], Top1ExpertsSpec(H, EXPERT_INTER, cfg.num_experts, "model.layers.0.moe"), n0[1]),
        BlockSpec(AttentionSpec(H, NQ, NKV, HD, NoPositionSpec(), "model.layers.1.self_attn"),
                  n1[0], SwiGLUSpec(H, INTER, "model.layers.1.mlp"), n1[1]),
    )
    return ModelSpec(H, VOCAB, 256, EmbeddingSpec(VOCAB, H), layers, (LayerCall(0), LayerCall(1)),
                     RMSNormSpec(H, EPS, "model.norm"), LMHeadSpec(VOCAB, H))


def plain_routed(w, ids):
    """The same model, whole sequence, float64, from the plain implementation's parts."""
    ids = torch.as_tensor(ids)
    S = len(ids)
    x = P.embed(ids, w["model.embed_tokens.weight"])
    c = {"num_attention_heads": NQ, "num_key_value_heads": NKV, "head_dim": HD}
    ident = lambda t: t  # noqa: E731
    # layer 0: only the first ROT elements of a head turn, by half the position: cos = 1 and sin = 0 elsewhere.
    # The plain rotation pairs element j with j + HD/2, the engine's partial rotation j with j + ROT/2 inside
    # the rotated part, so the plain tables are laid out per element here.
    inv_freq = 1.0 / (THETA ** (torch.arange(0, ROT, 2, dtype=torch.float32) / ROT))
    ang = torch.outer(torch.arange(S, dtype=torch.float32) * POSITION_SCALE, inv_freq).double()

    def rotate(t):  # (heads, S, HD)
        a, b, rest = t[..., :ROT // 2], t[..., ROT // 2:ROT], t[..., ROT:]
        return torch.cat([a * ang.cos() - b * ang.sin(), b * ang.cos() + a * ang.sin(), rest], dim=-1)

    def attention(h, prefix, turn):
        q = (h @ w[f"{prefix}.q_proj.weight"].T + w[f"{prefix}.q_proj.bias"]).view(S, NQ, HD).transpose(0, 1)
        k = (h @ w[f"{prefix}.k_proj.weight"].T + w[f"{prefix}.k_proj.bias"]).view(S, NKV, HD).transpose(0, 1)
        v = (h @ w[f"{prefix}.v_proj.weight"].T + w[f"{prefix}.v_proj.bias"]).view(S, NKV, HD).transpose(0, 1)
        if turn:
            q, k = rotate(q), rotate(k)
        out = P.causal_attention(q, P.repeat_kv(k, NQ // NKV), P.repeat_kv(v, NQ // NKV), HD ** -0.5)
        return out.transpose(0, 1).reshape(S, NQ * HD) @ w[f"{prefix}.o_proj.weight"].T

    p = "model.layers.0"
    x = x + attention(P.rms_norm(x, w[f"{p}.input_layernorm.weight"], EPS), f"{p}.self_attn", True)
    h = P.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], EPS)
    probs = torch.softmax(h @ w[f"{p}.moe.router.weight"].T, dim=-1)
    choice = probs.argmax(-1)
    y = torch.zeros_like(h)
    for t in range(S):
        e = int(choice[t])
        y[t] = probs[t, e] * (torch.relu(h[t] @ w[f"{p}.moe.experts.{e}.w1.weight"].T) @ w[f"{p}.moe.experts.{e}.w2.weight"].T)
    x = x + y
    p = "model.layers.1"
    x = x + attention(P.rms_norm(x, w[f"{p}.input_layernorm.weight"], EPS), f"{p}.self_attn", False)
    x = x + P.swiglu(P.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], EPS), w, f"{p}.mlp", ident)
    return (P.rms_norm(x, w["model.norm.weight"], EPS) @ w["lm_head.weight"].T).float(), choice


@pytest.fixture(scope="module")
def routed(tmp_path_factory):
    from pyre_amd.weights import write_random_model

    register_part("feed_forward", Top1ExpertsSpec.kind, Top1Experts)
    register_part("position", HalfSpeedRotarySpec.kind, HalfSpeedRotary)
    register_architecture(RoutedConfig.architecture, RoutedConfig, build_routed)
    folder = tmp_path_factory.mktemp("routed")
    write_random_model(folder, RoutedConfig(), seed=11, std=0.2, gain_std=0.1)
    yield folder, P.read_weights(folder)
    unregister_architecture(RoutedConfig.architecture)


def test_routed_model_whole_portions_and_mixed(routed):
    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.engine import Engine

    folder, w = routed
    reqs = {r: random_ids(VOCAB, n, seed=n) for r, n in (("a", 70), ("b", 33), ("c", 51))}
    want, used = {}, set()
    for r, ids in reqs.items():
        want[r], choice = plain_routed(w, ids)
        used |= set(choice.tolist())
    assert used == set(range(EXPERTS))  # every expert takes tokens: the routing is exercised
    eng = Engine.from_folder(folder, EngineConfig(dtype="float32", page_size=8, max_cached_tokens=256, max_num_seqs=3,
                                                  max_num_batched_tokens=128, use_graphs=False))
    assert "model.layers.0.moe.experts.2.w2.weight" in w and "model.layers.0.mlp.gate_proj.weight" not in w
    # whole
    got = replay(eng, [([(r, ids, list(range(len(ids))))], [r]) for r, ids in reqs.items()])
    bad, _ = first_bad(got, want, 2e-5)
    assert bad is None, bad
    # portions of changing size, then all three mixed in one batch per step
    steps = []
    for r, ids in reqs.items():
        pos, parts = 0, cut(len(ids), [9, 2, 14, 1, 3])
        for k, n in enumerate(parts):
            steps.append(([(r, ids[pos:pos + n], list(range(n)))], [r] if k == len(parts) - 1 else []))
            pos += n
    fed = {r: 0 for r in reqs}
    k = 0
    while any(fed[r] < len(reqs[r]) for r in reqs):
        entries, end = [], []
        for r in reqs:
            if fed[r] == len(reqs[r]):
                continue
            n = min([4, 1, 11, 2][k % 4], len(reqs[r]) - fed[r])
            k += 1
            entries.append((r, reqs[r][fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        steps.append((entries, end))
    got = replay(eng, steps)
    bad, _ = first_bad(got, want, 2e-5)
    assert bad is None, bad
    assert all(g.allocator.num_used == 0 for g in eng.cache.page_groups)
