"""A plain, slow Qwen2 forward pass: whole sequences, no cache, one function per
part, written from the reference's formulas (each function cites file:line of the
reference repository, pyre/model.py and its neighbours). It shares no code with
``pyre_amd``: it reads ``config.json`` with ``json`` and the weights with
``safetensors`` itself.

Everything runs where the weights lie (the CPU, unless a test moves them: the shapes of
real models are too slow there) in ``dtype`` (float64 by default: the engine's float32
path is then compared with something more exact than itself). ``rounding`` emulates
a 16-bit engine: the values that such an engine stores in 16 bits (normed rows,
rotated queries and keys, values, attention output, gated activations) are rounded
to that type and widened again; all arithmetic stays in ``dtype``.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


# ----------------------------------------------------------------------------- loading

def read_config(folder) -> dict:
    """The keys and defaults of pyre/config.py:34-62."""
    raw = json.loads((Path(folder) / "config.json").read_text())
    hidden, heads = raw["hidden_size"], raw["num_attention_heads"]
    return {
        "hidden_size": hidden,
        "intermediate_size": raw["intermediate_size"],
        "num_hidden_layers": raw["num_hidden_layers"],
        "num_attention_heads": heads,
        "num_key_value_heads": raw.get("num_key_value_heads", heads),
        "vocab_size": raw["vocab_size"],
        "rms_norm_eps": raw.get("rms_norm_eps", 1e-6),
        "rope_theta": float(raw.get("rope_theta", 10000.0)),
        "tie_word_embeddings": bool(raw.get("tie_word_embeddings", False)),
        "head_dim": raw.get("head_dim") or hidden // heads,
    }


def read_weights(folder, dtype=torch.float64) -> dict[str, torch.Tensor]:
    """All tensors of all shards, widened to ``dtype`` (pyre/loader.py:46-61)."""
    state = {}
    for f in sorted(Path(folder).glob("*.safetensors")):
        with safe_open(str(f), framework="pt") as sf:
            for name in sf.keys():
                state[name] = sf.get_tensor(name).to(dtype)
    if "lm_head.weight" not in state:  # tied head: pyre/loader.py:58-61
        state["lm_head.weight"] = state["model.embed_tokens.weight"]
    return state


def _rounder(rounding):
    if rounding is None:
        return lambda x: x
    return lambda x: x.to(rounding).to(x.dtype)


# ----------------------------------------------------------------------------- parts

def embed(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """pyre/model.py:196: x = embed_tokens(ids), no scaling."""
    return table[ids]


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """pyre/model.py:33-38: x * rsqrt(mean(x^2) + eps), then times the gain."""
    var = x.pow(2).mean(-1, keepdim=True)
    return weight * (x * torch.rsqrt(var + eps))


def rope_tables(n: int, head_dim: int, theta: float, dtype=torch.float64):
    """pyre/model.py:41-51: float32 inv_freq, angles and cos/sin, both halves of the
    table equal; then widened to the computing type."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    t = torch.arange(n, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """pyre/model.py:54-56: (-second half, first half)."""
    half = x.shape[-1] // 2
    return torch.cat([-x[..., half:], x[..., :half]], dim=-1)


def apply_rope(q, k, cos, sin):
    """pyre/model.py:59-63. q, k: (heads, S, D); cos, sin: (S, D)."""
    return q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """pyre/model.py:66-72: (KV, S, D) -> (KV * n_rep, S, D), query head i reads i // n_rep."""
    return x if n_rep == 1 else x.repeat_interleave(n_rep, dim=0)


def causal_attention(q, k, v, scale: float, window: int = 0) -> torch.Tensor:
    """pyre/model.py:109-123: softmax(q k^T * scale + causal mask) v, one head set.
    q, k, v: (heads, S, D). ``window`` > 0 (not in the reference) hides keys more
    than window-1 positions back."""
    S = q.shape[1]
    scores = torch.matmul(q, k.transpose(-1, -2)) * scale
    i = torch.arange(S, device=q.device).unsqueeze(1)
    j = torch.arange(S, device=q.device).unsqueeze(0)
    hidden = j > i
    if window > 0:
        hidden = hidden | (j < i - window + 1)
    scores = scores.masked_fill(hidden, -math.inf)
    return torch.matmul(torch.softmax(scores, dim=-1), v)


def attention_block(h, w: dict, prefix: str, cfg: dict, cos, sin, rnd, window: int = 0, kv=None, keep=None) -> torch.Tensor:
    """pyre/model.py:89-125 for one sequence at start_pos = 0. h: (S, H).
    Not in the reference: ``window``; ``kv`` = rotated keys and values of another
    layer to attend over instead of this layer's own; ``keep`` = a list that
    receives this layer's (keys, values)."""
    S = h.shape[0]
    nq, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = (h @ w[f"{prefix}.q_proj.weight"].T + w[f"{prefix}.q_proj.bias"]).view(S, nq, hd).transpose(0, 1)
    k = (h @ w[f"{prefix}.k_proj.weight"].T + w[f"{prefix}.k_proj.bias"]).view(S, nkv, hd).transpose(0, 1)
    v = (h @ w[f"{prefix}.v_proj.weight"].T + w[f"{prefix}.v_proj.bias"]).view(S, nkv, hd).transpose(0, 1)
    q, k = apply_rope(q, k, cos[:S], sin[:S])
    q, k, v = rnd(q), rnd(k), rnd(v)
    if keep is not None:
        keep.append((k, v))
    if kv is not None:
        k, v = kv
    k, v = repeat_kv(k, nq // nkv), repeat_kv(v, nq // nkv)
    out = causal_attention(q, k, v, hd ** -0.5, window)
    out = rnd(out.transpose(0, 1).reshape(S, nq * hd))
    return out @ w[f"{prefix}.o_proj.weight"].T


def swiglu(h, w: dict, prefix: str, rnd) -> torch.Tensor:
    """pyre/model.py:138-139: down(silu(gate(x)) * up(x))."""
    g = h @ w[f"{prefix}.gate_proj.weight"].T
    u = h @ w[f"{prefix}.up_proj.weight"].T
    return rnd(g * torch.sigmoid(g) * u) @ w[f"{prefix}.down_proj.weight"].T


def decoder_layer(x, w: dict, i: int, cfg: dict, cos, sin, rnd) -> torch.Tensor:
    """pyre/model.py:150-153: two pre-norm residual steps."""
    p = f"model.layers.{i}"
    eps = cfg["rms_norm_eps"]
    x = x + attention_block(rnd(rms_norm(x, w[f"{p}.input_layernorm.weight"], eps)), w, f"{p}.self_attn", cfg, cos, sin, rnd)
    x = x + swiglu(rnd(rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)), w, f"{p}.mlp", rnd)
    return x


def forward(w: dict, cfg: dict, ids, rounding=None, return_hidden: bool = False):
    """pyre/model.py:188-201 without a cache: token ids (S,) -> logits (S, vocab)."""
    table = w["model.embed_tokens.weight"]
    ids = torch.as_tensor(ids, dtype=torch.long, device=table.device)
    rnd = _rounder(rounding)
    x = embed(ids, table)
    cos, sin = rope_tables(len(ids), cfg["head_dim"], cfg["rope_theta"], x.dtype)
    cos, sin = cos.to(x.device), sin.to(x.device)
    hidden = []
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, w, i, cfg, cos, sin, rnd)
        hidden.append(x)
    logits = rnd(rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])) @ w["lm_head.weight"].T
    return (logits, hidden) if return_hidden else logits


def greedy(w: dict, cfg: dict, prompt: list[int], max_new_tokens: int, eos_id=None) -> list[int]:
    """pyre/model.py:203-215: recompute everything for every token, argmax of the last row."""
    ids = list(prompt)
    new = []
    for _ in range(max_new_tokens):
        nxt = int(forward(w, cfg, ids)[-1].argmax())
        ids.append(nxt)
        new.append(nxt)
        if eos_id is not None and nxt == eos_id:
            break
    return new


# ----------------------------------------------------------------------------- sampling twin

def sample_inverse_cdf(logits: torch.Tensor, temperature: float, u: float) -> int:
    """softmax(logits / T), cumulative sum in vocabulary order, first index whose
    cumulative probability exceeds u. (The reference only has argmax,
    pyre/scheduler.py:80,94; T -> 0 reduces to it.)"""
    if temperature <= 0:
        return int(logits.argmax())
    p = torch.softmax(logits.double() / temperature, dim=-1)
    c = torch.cumsum(p, dim=-1)
    return int(min(torch.searchsorted(c, torch.tensor(u, dtype=c.dtype), right=True), len(p) - 1))
