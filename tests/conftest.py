"""Shared fixtures: tiny model folders with random weights, made in a temporary folder."""

from __future__ import annotations

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(Path(__file__).resolve().parent)):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu); everything else runs on the CPU")


#: The two tiny shapes differ in every size and option: layers, width, heads and
#: groups, head size (16 / 12), feed-forward width, vocabulary, theta, eps, tied or
#: untied head, gains of 1 or random.
TINY = {
    "tiny-a": dict(seed=0, std=0.02, gain_std=0.0),
    "tiny-b": dict(seed=1, std=0.05, gain_std=0.1),
    "tiny-c": dict(seed=2, std=0.04, gain_std=0.05),
    "tiny-d": dict(seed=3, std=0.1, gain_std=0.2),
}

#: A third shape whose head size (32) and 16-token pages are taken by the MFMA
#: attention kernels in bfloat16; three query heads per key/value head.
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 80,
    "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 32, "intermediate_size": 144,
    "vocab_size": 777, "rope_theta": 5e4, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
    "max_position_embeddings": 1024,
}


#: Awkward sizes: nothing is a multiple of 8, heads * head_dim is not the width, one
#: key/value head for three query heads, a single layer.
TINY_D = {
    "architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 1, "hidden_size": 70,
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 10, "intermediate_size": 50,
    "vocab_size": 131, "rope_theta": 300.0, "rms_norm_eps": 1e-3, "tie_word_embeddings": True,
    "max_position_embeddings": 300,
}


def tiny_config(name):
    from pyre_amd.config import preset
    from pyre_amd.registry import config_from_dict

    custom = {"tiny-c": TINY_C, "tiny-d": TINY_D}
    return config_from_dict(custom[name]) if name in custom else preset(name)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """name -> folder with config.json + model.safetensors (bfloat16 weights)."""
    from pyre_amd.weights import write_random_model

    out = {}
    for name, kw in TINY.items():
        d = tmp_path_factory.mktemp(name.replace("-", "_"))
        write_random_model(d, tiny_config(name), **kw)
        out[name] = d
    return out


@pytest.fixture(scope="session")
def plain_models(model_dirs):
    """name -> (config dict, float64 weights) of the plain implementation."""
    import plain_qwen2 as P

    return {n: (P.read_config(d), P.read_weights(d)) for n, d in model_dirs.items()}
