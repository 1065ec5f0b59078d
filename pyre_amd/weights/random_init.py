"""Random weights from a configuration and a seed, as tensors or as a model folder
(``config.json`` + ``model.safetensors``) that the ordinary loader reads.

The reference has no such mode; a bare ``PyreQwen2(cfg)`` carries torch's default
initialisation, which its loader calls a failure mode (`pyre/loader.py:54-57`).
"""

from __future__ import annotations

from pathlib import Path

import torch

from pyre_amd.config.model import ModelConfig
from pyre_amd.parts.base import TensorSpec

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def model_tensor_specs(config: ModelConfig) -> list[TensorSpec]:
    from pyre_amd.parts.model import LayeredModel
    from pyre_amd.registry import get_architecture

    return LayeredModel(get_architecture(config.architecture).build(config)).tensor_specs()


def random_state(specs: list[TensorSpec], seed: int, std: float = 0.02, gain_std: float = 0.0,
                 dtype: str | torch.dtype = "bfloat16", device: str | torch.device = "cpu") -> dict[str, torch.Tensor]:
    """One seeded generator; tensors are drawn in float32 in the order of ``specs``
    and rounded to ``dtype``. Matrices, embeddings and biases ~ N(0, std); norm
    gains = 1 + N(0, gain_std); tensors with an alias (a tied head) are left out."""
    dt = _STORE[dtype] if isinstance(dtype, str) else dtype
    device = torch.device(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out: dict[str, torch.Tensor] = {}
    for s in specs:
        if s.alias_of is not None:
            continue
        if s.init == "normal":
            t = torch.randn(s.shape, generator=gen, dtype=torch.float32, device=device) * std
        elif s.init == "gain":
            t = torch.ones(s.shape, dtype=torch.float32, device=device)
            if gain_std:
                t = t + torch.randn(s.shape, generator=gen, dtype=torch.float32, device=device) * gain_std
        elif s.init == "zeros":
            t = torch.zeros(s.shape, dtype=torch.float32, device=device)
        elif s.init == "int":
            out[s.name] = torch.zeros(s.shape, dtype=torch.int32, device=device)
            continue
        else:
            raise ValueError(f"tensor {s.name}: unknown init {s.init!r}")
        out[s.name] = t.to(dt)
    return out


def write_random_model(folder: str | Path, config: ModelConfig, seed: int, std: float = 0.02,
                       gain_std: float = 0.0, dtype: str = "bfloat16") -> Path:
    """Write ``config.json`` and ``model.safetensors`` into ``folder``."""
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    config.save(folder)
    state = random_state(model_tensor_specs(config), seed, std, gain_std, dtype)
    save_file({k: v.contiguous() for k, v in state.items()}, str(folder / "model.safetensors"))
    return folder
