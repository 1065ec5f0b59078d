"""Weights from safetensors, bound by tensor name (`pyre/loader.py:33-79`).

The reference merges every shard into one dictionary and lets
``load_state_dict(strict=False)`` find what is missing or unexpected
(`pyre/loader.py:46-72`); a wrong shape surfaces as torch's own error. Here the
model's parts name the tensors they need (name and shape), the files' headers are
checked against that list before a byte of data is read, and everything that is
wrong is reported in one error.

Element types: a tensor stored in bfloat16 stays bfloat16 (float32 when the engine
runs in 32-bit: the widening is exact); a tensor stored in float32 stays float32 in
either mode; float16 is converted to the engine's type; integer tables become int32.
"""

from __future__ import annotations

from pathlib import Path

import torch
from safetensors import safe_open

from pyre_amd.parts.base import TensorSpec

_MAX_LISTED = 12


class WeightsError(RuntimeError):
    """The checkpoint does not fit the model: lists missing and unexpected
    tensors and tensors of the wrong shape."""

    def __init__(self, folder, missing, unexpected, wrong_shape):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)

        def some(items):
            items = list(items)
            more = f" ... and {len(items) - _MAX_LISTED} more" if len(items) > _MAX_LISTED else ""
            return ", ".join(str(i) for i in items[:_MAX_LISTED]) + more

        lines = [f"checkpoint in {folder} does not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): {some(self.missing)}")
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): {some(self.unexpected)}")
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + some(
                f"{n} is {tuple(got)}, expected {tuple(want)}" for n, got, want in self.wrong_shape))
        super().__init__("\n".join(lines))


def runtime_dtype(stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return compute  # bfloat16 / float16 -> the engine's type


def checkpoint_files(folder: str | Path) -> list[Path]:
    files = sorted(Path(folder).glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors found in {folder}")  # pyre/loader.py:47-48
    return files


def checkpoint_index(folder: str | Path) -> dict[str, tuple[Path, tuple[int, ...]]]:
    """name -> (file, shape), from the files' headers only."""
    index: dict[str, tuple[Path, tuple[int, ...]]] = {}
    for f in checkpoint_files(folder):
        with safe_open(str(f), framework="pt") as sf:
            for name in sf.keys():
                index[name] = (f, tuple(sf.get_slice(name).get_shape()))
    return index


def check_against(specs: list[TensorSpec], index: dict, folder) -> None:
    wanted = {s.name: s for s in specs}
    missing, wrong = [], []
    for s in specs:
        if s.name not in index:
            if s.alias_of is not None and s.alias_of in index:
                continue  # a tied tensor the file leaves out (pyre/loader.py:58-61)
            missing.append(s.name)
        elif tuple(index[s.name][1]) != tuple(s.shape):
            wrong.append((s.name, index[s.name][1], s.shape))
    unexpected = [n for n in index if n not in wanted]
    if missing or unexpected or wrong:
        raise WeightsError(folder, missing, unexpected, wrong)


def load_weights(folder: str | Path, specs: list[TensorSpec], device, compute_dtype: torch.dtype) -> dict[str, torch.Tensor]:
    """Read every tensor ``specs`` names onto ``device``."""
    index = checkpoint_index(folder)
    check_against(specs, index, folder)
    by_file: dict[Path, list[str]] = {}
    for s in specs:
        if s.name in index:
            by_file.setdefault(index[s.name][0], []).append(s.name)
    out: dict[str, torch.Tensor] = {}
    for f, names in by_file.items():
        with safe_open(str(f), framework="pt") as sf:
            for name in names:
                t = sf.get_tensor(name)
                out[name] = t.to(device=device, dtype=runtime_dtype(t.dtype, compute_dtype))
    for s in specs:
        if s.name not in out:
            out[s.name] = out[s.alias_of]  # same memory: a tied head costs nothing
    return out


def adopt_state(state: dict[str, torch.Tensor], specs: list[TensorSpec], device, compute_dtype: torch.dtype) -> dict[str, torch.Tensor]:
    """The same checks and conversions for tensors that are already in memory."""
    index = {n: (None, tuple(t.shape)) for n, t in state.items()}
    check_against(specs, index, "<memory>")
    out = {n: t.to(device=device, dtype=runtime_dtype(t.dtype, compute_dtype)) for n, t in state.items()}
    for s in specs:
        if s.name not in out:
            out[s.name] = out[s.alias_of]
    return out
