"""Weights from safetensors, bound by tensor name (`pyre/loader.py:33-79`).

The reference merges every shard into one dictionary and lets
``load_state_dict(strict=False)`` find what is missing or unexpected
(`pyre/loader.py:46-72`); a wrong shape surfaces as torch's own error. Here the
model's parts name the tensors they need (name and shape), the files' headers are
checked against that list before a byte of data is read, and everything that is
wrong is reported in one error: missing and unexpected tensors, wrong shapes, and
tensors of the wrong class of element type (integers where a weight is expected, or the
reverse). A tied tensor that the file holds beside the one it is tied to
(`lm_head.weight` with `tie_word_embeddings`) is accepted only if the two are equal, and
then shares the other's memory (the reference copies the embedding over a missing head,
`pyre/loader.py:58-61`, and never looks at a present one).

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
    tensors, tensors of the wrong shape or class of element type, and tied tensors
    that differ."""

    def __init__(self, folder, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=(), tied_mismatch=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        self.tied_mismatch = list(tied_mismatch)

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
        if self.wrong_dtype:
            lines.append(f"  wrong element type ({len(self.wrong_dtype)}): " + some(
                f"{n} is {got}, expected {want}" for n, got, want in self.wrong_dtype))
        if self.tied_mismatch:
            lines.append(f"  tied but different ({len(self.tied_mismatch)}): " + some(
                f"{n} differs from {other}" for n, other in self.tied_mismatch))
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


#: safetensors' names of floating-point element types
_FLOAT_CODES = {"F64", "F32", "F16", "BF16"}


def _is_float_code(code: str) -> bool:
    return code.upper() in _FLOAT_CODES


def checkpoint_index(folder: str | Path) -> dict[str, tuple[Path, tuple[int, ...], str]]:
    """name -> (file, shape, element type as safetensors names it), from the files' headers only."""
    index: dict[str, tuple[Path, tuple[int, ...], str]] = {}
    for f in checkpoint_files(folder):
        with safe_open(str(f), framework="pt") as sf:
            for name in sf.keys():
                sl = sf.get_slice(name)
                index[name] = (f, tuple(sl.get_shape()), str(sl.get_dtype()))
    return index


def check_against(specs: list[TensorSpec], index: dict, folder) -> None:
    wanted = {s.name: s for s in specs}
    missing, wrong, wrong_dtype = [], [], []
    for s in specs:
        if s.name not in index:
            if s.alias_of is not None and s.alias_of in index:
                continue  # a tied tensor the file leaves out (pyre/loader.py:58-61)
            missing.append(s.name)
            continue
        if tuple(index[s.name][1]) != tuple(s.shape):
            wrong.append((s.name, index[s.name][1], s.shape))
        code = index[s.name][2]
        if (s.init == "int") == _is_float_code(code):
            wrong_dtype.append((s.name, code, "an integer type" if s.init == "int" else "a floating-point type"))
    unexpected = [n for n in index if n not in wanted]
    if missing or unexpected or wrong or wrong_dtype:
        raise WeightsError(folder, missing, unexpected, wrong, wrong_dtype)


def _settle_tied(out: dict, specs: list[TensorSpec], folder) -> None:
    """A tied tensor that is absent takes the other's memory; one that is present must
    equal it, and then takes its memory too."""
    differ = []
    for s in specs:
        if s.alias_of is None:
            continue
        if s.name in out and not torch.equal(out[s.name], out[s.alias_of]):
            differ.append((s.name, s.alias_of))
        out[s.name] = out[s.alias_of]  # same memory: a tied head costs nothing
    if differ:
        raise WeightsError(folder, tied_mismatch=differ)


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
    _settle_tied(out, specs, folder)
    return out


def adopt_state(state: dict[str, torch.Tensor], specs: list[TensorSpec], device, compute_dtype: torch.dtype) -> dict[str, torch.Tensor]:
    """The same checks and conversions for tensors that are already in memory."""
    index = {n: (None, tuple(t.shape), "F32" if t.dtype.is_floating_point else "I64") for n, t in state.items()}
    check_against(specs, index, "<memory>")
    out = {n: t.to(device=device, dtype=runtime_dtype(t.dtype, compute_dtype)) for n, t in state.items()}
    _settle_tied(out, specs, "<memory>")
    return out
