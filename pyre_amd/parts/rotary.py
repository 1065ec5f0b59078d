"""Rotary positions as tables of cos and sin by absolute position.

The table is the reference's (`pyre/model.py:41-51`): inv_freq[j] = 1 / theta^(2j/d)
in float32, angle = position * inv_freq[j], cos and sin of it, kept in float32 (the
reference then rounds the table to the model's element type; here the rotation is
done in float32 and only its result is rounded). The halves of the reference's
table repeat each other, so one half is stored.
"""

from __future__ import annotations

import torch

from pyre_amd.parts.base import NoPositionSpec, PositionEncoding, RotarySpec


def rotary_tables(rotary_dim: int, theta: float, n_positions: int) -> tuple[torch.Tensor, torch.Tensor]:
    """cos, sin of shape [n_positions, rotary_dim / 2], float32, on the CPU."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    t = torch.arange(n_positions, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return freqs.cos(), freqs.sin()


class RotaryEncoding(PositionEncoding):
    def __init__(self, spec: RotarySpec):
        self.spec = spec
        self.rotary_dim = spec.rotary_dim if spec.rotary_dim is not None else spec.head_dim
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= spec.head_dim):
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {spec.head_dim}")
        self._tables = None

    def rotary(self, runtime):
        n = runtime.max_positions  # the engine's longest request decides, as the reference's table grows on demand
        if self._tables is None or self._tables[0].shape[0] < n or self._tables[0].device != runtime.device:
            cos, sin = rotary_tables(self.rotary_dim, self.spec.theta, n)
            self._tables = (cos.to(runtime.device).contiguous(), sin.to(runtime.device).contiguous())
        return self._tables[0], self._tables[1], self.rotary_dim


class NoPosition(PositionEncoding):
    def __init__(self, spec: NoPositionSpec):
        self.spec = spec
