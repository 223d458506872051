"""Position encodings.

Rotary, half-split pairing as in the reference (/root/reference/src/ops.cpp:154-179
for the frequency table, :392-458 for the rotation): for i in [0, d/2):
inv_freq_i = 1 / theta^(2i/d) (float32), angle = float(position) * inv_freq_i,
(x_i, x_{i+d/2}) <- (x_i cos - x_{i+d/2} sin, x_i sin + x_{i+d/2} cos); applied to
queries and keys, never to values.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import PositionEncoding, register_part


class RotaryHalfSplit(PositionEncoding):
    """Rotation of the first `rotary_dim` features of each head (all of them by default)."""

    graph_safe = True

    def __init__(self, prefix: str, head_dim: int, theta: float, rotary_dim: int | None = None, **_):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and in (0, head_dim={self.head_dim}]")
        if not self.theta > 0:
            raise ValueError("rope theta must be positive")
        self._inv_freq: dict = {}

    def inv_freq_host(self) -> torch.Tensor:
        d = self.rotary_dim
        i = torch.arange(0, d // 2, dtype=torch.float32)
        # float32 pow of a float32 base, then a float32 reciprocal, as in ops.cpp:172-175
        freq = torch.pow(torch.tensor(self.theta, dtype=torch.float32), (2.0 * i) / float(d))
        return (1.0 / freq).to(torch.float32)

    def rotary(self, device):
        key = str(device)
        if key not in self._inv_freq:
            self._inv_freq[key] = self.inv_freq_host().to(device)
        return self._inv_freq[key], self.rotary_dim

    def table(self, ctx):
        """The step's cosines and sines [T, rotary_dim / 2, 2], computed by the first layer that asks and
        shared by the others (the angles depend on the positions only); None if the backend has no such kernel."""
        key = ("rope_table", self.theta, self.rotary_dim)
        if key not in ctx.shared:
            inv_freq, _ = self.rotary(ctx.positions.device)
            ctx.shared[key] = kernels.backend().rope_table(ctx.positions, inv_freq)
        return ctx.shared[key]


class NoPosition(PositionEncoding):
    """No position information enters the mixer."""

    graph_safe = True

    def __init__(self, prefix: str = "", **_):
        pass

    def rotary(self, device):
        return None

    def apply(self, q, k, positions):
        return None


register_part("position_encoding", "rope_half_split", RotaryHalfSplit)
register_part("position_encoding", "none", NoPosition)
