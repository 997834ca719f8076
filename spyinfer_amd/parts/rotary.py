"""Rotary position encoding, half-split pairing.

Tables as the reference builds them (src/utils/constant_table.hpp:28-41):
``freq_j = theta^(-j / (rot/2))`` and ``cos/sin(p * freq_j)`` with ``p * freq_j``
formed in float32.  Pair (j, j + rot/2) of each head vector is rotated
(src/backends/cpu/cpu_operator.cpp:401-407).  ``rotary_dim`` < head_dim leaves
the remaining dims as they are (the reference always rotates the whole head).
"""
from __future__ import annotations

import torch

from .base import PositionEncoding


class RotaryEmbedding(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, rotary_dim: int = None):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= head_dim):
            raise ValueError("rotary_dim must be even and at most head_dim")
        self.cos = self.sin = None

    def prepare(self, device, max_positions: int) -> None:
        half = self.rotary_dim // 2
        # the exponent and the angle are formed in float32, as in the reference; the table is built
        # on the host once and then lies on the device
        j = torch.arange(half, dtype=torch.float32)
        freq = torch.pow(torch.tensor(self.theta, dtype=torch.float32), -j / float(half))
        p = torch.arange(max_positions, dtype=torch.float32)
        ang = p[:, None] * freq[None, :]
        self.cos = torch.cos(ang).contiguous().to(device)
        self.sin = torch.sin(ang).contiguous().to(device)

    def capturable(self, batch):
        return True

    def rotary(self):
        return self.cos, self.sin, self.rotary_dim
