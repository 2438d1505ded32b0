"""Position encodings for attention mixers.

Rotary, as the reference builds it (ullm/layers/rotary_embedding.py:52-75): inv_freq_i =
1 / base^(2i/d) for i < d/2, angle[p, i] = p * inv_freq_i, cos and sin in 32-bit, one table row per
position.  The table stays 32-bit (the reference casts cos/sin to the activation dtype before the
multiply, rotary_embedding.py:16-17; here the rotation itself is 32-bit).  Pairing "half" rotates
(x[i], x[i + d/2]) as the reference's chunk(2) does (rotary_embedding.py:19-22); the reference then
interleaves the two output halves (rotary_embedding.py:24), a fixed permutation applied to q and k
alike that leaves every q.k unchanged, so outputs are kept in place here.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import PartEnv, PositionEncoding, register_part


@register_part("position", "none")
class NoPosition(PositionEncoding):
    def kernel_args(self):
        return None, 0, 0


@register_part("position", "rotary")
class Rotary(PositionEncoding):
    """``rotary_dim`` leading dims of each head are rotated; ``pairing`` is "half" or "adjacent"."""

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None,
                 pairing: str = "half", max_positions: Optional[int] = None):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= head_dim):
            raise ValueError(f"rotary_dim={self.rotary_dim} must be even and at most head_dim={head_dim}")
        if pairing not in ("half", "adjacent"):
            raise ValueError(f"unknown rotary pairing {pairing!r}")
        self.style = 1 if pairing == "half" else 2
        self.max_positions = max_positions
        self.table: Optional[torch.Tensor] = None

    @staticmethod
    def make_table(rotary_dim: int, theta: float, rows: int) -> torch.Tensor:
        inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
        angles = torch.arange(rows, dtype=torch.float32)[:, None] * inv_freq[None, :]
        return torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous()

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        rows = env.context_len if self.max_positions is None else min(env.context_len, self.max_positions)
        # every layer with the same rotation shares one table: built once, read by all their kernels
        self.table = env.shared(("rotary", self.rotary_dim, self.theta, rows),
                                lambda: self.make_table(self.rotary_dim, self.theta, rows).to(env.device))

    def kernel_args(self):
        return self.table, self.rotary_dim, self.style
