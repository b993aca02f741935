"""Position encodings as parts.  A mixer is handed one and asks it for what its kernels need.

RotaryHalfSplit: f_i = theta^(-2i/rotary_dim), angle = position * f_i, all in 32-bit; the pair
(d, d + rotary_dim/2) is rotated by the angle of d; dims above rotary_dim pass through.
Tables as crates/synaptix-ops/src/pos/rope_cache.rs:16-38 builds them, rotation as
crates/synaptix-ops/src/pos/rope.rs:81-97 (Split layout).
"""
from __future__ import annotations

import numpy as np
import torch

from .base import Part


class Position(Part):
    def tables(self, device):
        """(cos, sin) float [capacity, rotary_dim / 2] on `device`, or (None, None) for no rotation."""
        return None, None

    def score_slopes(self, n_heads: int, device):
        """A scheme that acts on the attention scores instead of on q and k: float [n_heads] on `device`, the
        score of query position p and key position j <= p then gets - slope[head] * (p - j) (the linear bias of
        crates/synaptix-ops/src/pos/alibi.rs:47-66); None (the default): nothing is added."""
        return None

    capacity = None  # positions at and beyond it cannot be encoded; None: no limit


class NoPosition(Position):
    pass


class RotaryHalfSplit(Position):
    def __init__(self, theta: float, rotary_dim: int, capacity: int):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise ValueError(f"rotary_dim {rotary_dim} must be positive and even")
        if capacity <= 0:
            raise ValueError("capacity must be positive")
        self.theta = float(np.float32(theta))
        self.rotary_dim = rotary_dim
        self.capacity = capacity
        self._tables = {}

    def host_tables(self):
        half = self.rotary_dim // 2
        i = np.arange(half, dtype=np.float32)
        expo = -(np.float32(2.0) * i) / np.float32(self.rotary_dim)
        freqs = np.power(np.float32(self.theta), expo).astype(np.float32)
        t = np.arange(self.capacity, dtype=np.float32)
        ang = (t[:, None] * freqs[None, :]).astype(np.float32)
        return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)

    def tables(self, device):
        key = str(device)
        if key not in self._tables:
            cos, sin = self.host_tables()
            self._tables[key] = (torch.from_numpy(cos).to(device), torch.from_numpy(sin).to(device))
        return self._tables[key]
