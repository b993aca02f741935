"""Philox-4x32-10 as the reference's sampler uses it: the seed in the key, the counter from
zero, four 32-bit words a block (crates/synaptix-ops/src/rng.rs:16-25,32-36,50-58,82-97).
One stream for each sequence, on the host; the device gets the uniform numbers."""
from __future__ import annotations

import numpy as np

_M0, _M1 = 0xD2511F53, 0xCD9E8D57
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK = 0xFFFFFFFF


def philox4x32_10(counter, key):
    c0, c1, c2, c3 = counter
    k0, k1 = key
    for _ in range(10):
        p0 = _M0 * c0
        p1 = _M1 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & _MASK, p1 & _MASK, ((p0 >> 32) ^ c3 ^ k1) & _MASK, p0 & _MASK
        k0, k1 = (k0 + _W0) & _MASK, (k1 + _W1) & _MASK
    return [c0, c1, c2, c3]


class Philox4x32:
    def __init__(self, seed: int):
        seed = int(seed) & 0xFFFFFFFFFFFFFFFF
        self.key = (seed & _MASK, (seed >> 32) & _MASK)
        self.counter = [0, 0, 0, 0]
        self._buf = []

    def next_u32(self) -> int:
        if not self._buf:
            self._buf = philox4x32_10(self.counter, self.key)
            for i in range(4):
                self.counter[i] = (self.counter[i] + 1) & _MASK
                if self.counter[i]:
                    break
        return self._buf.pop(0)

    def next_f32_uniform(self) -> float:
        """(u32 >> 8) * 2^-24, in [0, 1) (rng.rs:66-69)."""
        return float(np.float32(self.next_u32() >> 8) * np.float32(1.0 / (1 << 24)))

    def next_multinomial_uniform(self) -> float:
        """u = (u32 as f32) / (u32::MAX as f32), as the multinomial sampler draws it
        (crates/synaptix-infer/src/sampling/multinomial.rs:30-32); it can be exactly 1."""
        return float(np.float32(np.float32(float(self.next_u32())) / np.float32(float(0xFFFFFFFF))))
