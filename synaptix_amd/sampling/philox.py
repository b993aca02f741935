"""Philox-4x32-10 as the reference's sampler uses it: the seed in the key, the counter from
zero, four 32-bit words a block (crates/synaptix-ops/src/rng.rs:16-25,32-36,50-58,82-97).
One stream for each sequence, on the host (kept by the native runtime); the device gets the
uniform numbers."""
from __future__ import annotations

import ctypes as C

from ..kernels import runtime as rt


def philox4x32_10(counter, key):
    """One block: four 32-bit words from a 128-bit counter and a 64-bit key."""
    c = (C.c_uint32 * 4)(*[int(x) & 0xFFFFFFFF for x in counter])
    k = (C.c_uint32 * 2)(*[int(x) & 0xFFFFFFFF for x in key])
    out = (C.c_uint32 * 4)()
    rt.lib().syn_philox_block(c, k, out)
    return list(out)


class Philox4x32:
    def __init__(self, seed: int):
        self._h = rt.lib().syn_philox_new(int(seed) & 0xFFFFFFFFFFFFFFFF)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                rt.lib().syn_philox_delete(h)
            except Exception:       # the interpreter is shutting down; the process's memory goes with it
                pass

    def next_u32(self) -> int:
        return rt.lib().syn_philox_next_u32(self._h)

    def next_f32_uniform(self) -> float:
        """(u32 >> 8) * 2^-24, in [0, 1) (rng.rs:66-69)."""
        return rt.lib().syn_philox_next_uniform(self._h)

    def next_multinomial_uniform(self) -> float:
        """u = (u32 as f32) / (u32::MAX as f32), as the multinomial sampler draws it
        (crates/synaptix-infer/src/sampling/multinomial.rs:30-32); it can be exactly 1."""
        return rt.lib().syn_philox_next_multinomial_uniform(self._h)
