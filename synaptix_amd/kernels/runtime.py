"""The host runtime library (csrc/runtime.cpp) through ctypes: argument types, and its return
codes as exceptions.  It holds the bookkeeping that every step goes through: pages and slots of
the cache, the integer tables of a step, the sampler's random stream."""
from __future__ import annotations

import ctypes as C

from .build import load_library


class CacheFull(RuntimeError):
    """No free page (or slot) is left; nothing was taken."""


class CacheError(RuntimeError):
    """A misuse of the cache: unknown slot, double release, overflow of the position range."""


_P, _I, _L = C.c_void_p, C.c_int, C.c_long
_IP, _LP, _FP, _UP = C.POINTER(C.c_int), C.POINTER(C.c_long), C.POINTER(C.c_float), C.POINTER(C.c_uint32)

_SIGNATURES = {
    "syn_rt_page_tokens": (_I, []),
    "syn_cache_new": (_P, [_I, _LP, _I, _IP, _I, _L]),
    "syn_cache_delete": (None, [_P]),
    "syn_cache_free_slots": (_I, [_P]),
    "syn_cache_free_pages": (_I, [_P, _I]),
    "syn_cache_is_live": (_I, [_P, _I]),
    "syn_cache_acquire": (_I, [_P, _IP]),
    "syn_cache_release": (_I, [_P, _I]),
    "syn_cache_length": (_I, [_P, _I, _LP]),
    "syn_cache_pages_needed": (_I, [_P, _I, _L, _LP]),
    "syn_cache_reserve": (_I, [_P, _I, _L]),
    "syn_cache_reserve_step": (_I, [_P, _I, _IP, _LP]),
    "syn_cache_commit": (_I, [_P, _I, _L]),
    "syn_cache_truncate": (_I, [_P, _I, _L]),
    "syn_cache_table_width": (_I, [_P, _I, _IP, _I, _IP]),
    "syn_cache_page_table": (_I, [_P, _I, _IP, _I, _I, _P]),
    "syn_cache_live_slots": (_I, [_P, _IP]),
    "syn_cache_check": (_I, [_P]),
    "syn_step_layout": (_L, [_L, _L, _L, _I, _IP, _LP]),
    "syn_step_fill": (_I, [_P, _I, _IP, _LP, _P, _L, _P, _I, _IP, _P]),
    "syn_step_fill_padded": (_I, [_P, _I, _IP, _LP, _P, _L, _P, _I, _IP, _IP, _L, _I, _L, _P]),
    "syn_decode_fill": (_I, [_P, _I, _I, _IP, _IP, _I, _IP, _IP, _FP, _FP, _IP, _P]),
    "syn_decode_items": (_I, [_IP, _I, _I, _L, _IP]),
    "syn_philox_block": (None, [_UP, _UP, _UP]),
    "syn_philox_new": (_P, [C.c_uint64]),
    "syn_philox_delete": (None, [_P]),
    "syn_philox_next_u32": (C.c_uint32, [_P]),
    "syn_philox_next_uniform": (C.c_float, [_P]),
    "syn_philox_next_multinomial_uniform": (C.c_float, [_P]),
}

_lib = None


def lib():
    """The loaded library, compiled at its first use."""
    global _lib
    if _lib is None:
        loaded = load_library("runtime")
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(loaded, name)
            fn.restype, fn.argtypes = res, args
        _lib = loaded
    return _lib


def last_error() -> str:
    return lib().syn_rt_last_error().decode(errors="replace")


def check(rc: int) -> None:
    """0, or the exception that the return code stands for."""
    if rc == 0:
        return
    raise (CacheFull if rc == 1 else CacheError)(last_error())


def ints(values):
    """A C array of int from a sequence of Python ints."""
    return (C.c_int * len(values))(*values)


def longs(values):
    return (C.c_long * len(values))(*values)


def decode_items(seq_len, n_splits: int, window=None) -> list:
    """The work list of a decode step's attention as the runtime lays it out and the kernel reads it,
    as a flat list of ints: for sequences of the lengths `seq_len`, len(seq_len) * n_splits items of
    four (sequence, split | splits of the sequence << 16, first, the sequence's length; spare items have
    sequence -1), then (first, splits) of every sequence."""
    rows = len(seq_len)
    out = (C.c_int * (4 * rows * n_splits + 2 * rows))()
    check(lib().syn_decode_items(ints([int(x) for x in seq_len]), rows, int(n_splits),
                                 -1 if window is None else int(window), out))
    return list(out)
