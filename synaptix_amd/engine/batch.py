"""The sequence table of one step, as the kernels read it.

A step brings, for each of its sequences, a slot and the next tokens.  Tokens of all sequences
lie one after another (no padding); everything that depends on where a sequence begins or
how long it is comes from these small integer arrays, which are written into one host
buffer and copied to the device in one piece:

    tokens   [N]    token ids                 tok_seq  [N]  which sequence of the step a token is in
    tok_pos  [N]    absolute position         seq_start[B+1] offsets of the sequences' tokens
    seq_past [B]    tokens cached before      seq_len  [B]  tokens cached after the step
    seq_slot [B]    slot ids                  want     [n]  rows whose logits are asked for
    page tables     one [B, P_g] for each cache group

The reference has such per-row device arrays only for its graph decode
(crates/synaptix-models/llm/common/src/model.rs:519-553); here every step uses them.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from ..kernels import ops
from ..kernels import runtime as rt

_NAMES = ("tokens", "tok_seq", "tok_pos", "seq_start", "seq_past", "seq_len", "seq_slot", "want")


class StepLayout:
    """Offsets of the arrays inside the one int32 buffer, for given counts (the native runtime
    lays the buffer out and fills it; this is its map)."""

    def __init__(self, n_tokens: int, n_seqs: int, n_want: int, table_widths: list):
        self.N, self.B, self.n_want, self.widths = n_tokens, n_seqs, n_want, [int(w) for w in table_widths]
        offsets = (C.c_long * (len(_NAMES) + len(self.widths)))()
        self.total = rt.lib().syn_step_layout(n_tokens, n_seqs, n_want, len(self.widths), rt.ints(self.widths), offsets)
        counts = (n_tokens, n_tokens, n_tokens, n_seqs + 1, n_seqs, n_seqs, n_seqs, n_want)
        self.off = {name: (offsets[i], n) for i, (name, n) in enumerate(zip(_NAMES, counts))}
        self.table_off = [(offsets[len(_NAMES) + g], n_seqs * w) for g, w in enumerate(self.widths)]


class ScratchPool:
    """Named float scratch tensors that grow on demand.  A tensor that grows is replaced and the old
    one goes back to the allocator, so a pool belongs to one user: the engine's eager steps share
    one, every captured decode step has its own and freezes it before the capture (a graph holds
    the addresses it was captured with; growth after that would be a use of freed memory)."""

    def __init__(self, device):
        self.device, self.tensors, self.frozen = device, {}, False

    def get(self, name: str, numel: int) -> torch.Tensor:
        t = self.tensors.get(name)
        if t is None or t.numel() < numel:
            if self.frozen:
                raise RuntimeError(f"scratch {name!r} of a captured step would have to grow to {numel} floats")
            t = torch.empty(max(numel, 1), dtype=torch.float32, device=self.device)
            self.tensors[name] = t
        return t

    def counters(self, name: str, numel: int) -> torch.Tensor:
        """int32 counters that are zero when handed out first; their users leave them zero."""
        t = self.tensors.get(name)
        if t is None or t.numel() < numel:
            if self.frozen:
                raise RuntimeError(f"counters {name!r} of a captured step would have to grow to {numel}")
            t = torch.zeros(max(numel, 1), dtype=torch.int32, device=self.device)
            self.tensors[name] = t
        return t


class StepContext:
    """What parts see of a step.  Device arrays are views into one buffer."""

    def __init__(self, layout: StepLayout, buffer: torch.Tensor, act_dtype, slots, past, new_counts, scratch_pool):
        self.layout, self.buffer = layout, buffer
        self.act_dtype, self.device = act_dtype, buffer.device
        self.n_tokens, self.n_seqs = layout.N, layout.B
        self.slots, self.past, self.new_counts = list(slots), list(past), list(new_counts)
        self.one_token_each = all(n == 1 for n in new_counts)
        self.max_position = max(p + n for p, n in zip(past, new_counts)) - 1
        self._scratch = scratch_pool
        for name, (o, n) in layout.off.items():
            setattr(self, name, buffer[o:o + n])
        self._tables = [buffer[o:o + n].view(layout.B, w) for (o, n), w in zip(layout.table_off, layout.widths)]
        self.items = None       # a work list of decode attention for each group, where the step's owner keeps them

    def page_table(self, group: int) -> torch.Tensor:
        return self._tables[group]

    def decode_splits(self, n_kv_heads: int, group: int) -> int:
        return ops.decode_splits(self.n_seqs, n_kv_heads, self.layout.widths[group])

    def decode_items(self, group: int):
        """The group's work list for decode attention (int32 [n_seqs * decode_splits, 4]) or None."""
        return None if self.items is None else self.items[group]

    def single_token_rows(self):
        """In a step that brings whole prompts for some sequences and one token for others: (the token rows, the
        sequence indices) of those with one token, as int64 tensors on the device; None in every other step.  A
        mixer may hand these sequences to its kernel for single tokens (one workgroup a tile of query rows would
        walk a long sequence's keys alone)."""
        if not hasattr(self, "_singles"):
            self._singles = None
            seqs = [i for i, n in enumerate(self.new_counts) if n == 1]
            if seqs and len(seqs) < len(self.new_counts):
                starts = np.concatenate([[0], np.cumsum(self.new_counts)])
                self._singles = (torch.tensor([int(starts[i]) for i in seqs], dtype=torch.long, device=self.device),
                                 torch.tensor(seqs, dtype=torch.long, device=self.device))
        return self._singles

    def scratch(self, name: str, numel: int) -> torch.Tensor:
        """Float scratch memory that lives as long as its pool's owner; contents are undefined."""
        return self._scratch.get(name, numel)

    def counters(self, name: str, numel: int) -> torch.Tensor:
        """Zeroed int32 counters that live as long as the pool's owner; whoever counts with them leaves them zero."""
        return self._scratch.counters(name, numel)


def fill_host_buffer(layout: StepLayout, host: np.ndarray, cache, slots, tokens_flat: np.ndarray, counts,
                     want_rows) -> None:
    """Write every array of the step into `host` (int32, at least layout.total long): positions
    and page tables come from the cache's own state."""
    if host.size < layout.total or host.dtype != np.int32:
        raise ValueError("the step's host buffer is too small")
    tokens_flat = np.ascontiguousarray(tokens_flat, dtype=np.int32)
    want = np.ascontiguousarray(want_rows, dtype=np.int32)
    rt.check(rt.lib().syn_step_fill(cache._h, len(slots), rt.ints([int(s) for s in slots]),
                                    rt.longs([int(c) for c in counts]), tokens_flat.ctypes.data, want.size,
                                    want.ctypes.data, len(layout.widths), rt.ints(layout.widths), host.ctypes.data))
