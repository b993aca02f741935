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

import numpy as np
import torch

from ..kernels import ops


class StepLayout:
    """Offsets of the arrays inside the one int32 buffer, for given counts."""

    def __init__(self, n_tokens: int, n_seqs: int, n_want: int, table_widths: list):
        self.N, self.B, self.n_want, self.widths = n_tokens, n_seqs, n_want, list(table_widths)
        off = 0
        self.off = {}
        for name, n in (("tokens", n_tokens), ("tok_seq", n_tokens), ("tok_pos", n_tokens),
                        ("seq_start", n_seqs + 1), ("seq_past", n_seqs), ("seq_len", n_seqs),
                        ("seq_slot", n_seqs), ("want", n_want)):
            self.off[name] = (off, n)
            off += n
        self.table_off = []
        for w in self.widths:
            self.table_off.append((off, n_seqs * w))
            off += n_seqs * w
        self.total = max(off, 1)


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

    def page_table(self, group: int) -> torch.Tensor:
        return self._tables[group]

    def decode_splits(self, n_kv_heads: int, group: int) -> int:
        return ops.decode_splits(self.n_seqs, n_kv_heads, self.layout.widths[group])

    def scratch(self, name: str, numel: int) -> torch.Tensor:
        """Float scratch memory that lives as long as the engine; contents are undefined."""
        t = self._scratch.get(name)
        if t is None or t.numel() < numel:
            t = torch.empty(max(numel, 1), dtype=torch.float32, device=self.device)
            self._scratch[name] = t
        return t


def fill_host_buffer(layout: StepLayout, host: np.ndarray, token_lists, past, slots, want_rows, tables) -> None:
    """Write every array of the step into `host` (int32, at least layout.total long)."""
    o = layout.off
    pos = 0
    starts = [0]
    for i, toks in enumerate(token_lists):
        n = len(toks)
        host[o["tokens"][0] + pos:o["tokens"][0] + pos + n] = toks
        host[o["tok_seq"][0] + pos:o["tok_seq"][0] + pos + n] = i
        host[o["tok_pos"][0] + pos:o["tok_pos"][0] + pos + n] = np.arange(past[i], past[i] + n, dtype=np.int32)
        pos += n
        starts.append(pos)
    B = layout.B
    host[o["seq_start"][0]:o["seq_start"][0] + B + 1] = starts
    host[o["seq_past"][0]:o["seq_past"][0] + B] = past
    host[o["seq_len"][0]:o["seq_len"][0] + B] = [p + len(t) for p, t in zip(past, token_lists)]
    host[o["seq_slot"][0]:o["seq_slot"][0] + B] = slots
    if layout.n_want:
        host[o["want"][0]:o["want"][0] + layout.n_want] = want_rows
    for (off, n), w, tab in zip(layout.table_off, layout.widths, tables):
        host[off:off + n] = tab.reshape(-1)
