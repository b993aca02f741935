"""Decode steps replayed from a HIP graph.

A decode step is some hundreds of small launches; launched one by one from the host they cost
more than the step's work at small batch sizes.  The step for a fixed number of rows is
therefore captured once and replayed; what changes from step to step (tokens, positions,
lengths, page tables, temperatures, uniform numbers) lies in one device buffer that is
refreshed by one copy before each replay.  The reference does the same for its single sequence
(crates/synaptix-models/llm/qwen3/src/pipeline.rs:192-316, crates/synaptix-infer/src/graph_capture/capture.rs:24-122).

Rows beyond the live sequences are padding: they run token 0 at position 0 against a spare
cache page that no sequence owns, and their results are dropped.  No row reads another row's
data, so padding changes no result.

Short prompt steps are replayed likewise (PromptRunner): launched one by one, the some hundred
kernels of a prompt of a few dozen tokens cost the host more time than they cost the GPU.

Captured are this package's kernels and torch's allocations only; no memset nodes.
"""
from __future__ import annotations

import ctypes as C
import gc

import numpy as np
import torch

from ..kernels import ops
from ..kernels import runtime as rt
from .batch import StepLayout, StepContext, ScratchPool


def bucket_for(n: int) -> int:
    """Row counts for which graphs are captured: powers of two up to 64, then multiples of 32."""
    if n <= 64:
        b = 1
        while b < n:
            b *= 2
        return b
    return (n + 31) // 32 * 32


def _captured(forward, scratch, rewind=None):
    """Run `forward` twice on a side stream, freeze its scratch pool, then capture it; returns (graph, what
    forward returned).  Keys and values are written to the same places with the same values every time; what a
    run changes for good (running states) `rewind` puts back after each of the two runs, so that the first
    replay finds the sequences where the step found them."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        for _ in range(2):
            forward()
            if rewind is not None:
                rewind()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    scratch.frozen = True
    graph = torch.cuda.CUDAGraph()
    # No garbage collection while the stream is being captured: a dead object's finalizer may free
    # device or pinned memory or destroy another graph (an engine and its runners form a cycle, so
    # they die in the collector), which the runtime refuses during a capture and torch answers by
    # ending the process.  Collect what is dead now, then hold the collector off until the capture ends.
    gc.collect()
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        with torch.no_grad(), torch.cuda.graph(graph):
            out = forward()
    finally:
        if was_enabled:
            gc.enable()
    return graph, out


def _state_rewind(engine, slots):
    """What puts the running states of these slots back to where they are now, or None if there are none."""
    if not engine.has_states:
        return None
    saved = engine.cache.states_of(slots)
    return lambda: engine.cache.put_states(saved)


class DecodeRunner:
    def __init__(self, engine, rows: int, widths: list):
        self.engine, self.rows, self.widths = engine, rows, list(widths)
        self.layout = StepLayout(rows, rows, rows, widths)
        n_int = self.layout.total
        # the work lists of decode attention, one for each group of layers whose keys are split: longer sequences
        # get more of the group's rows * splits workgroups (per kv head), refreshed with the step's other tables
        groups = engine.cache.groups
        self.item_splits = [ops.decode_splits(rows, g.need.kv_heads, w) if engine.dtype == torch.bfloat16 else 0
                            for g, w in zip(groups, self.widths)]
        self.item_splits = [s if s > 1 else 0 for s in self.item_splits]
        n_items = [4 * rows * s + 2 * rows if s else 0 for s in self.item_splits]       # ints of each list
        self.total = n_int + 2 * rows + sum(n_items)           # + temperatures and uniforms as float bits + work lists
        dev = engine.device
        self.dev = torch.zeros(self.total, dtype=torch.int32, device=dev)
        self.host = [torch.zeros(self.total, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.copied = [None, None]
        self.turn = 0
        self.temps = self.dev[n_int:n_int + rows].view(torch.float32)
        self.uniforms = self.dev[n_int + rows:n_int + 2 * rows].view(torch.float32)
        self.items, at = [], n_int + 2 * rows
        for n in n_items:
            self.items.append(self.dev[at:at + n] if n else None)
            at += n
        self.out_tokens = torch.zeros(rows, dtype=torch.int32, device=dev)
        self.logits = None
        self.graph = None
        self.spare = [g.spare_page for g in engine.cache.groups]
        # scratch memory of this runner's own: the captured graph holds its addresses, so no later
        # step or larger runner may ever replace these tensors (row count, table widths and with them
        # the number of splits are fixed here, so the first pass sizes them for good)
        self.scratch = ScratchPool(dev)

    def _fill(self, host: np.ndarray, slots, tokens, temps, uniforms):
        """The padded tables of the step and, behind them, temperatures and uniform numbers."""
        B = len(slots)
        t = u = None
        if temps is not None:
            t = (C.c_float * B)(*[float(x) for x in temps])
            u = (C.c_float * B)(*[float(x) for x in uniforms])
        rt.check(rt.lib().syn_decode_fill(self.engine.cache._h, self.rows, B, rt.ints([int(s) for s in slots]),
                                          rt.ints([int(x) for x in tokens]), len(self.widths), rt.ints(self.widths),
                                          rt.ints(self.spare), t, u, rt.ints(self.item_splits), host.ctypes.data))

    def _forward(self, ctx):
        eng = self.engine
        logits = eng.model.forward(ctx, ctx.tokens, ctx.want, eng.cache)
        ops.sample_rows(logits, self.temps, self.uniforms, self.out_tokens)
        return logits

    def step(self, slots, tokens, temps=None, uniforms=None):
        """One token for each of `slots`; returns (sampled tokens as a host list, logits [B, V]).
        temps None: greedy for every row."""
        eng, B = self.engine, len(slots)
        if ops.timing_active():
            raise ops.KernelError("op_timing: per-op times need eager steps; a captured decode step cannot be timed op by op")
        if B > self.rows:
            raise ValueError(f"{B} sequences for a graph of {self.rows} rows")
        eng.cache.reserve_step(slots, [1] * B)        # all pages of the step, or none
        i = self.turn
        self.turn ^= 1
        if self.copied[i] is not None:
            self.copied[i].synchronize()
        self._fill(self.host[i].numpy(), slots, tokens, temps, uniforms)
        self.dev.copy_(self.host[i], non_blocking=True)
        self.copied[i] = torch.cuda.Event()
        self.copied[i].record()
        if self.graph is None:
            ctx = StepContext(self.layout, self.dev, eng.dtype, [-1] * self.rows, [0] * self.rows, [1] * self.rows,
                              self.scratch)
            ctx.max_position = eng.max_positions - 1 if eng.max_positions else 0   # checked on the host each step
            ctx.items = self.items
            self.graph, self.logits = _captured(lambda: self._forward(ctx), self.scratch, _state_rewind(eng, slots))
        self.graph.replay()
        out = self.out_tokens[:B].cpu().tolist()      # waits for the step
        for s in slots:
            eng.cache.commit(s, 1)
        return out, self.logits[:B]


# ----------------------------------------------------------------------------- short prompts
PROMPT_ROWS = (16, 32, 64, 128)        # token counts for which prompt steps are captured (beyond them the GPU takes
                                       # as long as the host: 256 rows replayed 7.1 ms, launched one by one 7.3 ms)
PROMPT_SEQS = (1, 2, 4, 8)             # sequences of the step (one more, for the padding tokens, is added)


def prompt_bucket(n_tokens: int, n_seqs: int):
    """(rows, sequences) of the captured step that takes a prompt step of this size, or None."""
    rows = next((r for r in PROMPT_ROWS if n_tokens <= r), None)
    seqs = next((b for b in PROMPT_SEQS if n_seqs <= b), None)
    return None if rows is None or seqs is None else (rows, seqs + 1)


class PromptRunner:
    """A prompt step of up to `rows` tokens in up to `seqs - 1` sequences, each with one wanted row,
    replayed from a graph.  The step's own tokens come first; the rows behind them are padding: token 0
    at positions 0, 1, ... of one more sequence that owns no slot and whose page table names only the
    spare page (and whose running state, where there is one, is the spare row)."""

    def __init__(self, engine, rows: int, seqs: int, widths: list):
        self.engine, self.rows, self.seqs, self.widths = engine, rows, seqs, list(widths)
        self.layout = StepLayout(rows, seqs, seqs, self.widths)
        dev = engine.device
        self.dev = torch.zeros(self.layout.total, dtype=torch.int32, device=dev)
        self.host = [torch.zeros(self.layout.total, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.copied = [None, None]
        self.turn = 0
        self.spare = [g.spare_page for g in engine.cache.groups]
        self.scratch = ScratchPool(dev)         # of this runner alone: the graph holds its addresses
        self.graph = self.logits = None

    def step(self, slots, token_lists, counts, want_rows) -> torch.Tensor:
        """Logits [len(want_rows), vocab] of the step; the caller has checked it and holds its pages."""
        eng = self.engine
        i = self.turn
        self.turn ^= 1
        if self.copied[i] is not None:
            self.copied[i].synchronize()
        tokens = np.ascontiguousarray(np.concatenate(token_lists), dtype=np.int32)
        want = np.ascontiguousarray(want_rows, dtype=np.int32)
        rt.check(rt.lib().syn_step_fill_padded(
            eng.cache._h, len(slots), rt.ints([int(s) for s in slots]), rt.longs([int(c) for c in counts]),
            tokens.ctypes.data, want.size, want.ctypes.data, len(self.widths), rt.ints(self.widths), rt.ints(self.spare),
            self.rows, self.seqs, self.seqs, self.host[i].numpy().ctypes.data))
        self.dev.copy_(self.host[i], non_blocking=True)
        self.copied[i] = torch.cuda.Event()
        self.copied[i].record()
        if self.graph is None:
            ctx = StepContext(self.layout, self.dev, eng.dtype, [-1] * self.seqs, [0] * self.seqs,
                              [self.rows] + [0] * (self.seqs - 1), self.scratch)
            ctx.max_position = eng.max_positions - 1 if eng.max_positions else 0   # checked on the host each step
            self.graph, self.logits = _captured(lambda: eng.model.forward(ctx, ctx.tokens, ctx.want, eng.cache),
                                                self.scratch, _state_rewind(eng, slots))
        self.graph.replay()
        return self.logits[:len(want_rows)].clone()     # the next replay writes the same rows again
