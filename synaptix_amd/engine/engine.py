"""The engine: a model on the GPU, its cache, and one step function.

`step` runs only the tokens it is given, as one packed batch, from the cache that earlier
steps left, and returns the logits at the wanted places.  Prompts of unequal lengths go in one
step; later steps bring one token for each sequence that is still alive.  Nothing is padded,
so a sequence's results cannot depend on its neighbours beyond the rounding of reductions.

The reference's forward takes [B, S] ids with one shared length
(crates/synaptix-models/llm/common/src/model.rs:1107-1117,1169-1172); unequal lengths, slots and
their reuse are this engine's own.
"""
from __future__ import annotations

import numpy as np
import torch

from ..cache import SequenceCache, CacheError, PAGE_TOKENS, pages_for
from ..config.registry import load_config, resolve_architecture
from ..kernels import ops
from ..weights import FolderSource, RandomSource, load_weights
from .batch import StepLayout, StepContext, ScratchPool, fill_host_buffer

assert ops.PAGE_TOKENS == PAGE_TOKENS

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "f32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


class StepError(ValueError):
    """A step that cannot be run: bad token id, unknown slot, empty entry, ..."""


def parse_dtype(dtype) -> torch.dtype:
    if dtype not in _DTYPES:
        raise ValueError(f"dtype {dtype!r}: expected bfloat16 or float32")
    return _DTYPES[dtype]


class Engine:
    def __init__(self, model, dtype, max_tokens: int, max_slots: int | None = None, max_step_tokens: int | None = None):
        """`model` has its weights loaded on a GPU.  max_step_tokens: see SequenceCache (smaller storage for
        groups of layers that keep a window, if no step brings more tokens than this for one sequence)."""
        self.model = model
        self.dtype = parse_dtype(dtype)
        self.device = model.device
        self._require_gpu()
        self.vocab = model.vocab
        model.check(self.dtype)          # sizes that no kernel takes in this type are refused here
        max_positions = getattr(model.config, "max_position_embeddings", None)
        for b in model.blocks:
            cap = getattr(getattr(b.mixer, "position", None), "capacity", None)
            if cap is not None:
                max_positions = cap if max_positions is None else min(max_positions, cap)
        self.max_positions = max_positions
        self.cache = SequenceCache(model.cache_needs(), max_tokens, max_slots, self.dtype, self.device,
                                   max_positions=max_positions, max_step_tokens=max_step_tokens)
        self._scratch = ScratchPool(self.device)      # of the eager steps; captured steps have their own
        self._host = None
        self._dev = None
        self._runners = {}
        from ..parts.base import StateNeed
        # steps are replayed from graphs only if every part says of itself that it only launches kernels and
        # finds its sequences through arrays on the device (Part.capturable).  A step is run before it is
        # captured; where sequences have running states the runner puts them back after each such run.
        self.has_states = any(isinstance(n, StateNeed) for n in model.cache_needs())
        self.graph_ok = bool(getattr(model, "capturable", lambda: False)())
        self.prompt_graphs = True        # short prompt steps are replayed from graphs (see _prompt_runner)

    # ------------------------------------------------------------------ construction
    @classmethod
    def load(cls, folder: str, dtype="bfloat16", max_tokens: int = 8192, max_slots: int | None = None,
             max_seq: int | None = None, device="cuda:0", strict: bool = True) -> "Engine":
        """A model folder (config.json + safetensors); the model class is chosen by config.json."""
        arch, cfg = load_config(folder)
        model = arch.build(cfg, max_positions=max_seq)
        load_weights(model, FolderSource(folder), parse_dtype(dtype), device, strict=strict)
        return cls(model, dtype, max_tokens, max_slots)

    @classmethod
    def from_config(cls, config, seed: int = 0, dtype="bfloat16", max_tokens: int = 8192,
                    max_slots: int | None = None, max_seq: int | None = None, device="cuda:0") -> "Engine":
        """Random weights drawn on the device (for measurements; no files are written)."""
        arch = resolve_architecture(config.to_dict())
        model = arch.build(config, max_positions=max_seq)
        dt = parse_dtype(dtype)
        src = RandomSource(model.tensor_specs(), seed, store_dtype=dt, device=device)
        load_weights(model, src, dt, device)
        return cls(model, dtype, max_tokens, max_slots)

    # ------------------------------------------------------------------ slots
    def acquire(self) -> int:
        return self.cache.acquire()

    def release(self, slot: int) -> None:
        self.cache.release(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    def snapshot(self, slot: int):
        """A point of the sequence to come back to with `restore` (its length and running states)."""
        return self.cache.snapshot(slot)

    def restore(self, snap) -> None:
        """Back to a snapshot: later steps write the positions behind it again."""
        self.cache.restore(snap)

    # ------------------------------------------------------------------ the step
    def _require_gpu(self):
        if self.device is None or self.device.type != "cuda":
            raise RuntimeError("the engine runs on the GPU only; load the model's weights on a cuda device")

    _RING = 4

    def _buffers(self, total: int):
        """A pinned host buffer whose last copy has left, and the device buffer of the step."""
        if self._host is None or self._host[0].numel() < total:
            n = max(2 * total, 4096)
            self._host = [torch.empty(n, dtype=torch.int32, pin_memory=True) for _ in range(self._RING)]
            self._dev = [torch.empty(n, dtype=torch.int32, device=self.device) for _ in range(self._RING)]
            self._copied = [None] * self._RING
            self._turn = 0
        i = self._turn
        self._turn = (i + 1) % self._RING
        if self._copied[i] is not None:
            self._copied[i].synchronize()
        return i, self._host[i], self._dev[i]

    def _checked(self, entries, want) -> tuple:
        """A step's entries and wanted places, checked: (slots, token arrays, tokens cached before, counts, wanted rows)."""
        if not entries:
            raise StepError("a step needs at least one sequence")
        slots = [e[0] for e in entries]
        token_lists = [np.asarray(e[1], dtype=np.int64).reshape(-1) for e in entries]
        if len(set(slots)) != len(slots):
            raise StepError("a slot appears twice in one step")
        past = []
        for sid, toks in zip(slots, token_lists):
            past.append(self.cache.length(sid))          # raises CacheError for an unknown slot
            if toks.size == 0:
                raise StepError(f"slot {sid}: a step brings at least one token for each of its sequences")
            if toks.min() < 0 or toks.max() >= self.vocab:
                raise StepError(f"slot {sid}: token id outside the vocabulary [0, {self.vocab})")
            if self.max_positions is not None and past[-1] + toks.size > self.max_positions:
                raise CacheError(f"KV overflow: slot {sid} holds {past[-1]} tokens, {toks.size} more exceed "
                                 f"the position range {self.max_positions}")
        starts = np.concatenate([[0], np.cumsum([t.size for t in token_lists])])
        if want is None:
            want_rows = []
        elif isinstance(want, str) and want == "last":
            want_rows = [int(starts[i + 1]) - 1 for i in range(len(entries))]
        elif isinstance(want, str) and want == "all":
            want_rows = list(range(int(starts[-1])))
        else:
            if len(want) != len(entries):
                raise StepError("`want` needs one list of places for each sequence of the step")
            want_rows = []
            for i, places in enumerate(want):
                for p in places:
                    if not (0 <= p < token_lists[i].size):
                        raise StepError(f"slot {slots[i]}: wanted place {p} is outside its {token_lists[i].size} tokens")
                    want_rows.append(int(starts[i]) + int(p))
        counts = [int(t.size) for t in token_lists]
        return slots, token_lists, past, counts, want_rows

    def prepare(self, entries, want) -> tuple:
        """Check a step, hold its pages, and write its arrays to the device.  Returns (ctx, n_want)."""
        slots, token_lists, past, counts, want_rows = self._checked(entries, want)
        self.cache.reserve_step(slots, counts)            # all pages of the step, or none
        return self._context(slots, token_lists, past, counts, want_rows), len(want_rows)

    def _context(self, slots, token_lists, past, counts, want_rows):
        widths = [self.cache.table_width(gi, slots) for gi in range(len(self.cache.groups))]
        layout = StepLayout(sum(counts), len(slots), len(want_rows), widths)
        dev = self._upload(layout, slots, np.concatenate(token_lists), counts, want_rows)
        return StepContext(layout, dev, self.dtype, slots, past, counts, self._scratch)

    def _upload(self, layout, slots, tokens_flat, counts, want_rows) -> torch.Tensor:
        """The step's arrays on the device, through a pinned buffer and one asynchronous copy."""
        i, host, dev = self._buffers(layout.total)
        fill_host_buffer(layout, host.numpy(), self.cache, slots, tokens_flat, counts, want_rows)
        dev[:layout.total].copy_(host[:layout.total], non_blocking=True)
        self._copied[i] = torch.cuda.Event()
        self._copied[i].record()
        return dev

    def step(self, entries, want="last") -> torch.Tensor:
        """entries: [(slot, tokens), ...]; want: "last", "all", None or a list of places for each
        entry.  Returns float logits [wanted, vocab] on the device, in the order of the entries and
        of their places."""
        slots, token_lists, past, counts, want_rows = self._checked(entries, want)
        self.cache.reserve_step(slots, counts)            # all pages of the step, or none
        runner = self._prompt_runner(slots, counts, want_rows)
        if runner is not None:
            logits = runner.step(slots, token_lists, counts, want_rows)
        else:
            ctx = self._context(slots, token_lists, past, counts, want_rows)
            with torch.no_grad():
                logits = self.model.forward(ctx, ctx.tokens, ctx.want if want_rows else None, self.cache)
        for s, n in zip(slots, counts):
            self.cache.commit(s, n)
        if logits is None:
            logits = torch.empty((0, self.vocab), dtype=torch.float32, device=self.device)
        return logits

    def _prompt_runner(self, slots, counts, want_rows):
        """The captured step for a short prompt step with one wanted row a sequence, or None: launched one by
        one, the kernels of a few dozen tokens take the host longer than the GPU."""
        if not (self.prompt_graphs and self.graph_ok and self.dtype == torch.bfloat16) or ops.timing_active():
            return None
        if len(want_rows) != len(slots) or any(c == 1 for c in counts):
            return None         # (single tokens beside prompts go to their own attention kernel, which a captured
                                # prompt step, knowing no counts on the host, cannot arrange)
        starts = np.concatenate([[0], np.cumsum(counts)])
        if any(not (starts[i] <= r < starts[i + 1]) for i, r in enumerate(want_rows)):
            return None
        from .graph import PromptRunner, prompt_bucket
        bucket = prompt_bucket(int(starts[-1]), len(slots))
        if bucket is None or (self.max_positions is not None and self.max_positions < bucket[0]):
            return None
        widths = []
        for gi in range(len(self.cache.groups)):
            width = 1                                  # few distinct widths, so that graphs are shared; the
            while width < max(self.cache.table_width(gi, slots), pages_for(bucket[0])):   # padding tokens fit a row
                width *= 2
            widths.append(width)
        key = ("prompt",) + bucket + tuple(widths)
        if key not in self._runners:
            self._runners[key] = PromptRunner(self, bucket[0], bucket[1], widths)
        return self._runners[key]

    def decode_runner(self, n_seqs: int, max_len: int):
        """The captured decode step for up to n_seqs sequences of at most max_len tokens."""
        from .graph import DecodeRunner, bucket_for
        rows = bucket_for(n_seqs)
        cap = max_len if self.max_positions is None else min(max_len, self.max_positions)
        width = 1
        while width < pages_for(cap):          # few distinct widths, so that graphs are shared
            width *= 2
        key = (rows, width)
        if key not in self._runners:
            self._runners[key] = DecodeRunner(self, rows, [width] * len(self.cache.groups))
        return self._runners[key]

    def sample(self, logits, temperatures=None, uniforms=None) -> torch.Tensor:
        """Token ids (int32, device) for rows of logits; see kernels.ops.sample_rows."""
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        t = u = None
        if temperatures is not None:
            t = torch.as_tensor(temperatures, dtype=torch.float32).to(logits.device)
            u = torch.as_tensor(uniforms, dtype=torch.float32).to(logits.device)
        ops.sample_rows(logits, t, u, out)
        return out
