"""A decoder as data: an embedding, a list of blocks, the order in which they run, a final norm
and an output head.

The order is a list of LayerRun(block, cache): it may name a block twice (its weights are then
used twice, each run with a cache of its own), or give two runs the same cache index (the first
run that names a cache writes it, the later ones only read it).  Which mixer, feed-forward and
norm a block has is decided layer by layer by whoever builds the list of blocks.

Forward of one step, as crates/synaptix-models/llm/common/src/model.rs:1052-1105,1160-1262:
embedding (no scale), the runs in order, final norm on the wanted rows only, output product in
float.  The reference norms every row and keeps the last (1068-1074); gathering first is the
same arithmetic on fewer rows.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..kernels import ops
from ..parts.base import Part
from ..parts.linear import Matrix, linear, as_delta, as_rows
from ..weights.source import TensorSpec


@dataclass(frozen=True)
class LayerRun:
    block: int     # index into DecoderModel.blocks
    cache: int     # index of the cache layer it uses


class TokenEmbedding(Part):
    """x[n, :] = E[id[n], :] (crates/synaptix-ops/src/embed/token_embed.rs:4-15)."""
    capturable = True

    def __init__(self, name: str, vocab: int, hidden: int):
        self.name, self.vocab, self.hidden = name, vocab, hidden
        self.table = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.vocab, self.hidden), "table")}

    def load(self, get):
        self.table = Matrix(get(self.name))       # (a tied output head multiplies with the same matrix)

    def forward(self, ids):
        resid = torch.empty((ids.shape[0], self.hidden), dtype=torch.float32, device=ids.device)
        ops.embed(self.table.data, ids, resid)
        return resid


class OutputHead(Part):
    """logits = h . W^T in float; tied: W is the embedding table
    (crates/synaptix-models/llm/common/src/model.rs:757-764)."""
    capturable = True

    def __init__(self, name: str, vocab: int, hidden: int, tied_to: TokenEmbedding | None = None):
        self.name, self.vocab, self.hidden, self.tied_to = name, vocab, hidden, tied_to
        self.weight = None

    def tensor_specs(self):
        return {} if self.tied_to is not None else {self.name: TensorSpec((self.vocab, self.hidden))}

    def ignored_tensors(self):
        # a tied checkpoint may still carry the matrix; it is not read
        return [self.name] if self.tied_to is not None else []

    def load(self, get):
        self.weight = self.tied_to.table if self.tied_to is not None else Matrix(get(self.name))

    def forward(self, h):
        return linear(h, self.weight, torch.float32)


class DecoderModel:
    def __init__(self, config, embedding: TokenEmbedding, blocks: list, schedule: list, final_norm, head: OutputHead):
        self.config = config
        self.embedding, self.blocks, self.schedule = embedding, list(blocks), list(schedule)
        self.final_norm, self.head = final_norm, head
        self.vocab, self.hidden = embedding.vocab, embedding.hidden
        self.act_dtype = None
        self.device = None
        for run in self.schedule:
            if not (0 <= run.block < len(self.blocks)):
                raise ValueError(f"schedule names block {run.block}; there are {len(self.blocks)}")
        # the first run that names a cache owns (writes) it
        seen, self._owner = set(), []
        for run in self.schedule:
            self._owner.append(run.cache not in seen)
            seen.add(run.cache)
        if seen and seen != set(range(len(seen))):
            raise ValueError("cache indices of the schedule must be 0 .. n-1 without gaps")
        self.n_caches = len(seen)

    # ------------------------------------------------------------------ weights
    def _parts(self):
        return [self.embedding] + self.blocks + [self.final_norm, self.head]

    def tensor_specs(self) -> dict:
        specs = {}
        for p in self._parts():
            for n, s in p.tensor_specs().items():
                if n in specs and specs[n] != s:
                    raise ValueError(f"tensor {n} is declared twice with different shapes")
                specs[n] = s
        return specs

    def ignored_tensors(self) -> list:
        return self.head.ignored_tensors()

    def load(self, get) -> None:
        for p in self._parts():
            p.load(get)
        self.device = self.embedding.table.device

    def check(self, dtype) -> None:
        """Every part is asked whether its kernels take its sizes in `dtype`."""
        for p in self._parts():
            p.check(dtype)

    def capturable(self) -> bool:
        """Whether a step of this model may be captured into a graph: every part says so of itself."""
        return all(getattr(p, "capturable", False) for p in self._parts())

    # ------------------------------------------------------------------ cache
    def cache_needs(self) -> list:
        """Need of each cache layer, from the mixer of the run that owns it."""
        needs = [None] * self.n_caches
        for run, owner in zip(self.schedule, self._owner):
            need = self.blocks[run.block].mixer.cache_need()
            if owner:
                needs[run.cache] = need
            elif needs[run.cache] != need:
                raise ValueError(f"block {run.block} reads cache {run.cache} but needs {need}, "
                                 f"its owner keeps {needs[run.cache]}")
        return needs

    # ------------------------------------------------------------------ one step
    def forward(self, ctx, tokens, want_rows, cache) -> torch.Tensor:
        """tokens [N] int32 and want_rows [n] int32 (or None) on the device; returns logits [n, vocab] float."""
        with ops.stream_scope():     # one stream for the whole pass, asked for once
            resid = self.embedding.forward(tokens)
            pending = None
            for run, owner in zip(self.schedule, self._owner):
                block = self.blocks[run.block]
                if not block.takes_deferred_product:
                    pending = as_delta(pending)      # a product that the last block left for a norm to take in
                pending = block.forward(resid, pending, ctx, cache.layer_view(run.cache), owner)
            if want_rows is None:
                return None          # nothing is asked for: the cache has been written, that is all
            if not getattr(self.final_norm, "takes_deferred_product", False):
                pending = as_delta(pending)
            h = self.final_norm.add_apply(resid, pending, ctx.act_dtype, rows=want_rows)
            return self.head.forward(as_rows(h))
