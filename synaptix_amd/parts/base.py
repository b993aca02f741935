"""What every part of a layer has in common.

A part owns the names, shapes and storage of its tensors and the launches that compute it.
It receives its sizes and constants as parameters and its tensor-name prefix as a string; it
does not know which model it is in (the reference produces tensor names the same way, from
the layer: crates/synaptix-models/llm/common/src/model.rs:780).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


class Part:
    """Base of norms, position encodings, mixers, feed-forwards and blocks."""

    # True: the part's forward only launches kernels on the current stream (no wait for the device, no shape that
    # depends on device data), finds the step's sequences through the context's device arrays alone (a captured
    # step's `ctx.slots`, `ctx.past` and `ctx.new_counts` are placeholders; a running state is reached with
    # StateLayerView.seq_rows / token_rows) and, apart from such a state, writes the same values when it is run
    # again, so that a step that contains it may be captured into a graph and replayed.  False (the default, for
    # parts from elsewhere): the steps of a model that contains it are launched one by one.
    capturable = False

    def tensor_specs(self) -> dict:
        """name -> TensorSpec of every tensor this part reads from the weight source."""
        return {}

    def load(self, get) -> None:
        """Fetch the tensors; `get(name)` returns the tensor on the device in its kept type."""

    def check(self, dtype) -> None:
        """Raise if no kernel takes this part's sizes in the engine's type `dtype`: asked once when an
        engine is made, so that a size is refused before the first step, not in the middle of it."""


@dataclass(frozen=True)
class KvNeed:
    """A mixer that keeps keys and values of the tokens it has seen: all of them, or a window."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None      # None: all keys


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a state of fixed size for each sequence, zero when the sequence starts."""
    shape: tuple
    dtype: torch.dtype = torch.float32
