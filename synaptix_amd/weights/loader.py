"""Check a source against what a model expects, then hand tensors to its parts.

The reference reports a missing name when a layer asks for it and does not check
shapes at load (crates/synaptix-models/llm/qwen3/src/loader.rs:49-53,71-73).  Here every name
and shape is checked before anything is uploaded, and all faults are listed in one error.

Kept types: a tensor stored in 32 bits stays 32-bit, other float types become
bfloat16, integer tables become int32.  In the 32-bit mode every float tensor is
widened to float32.
"""
from __future__ import annotations

import torch

from .source import WeightSource


class WeightError(ValueError):
    """Lists every missing tensor, unexpected tensor and wrong shape at once."""

    def __init__(self, missing, unexpected, wrong_shape, where=""):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        lines = [f"weights do not fit the model{' (' + where + ')' if where else ''}:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n}: file {list(got)}, model {list(want)}" for n, got, want in self.wrong_shape))
        super().__init__("\n".join(lines))


_FLOAT_NAMES = {"F64", "F32", "F16", "BF16"}
_INT_NAMES = {"I64", "I32", "I16", "I8", "U8", "BOOL"}


def kept_dtype(stored: str, engine_dtype: torch.dtype) -> torch.dtype:
    if stored in _INT_NAMES:
        return torch.int32
    if stored not in _FLOAT_NAMES:
        raise ValueError(f"unsupported dtype {stored}")
    if engine_dtype == torch.float32:
        return torch.float32
    return torch.float32 if stored in ("F32", "F64") else torch.bfloat16


def check_source(specs: dict, source: WeightSource, ignored=(), where="") -> None:
    names = set(source.names())
    missing = [n for n in specs if n not in names]
    unexpected = sorted(n for n in names if n not in specs and n not in set(ignored))
    wrong = []
    for n, spec in specs.items():
        if n in names:
            _, shape = source.info(n)
            if tuple(shape) != tuple(spec.shape):
                wrong.append((n, tuple(shape), tuple(spec.shape)))
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong, where)


def load_weights(model, source: WeightSource, engine_dtype: torch.dtype, device, strict: bool = True) -> None:
    """Verify, then let every part of `model` fetch its tensors on `device`."""
    specs = model.tensor_specs()
    try:
        check_source(specs, source, ignored=model.ignored_tensors(), where=getattr(source, "folder", ""))
    except WeightError as e:
        if strict or e.missing or e.wrong_shape:
            raise
    device = torch.device(device)

    def get(name: str) -> torch.Tensor:
        stored, _ = source.info(name)
        t = source.tensor(name)
        return t.to(device=device, dtype=kept_dtype(stored, engine_dtype)).contiguous()

    model.load(get)
