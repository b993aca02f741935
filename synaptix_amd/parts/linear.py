"""A weight matrix [out, in] without bias: y = x . W^T, 32-bit accumulation.

crates/synaptix-nn/src/linear.rs:67-73; the decoder builds every projection without a bias
(crates/synaptix-models/llm/common/src/weights.rs:49).
"""
from __future__ import annotations

import torch

from ..kernels import ops


_KEEP_PACKED_COPIES = True


def keep_packed_copies(flag: bool) -> None:
    """Whether models loaded from now on keep the second copy of their bf16 weights (packed_copy).
    Without it single tokens read the plain matrices through the slower kernels."""
    global _KEEP_PACKED_COPIES
    _KEEP_PACKED_COPIES = bool(flag)


def packed_copy(w):
    """What a part keeps beside a bf16 weight for single tokens: the same matrix in the order of the MFMA
    fragments (ops.pack_weight), or None.  It doubles the memory of the weight; a step of up to
    ops.PACKED_MAX_ROWS rows reads it instead of w."""
    return ops.pack_weight(w) if _KEEP_PACKED_COPIES and w.dtype == torch.bfloat16 else None


def _use_packed(x, packed):
    return packed is not None and x.dtype == torch.bfloat16 and x.shape[0] <= ops.PACKED_MAX_ROWS


def linear(x, w, out_dtype, packed=None):
    """x [M, K] in the activation type, w [N, K]; a weight kept in 32-bit takes the 32-bit product.
    packed: packed_copy(w), taken for few rows."""
    if _use_packed(x, packed) and out_dtype in (torch.bfloat16, torch.float32):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=x.device)
        ops.gemm_packed(x, packed, out)
        return out
    if w.dtype != x.dtype:
        if w.dtype == torch.float32:
            x = x.to(torch.float32)
        else:
            raise TypeError(f"linear: activation {x.dtype} with weight {w.dtype}")
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32 if x.dtype == torch.float32 else out_dtype,
                      device=x.device)
    ops.gemm(x, w, out)
    return out if out.dtype == out_dtype else out.to(out_dtype)


def linear_for_sum(x, w, packed=None):
    """The product as float partial sums for a consumer that adds them up (the residual sum fused
    into the next norm): [S, M, N] when cutting K into S slices gives a small product more
    workgroups, else [M, N]."""
    if _use_packed(x, packed):
        slices = ops.packed_slices(w.shape[0], w.shape[1])
        if slices <= 1:
            return linear(x, w, torch.float32, packed)
        out = torch.empty((slices, x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device)
        ops.gemm_packed(x, packed, out)
        return out
    M, K = x.shape
    N = w.shape[0]
    slices = ops.gemm_slices(M, N, K, x.dtype) if w.dtype == x.dtype else 1
    if slices <= 1:
        return linear(x, w, torch.float32)
    out = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    ops.gemm(x, w, out)
    return out

