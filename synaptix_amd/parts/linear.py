"""A weight matrix [out, in] without bias: y = x . W^T, 32-bit accumulation.

crates/synaptix-nn/src/linear.rs:67-73; the decoder builds every projection without a bias
(crates/synaptix-models/llm/common/src/weights.rs:49).
"""
from __future__ import annotations

import torch

from ..kernels import ops


def linear(x, w, out_dtype):
    """x [M, K] in the activation type, w [N, K]; a weight kept in 32-bit takes the 32-bit product."""
    if w.dtype != x.dtype:
        if w.dtype == torch.float32:
            x = x.to(torch.float32)
        else:
            raise TypeError(f"linear: activation {x.dtype} with weight {w.dtype}")
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32 if x.dtype == torch.float32 else out_dtype,
                      device=x.device)
    ops.gemm(x, w, out)
    return out if out.dtype == out_dtype else out.to(out_dtype)


def linear_for_sum(x, w):
    """The product as float partial sums for a consumer that adds them up (the residual sum fused
    into the next norm): [S, M, N] when cutting K into S slices gives a small product more
    workgroups, else [M, N]."""
    M, K = x.shape
    N = w.shape[0]
    slices = ops.gemm_slices(M, N, K, x.dtype) if w.dtype == x.dtype else 1
    if slices <= 1:
        return linear(x, w, torch.float32)
    out = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    ops.gemm(x, w, out)
    return out

