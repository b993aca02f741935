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


def gated_linear_for_sum(gate_up, w):
    """(silu(g) * u) . W^T for rows [g | u] of gate_up, as linear_for_sum gives it, with the
    activation inside the product where the product is cut along K and has at most 16 rows (every
    workgroup of the product computes the activation of its k range again, which costs more than
    the activation's own kernel saves once there are more rows: measured at 64); None where it
    is not, and the caller applies the activation on its own."""
    M, K = gate_up.shape[0], gate_up.shape[1] // 2
    N = w.shape[0]
    if w.dtype != gate_up.dtype or M > 16 or ops.gemm_slices(M, N, K, gate_up.dtype) <= 1:
        return None
    out = torch.empty((ops.gemm_slices(M, N, K, gate_up.dtype), M, N), dtype=torch.float32, device=gate_up.device)
    ops.gemm_gated(gate_up, w, out)
    return out
