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


class ScaledRows:
    """Rows on their way through an RMSNorm whose last step has not been taken: `rows` [M, dim] bf16 hold
    gain * x, `ss` [M, groups] float the sums of x^2 over groups of columns; the normed rows are
    rows[m] * rsqrt(sum(ss[m]) / dim + eps).  A product over packed weights takes them as they are and applies the
    row's factor to its finished sums (it is linear in its input); everything else asks for `plain()`, which norms
    the float rows `resid` they were made from.  Made by a norm from a DeferredProduct; has the shape, type and
    device of the normed rows, so that code which only passes them on need not know."""

    def __init__(self, rows, ss, eps, resid, norm):
        self.rows, self.ss, self.eps, self.resid, self.norm = rows, ss, float(eps), resid, norm
        self.shape, self.dtype, self.device = rows.shape, rows.dtype, rows.device
        self.dim = rows.shape[1]

    @property
    def row_scale(self):
        return (self.ss, self.dim, self.eps)

    def plain(self):
        return self.norm.add_apply(self.resid, None, self.dtype)


def as_rows(h):
    """The normed rows as a tensor, whatever form they arrive in."""
    return h.plain() if isinstance(h, ScaledRows) else h


class DeferredProduct:
    """A product x . W^T over packed weights that has not been run: the norm that receives it as the delta of
    the residual rows runs it with the residual sum and its own first half as the epilogue (ops.gemm_packed,
    resid_norm), or asks for `run()`, the float product itself."""

    def __init__(self, x, w, packed):
        self.x, self.w, self.packed = x, w, packed
        self.shape = (x.shape[0], w.shape[0])

    def run(self):
        return linear_for_sum(self.x, self.w, self.packed)


def as_delta(d):
    """The delta of the residual rows as a tensor (or None), whatever form it arrives in."""
    return d.run() if isinstance(d, DeferredProduct) else d


def deferred_product(x, w, packed=None):
    """linear_for_sum, but where the product would run over packed weights in one slice it is only described:
    the caller's result is the delta that a following norm adds to the residual rows, and that norm can take the
    product in (RmsNorm.add_apply)."""
    if isinstance(x, torch.Tensor) and _use_packed(x, packed) and ops.packed_slices(w.shape[0], w.shape[1]) <= 1:
        return DeferredProduct(x, w, packed)
    return linear_for_sum(x, w, packed)


def linear(x, w, out_dtype, packed=None):
    """x [M, K] in the activation type, w [N, K]; a weight kept in 32-bit takes the 32-bit product.
    packed: packed_copy(w), taken for few rows."""
    if _use_packed(x, packed) and out_dtype in (torch.bfloat16, torch.float32):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=x.device)
        if isinstance(x, ScaledRows):
            ops.gemm_packed(x.rows, packed, out, row_scale=x.row_scale)
        else:
            ops.gemm_packed(x, packed, out)
        return out
    x = as_rows(x)
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
        if isinstance(x, ScaledRows):
            ops.gemm_packed(x.rows, packed, out, row_scale=x.row_scale)
        else:
            ops.gemm_packed(x, packed, out)
        return out
    x = as_rows(x)
    M, K = x.shape
    N = w.shape[0]
    slices = ops.gemm_slices(M, N, K, x.dtype) if w.dtype == x.dtype else 1
    if slices <= 1:
        return linear(x, w, torch.float32)
    out = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    ops.gemm(x, w, out)
    return out

