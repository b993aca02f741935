"""A weight matrix [out, in] without bias: y = x . W^T, 32-bit accumulation.

crates/synaptix-nn/src/linear.rs:67-73; the decoder builds every projection without a bias
(crates/synaptix-models/llm/common/src/weights.rs:49).
"""
from __future__ import annotations

import torch

from ..kernels import ops


class Matrix:
    """A weight [N, K] as the products read it, kept once: a bf16 matrix whose sizes allow it (N a multiple of
    16, K of 32) lies in the order of the MFMA fragments (ops.pack_weight), which the products for single tokens
    need and the tiles for prompts read as well; any other lies in plain rows (`plain`)."""

    def __init__(self, w, keep_rows: bool = False):
        """keep_rows: leave w in plain rows whatever its sizes (a small matrix that only ever meets many rows)."""
        self.shape, self.dtype, self.device = tuple(w.shape), w.dtype, w.device
        self.packed = None if keep_rows else ops.pack_weight(w)
        self.plain = w if self.packed is None else None

    @property
    def data(self):
        """What ops.gemm, ops.gemm_swiglu and ops.embed take for this weight."""
        return self.plain if self.packed is None else self.packed

    def rows(self):
        """The matrix in plain rows (a copy, if it is kept in fragment order): for tests and tools."""
        return self.plain if self.packed is None else ops.unpack_weight(self.packed)

    def nbytes(self):
        t = self.data
        return t.numel() * t.element_size()


def _use_packed(x, m):
    return m.packed is not None and x.dtype == torch.bfloat16 and x.shape[0] <= ops.packed_max_rows(m.shape[0])


def _matrix(w):
    """The products below take a Matrix; a tensor [N, K] in plain rows is taken as it is."""
    return w if isinstance(w, Matrix) else Matrix(w, keep_rows=True)


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

    def __init__(self, x, w):
        self.x, self.w, self.packed = x, w, w.packed
        self.shape = (x.shape[0], w.shape[0])

    def run(self):
        return linear_for_sum(self.x, self.w)


def as_delta(d):
    """The delta of the residual rows as a tensor (or None), whatever form it arrives in."""
    return d.run() if isinstance(d, DeferredProduct) else d


def deferred_product(x, w):
    """linear_for_sum, but where the product would run over few rows in one slice it is only described:
    the caller's result is the delta that a following norm adds to the residual rows, and that norm can take the
    product in (RmsNorm.add_apply)."""
    w = _matrix(w)
    if isinstance(x, torch.Tensor) and _use_packed(x, w) and ops.packed_slices(w.shape[0], w.shape[1]) <= 1:
        return DeferredProduct(x, w)
    return linear_for_sum(x, w)


def linear(x, w, out_dtype):
    """x [M, K] in the activation type, w a Matrix [N, K]; a weight kept in 32-bit takes the 32-bit product."""
    w = _matrix(w)
    if _use_packed(x, w) and out_dtype in (torch.bfloat16, torch.float32):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=x.device)
        if isinstance(x, ScaledRows):
            ops.gemm_packed(x.rows, w.packed, out, row_scale=x.row_scale)
        else:
            ops.gemm_packed(x, w.packed, out)
        return out
    x = as_rows(x)
    if w.dtype != x.dtype:
        if w.dtype == torch.float32:
            x = x.to(torch.float32)
        else:
            raise TypeError(f"linear: activation {x.dtype} with weight {w.dtype}")
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32 if x.dtype == torch.float32 else out_dtype,
                      device=x.device)
    ops.gemm(x, w.data, out)
    return out if out.dtype == out_dtype else out.to(out_dtype)


def product_slices(n_rows, w, dtype) -> int:
    """Into how many slices of K the product of n_rows rows with w is cut for a reader that adds partial sums."""
    if w.dtype != dtype or (w.packed is not None and w.shape[1] % 128):
        return 1            # (in fragment order the tiles for many rows take a K that is a multiple of 128 only)
    return ops.gemm_slices(n_rows, w.shape[0], w.shape[1], dtype)


def linear_for_sum(x, w):
    """The product as float partial sums for a consumer that adds them up (the residual sum fused
    into the next norm): [S, M, N] when cutting K into S slices gives a small product more
    workgroups, else [M, N]."""
    w = _matrix(w)
    if _use_packed(x, w):
        slices = ops.packed_slices(w.shape[0], w.shape[1])
        if slices <= 1:
            return linear(x, w, torch.float32)
        out = torch.empty((slices, x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device)
        if isinstance(x, ScaledRows):
            ops.gemm_packed(x.rows, w.packed, out, row_scale=x.row_scale)
        else:
            ops.gemm_packed(x, w.packed, out)
        return out
    x = as_rows(x)
    M = x.shape[0]
    slices = product_slices(M, w, x.dtype)
    if slices <= 1:
        return linear(x, w, torch.float32)
    out = torch.empty((slices, M, w.shape[0]), dtype=torch.float32, device=x.device)
    ops.gemm(x, w.data, out)
    return out
