"""RMSNorm as a part: y = gain * x * rsqrt(mean(x^2) + eps), arithmetic in 32-bit.

Formula and order of the product as in crates/synaptix-ops/src/norm/rms_norm.rs:16-26 and
crates/synaptix-kernels-cuda/src/cu/reduction/rms_norm.cu:65-98 (plain gain `w`, not `1 + w`).
The residual sum of the block is fused in (`add_apply`), as the reference's graph path does with
crates/synaptix-kernels-cuda/src/cu/fused/norm/rmsnorm_residual.cu:97-159; here the residual stream
itself stays in 32-bit.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import Part
from .linear import DeferredProduct, ScaledRows


class RmsNorm(Part):
    capturable = True
    takes_deferred_product = True     # add_apply accepts a parts.linear.DeferredProduct as delta and may return ScaledRows

    def __init__(self, name: str, dim: int, eps: float, gain_offset: float = 0.0):
        """gain_offset: the gain is gain_offset + the stored tensor (0 here; 1 for checkpoints that store
        the gain as a difference from one, crates/synaptix-models/llm/common/src/config.rs:1-5)."""
        self.name = name          # full tensor name of the gain
        self.dim = dim
        self.eps = float(eps)
        self.gain_offset = float(gain_offset)
        self.gain = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.dim,), "gain")}

    def load(self, get):
        self.gain = get(self.name)

    def add_apply(self, resid, delta, out_dtype, rows=None):
        """resid [N, dim] float: with rows None, resid += delta (if any) in place and every row is
        normed; with rows [n] int32 only those rows of resid + delta are normed and resid is kept."""
        if isinstance(delta, DeferredProduct):
            # a product over packed weights for few rows: it adds its sums into resid itself and leaves the rows with
            # the gain and the row statistic in groups; the product that follows applies the row's factor
            if (rows is None and out_dtype == torch.bfloat16 and delta.shape == tuple(resid.shape)
                    and self.dim % 16 == 0):
                xs = torch.empty(resid.shape, dtype=torch.bfloat16, device=resid.device)
                ss = torch.empty((resid.shape[0], self.dim // 16), dtype=torch.float32, device=resid.device)
                ops.gemm_packed(delta.x, delta.packed, None, resid_norm=(resid, self.gain, self.gain_offset, xs, ss))
                return ScaledRows(xs, ss, self.eps, resid, self)
            delta = delta.run()
        n = resid.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n, self.dim), dtype=out_dtype, device=resid.device)
        ops.add_rmsnorm(resid, delta, self.gain, self.eps, out, rows, self.gain_offset)
        return out

    def apply(self, x):
        """Norm over the last axis of a tensor in the activation type."""
        out = torch.empty_like(x)
        ops.rmsnorm_rows(x, self.gain, self.eps, out, self.gain_offset)
        return out
