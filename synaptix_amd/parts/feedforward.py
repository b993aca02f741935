"""Feed-forward parts.  Here: the gated MLP  down( act(gate(h)) * up(h) ), dense.

crates/synaptix-models/llm/common/src/model.rs:1670-1691; activation silu(z) = z / (1 + e^-z) in
32-bit as crates/synaptix-kernels-cuda/src/cu/fused/mlp/silu_and_mul.cu:11-52.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import Part
from .linear import Matrix, linear, linear_for_sum, deferred_product, as_rows, ScaledRows


class FeedForward(Part):
    """Interface: forward(h [N, hidden] activation type, ctx) -> residual delta [N, hidden] float."""

    takes_scaled_rows = False     # as Mixer.takes_scaled_rows

    def forward(self, h, ctx):
        raise NotImplementedError


class GatedMlp(FeedForward):
    takes_scaled_rows = True
    capturable = True

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "silu"):
        try:
            ops.activation_code(activation)       # the kernels apply it by its code; an unknown name is refused here
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        self.prefix, self.hidden, self.intermediate, self.activation = prefix, hidden, intermediate, activation
        self.w_gate_up = self.w_down = None
        self.paired = False      # gate and up rows in turns of 16: the activation runs inside the product

    def tensor_specs(self):
        p = self.prefix
        return {
            p + "gate_proj.weight": TensorSpec((self.intermediate, self.hidden)),
            p + "up_proj.weight": TensorSpec((self.intermediate, self.hidden)),
            p + "down_proj.weight": TensorSpec((self.hidden, self.intermediate)),
        }

    def load(self, get):
        p = self.prefix
        gate, up = get(p + "gate_proj.weight"), get(p + "up_proj.weight")
        self.paired = (gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16
                       and self.intermediate % ops.PAIR == 0 and self.hidden % 8 == 0)
        self.w_gate_up = Matrix(ops.pair_rows(gate, up) if self.paired else torch.cat([gate, up], 0))
        self.w_down = Matrix(get(p + "down_proj.weight"))

    def forward(self, h, ctx):
        m = torch.empty((h.shape[0], self.intermediate), dtype=h.dtype, device=h.device)
        if self.paired and h.dtype == torch.bfloat16:
            if self.w_gate_up.packed is not None and h.shape[0] <= ops.PACKED_MAX_ROWS_GATED:
                if isinstance(h, ScaledRows):      # the norm's last step is the product's epilogue
                    ops.gemm_packed(h.rows, self.w_gate_up.packed, m, paired=True, activation=self.activation,
                                    row_scale=h.row_scale)
                else:
                    ops.gemm_packed(h, self.w_gate_up.packed, m, paired=True, activation=self.activation)
            else:
                ops.gemm_swiglu(as_rows(h), self.w_gate_up.data, m, self.activation)
        else:
            h = as_rows(h)
            ops.swiglu(linear(h, self.w_gate_up, h.dtype), m, self.activation)
        return deferred_product(m, self.w_down)
