"""Token mixers.  Here: grouped-query attention over the paged cache.

GqaAttention: q/k/v projections (one fused product), optional per-head RMSNorm of q and k,
a position encoding, cache write, causal attention (optionally a window), output projection.
Order and formulas as crates/synaptix-models/llm/common/src/model.rs:1715-1734 (projections,
q/k norm before the rotation, the layer's eps), 1781-1782 (cache write), 1740-1869
(scores, scale, mask, softmax, PV), 1872-1878 (merge heads, o_proj).
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import Part, KvNeed
from .linear import Matrix, linear, linear_for_sum, product_slices, deferred_product, as_rows, ScaledRows
from .position import Position, NoPosition


class Mixer(Part):
    """Interface of a token mixer.

    cache_need(): KvNeed, StateNeed or None: what it keeps for each sequence.
    forward(h, ctx, cache, owner): h [N, hidden] in the activation type, ctx the step's
    StepContext, cache the view of its cache layer (None without a need); owner is False when the
    layer reads a cache that another layer writes.  Returns the residual delta as float [N, hidden],
    or as partial sums [S, N, hidden] that the following norm adds up.
    """

    # True: `h` may arrive as parts.linear.ScaledRows (rows whose norm a product over packed weights finishes)
    # and the returned delta may be a parts.linear.DeferredProduct; False (the default): plain tensors both ways
    takes_scaled_rows = False

    def cache_need(self):
        return None

    def forward(self, h, ctx, cache, owner=True):
        raise NotImplementedError


class GqaAttention(Mixer):
    takes_scaled_rows = True
    capturable = True

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, *,
                 position: Position | None = None, qk_norm_eps: float | None = None, scale: float | None = None,
                 window: int | None = None, qk_gain_offset: float = 0.0, score_softcap: float | None = None):
        if n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not divide into {n_kv_heads} kv heads")
        self.prefix = prefix
        self.hidden, self.nh, self.nkv, self.hd = hidden, n_heads, n_kv_heads, head_dim
        self.position = position or NoPosition()
        self.qk_norm_eps = qk_norm_eps
        self.qk_gain_offset = float(qk_gain_offset)     # the q/k gains are this + their tensors
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.window = window
        # a soft cap on the scaled scores, cap * tanh(score / cap); None: none.  What the position scheme adds to the
        # scores (Position.score_slopes) is asked for at the first step.
        self.score_softcap = float(score_softcap) if score_softcap else 0.0
        self._slopes = {}
        self.w_qkv = self.w_o = self.q_gain = self.k_gain = None

    def tensor_specs(self):
        p, hd = self.prefix, self.hd
        specs = {
            p + "q_proj.weight": TensorSpec((self.nh * hd, self.hidden)),
            p + "k_proj.weight": TensorSpec((self.nkv * hd, self.hidden)),
            p + "v_proj.weight": TensorSpec((self.nkv * hd, self.hidden)),
            p + "o_proj.weight": TensorSpec((self.hidden, self.nh * hd)),
        }
        if self.qk_norm_eps is not None:
            specs[p + "q_norm.weight"] = TensorSpec((hd,), "gain")
            specs[p + "k_norm.weight"] = TensorSpec((hd,), "gain")
        return specs

    def load(self, get):
        p = self.prefix
        # one product for q, k and v: rows of the three matrices one after another
        self.w_qkv = Matrix(torch.cat([get(p + "q_proj.weight"), get(p + "k_proj.weight"), get(p + "v_proj.weight")], 0))
        self.w_o = Matrix(get(p + "o_proj.weight"))
        if self.qk_norm_eps is not None:
            self.q_gain = get(p + "q_norm.weight")
            self.k_gain = get(p + "k_norm.weight").to(self.q_gain.dtype)

    def cache_need(self):
        return KvNeed(self.nkv, self.hd, self.window)

    def check(self, dtype):
        if self.hd % 2 or self.hd > ops.MAX_HEAD_DIM:
            raise ValueError(f"{self.prefix}: head size {self.hd} must be even and at most {ops.MAX_HEAD_DIM}")
        if dtype == torch.bfloat16 and self.hd % 16:
            raise ValueError(f"{self.prefix}: the bf16 attention kernels take head sizes in steps of 16 "
                             f"(16, 32, ..., {ops.MAX_HEAD_DIM}); {self.hd} runs in float32 only")

    def _score_terms(self, device):
        key = str(device)
        if key not in self._slopes:
            sl = self.position.score_slopes(self.nh, device)
            self._slopes[key] = None if sl is None else sl.to(device=device, dtype=torch.float32).contiguous()
        return dict(slopes=self._slopes[key], softcap=self.score_softcap)

    def _decode_work(self, ctx, cache, n_seqs):
        """For single tokens: the workspace of the splits' partial results, the number of splits, and
        what merges them inside the attention kernel (counters, and the step's work list if it keeps one)."""
        splits = ctx.decode_splits(self.nkv, cache.group)
        work = ctx.scratch("attention_decode", n_seqs * self.nh * splits * (self.hd + 2))
        merge = {}
        if splits > 1:
            chunks = -(-(self.nh // self.nkv) // 16)
            items = ctx.decode_items(cache.group)
            if items is not None and items.numel() != 4 * n_seqs * splits + 2 * n_seqs:
                items = None
            merge = dict(counters=ctx.counters("attention_decode_arrivals", n_seqs * self.nkv * chunks), items=items)
        return work, splits, merge

    def forward(self, h, ctx, cache, owner=True):
        nh, nkv, hd = self.nh, self.nkv, self.hd
        N, act = h.shape[0], h.dtype
        terms = self._score_terms(h.device)
        cap = self.position.capacity
        if cap is not None and ctx.max_position >= cap:
            raise ValueError(f"position {ctx.max_position} is beyond the position encoding's capacity {cap}")
        # single tokens: partial sums over slices of K, which the attention kernel adds; prompts: the plain product
        if self.w_qkv.packed is not None and N <= ops.PACKED_MAX_ROWS and act == torch.bfloat16:
            qkv = linear_for_sum(h, self.w_qkv)       # float partial sums [S, N, width]
            if qkv.dim() == 2:
                qkv = qkv.unsqueeze(0)
        else:
            h = as_rows(h)
            # (every kernel behind it adds partial sums itself; ops.gemm_slices cuts where the product would
            # otherwise leave compute units without work: single tokens and prompts up to about 1,200 tokens)
            sliced = product_slices(N, self.w_qkv, act) > 1
            qkv = linear_for_sum(h, self.w_qkv) if sliced else linear(h, self.w_qkv, act)
        cos, sin = self.position.tables(h.device)
        table = ctx.page_table(cache.group)
        o = torch.empty((N, nh * hd), dtype=act, device=h.device)
        window = self.window or 0
        if act == torch.bfloat16 and ctx.one_token_each:
            # single tokens: the attention kernel takes q, k and v from the projection itself
            work, splits, merge = self._decode_work(ctx, cache, N)
            ops.attention_decode_fused_bf16(qkv, cache.k_pages, cache.v_pages, table, ctx.seq_len, o, work, splits,
                                            self.scale, window, nh, nkv, hd, self.q_gain, self.k_gain,
                                            self.qk_norm_eps or 0.0, cos, sin, write_kv=owner,
                                            gain_offset=self.qk_gain_offset, **terms, **merge)
            return deferred_product(o, self.w_o)
        q = torch.empty((N, nh * hd), dtype=act, device=h.device)
        ops.qk_norm_rope_kv_write(qkv, q, cache.k_pages, cache.v_pages, table, ctx.tok_seq, ctx.tok_pos,
                                  self.q_gain, self.k_gain, self.qk_norm_eps or 0.0, cos, sin, nh, nkv, hd,
                                  write_kv=owner, gain_offset=self.qk_gain_offset)
        if act == torch.float32:
            ops.attention_f32(q, cache.k_pages, cache.v_pages, table, ctx.tok_seq, ctx.tok_pos, o, self.scale, window,
                              nh, nkv, hd, **terms)
        elif ctx.one_token_each:
            work, splits, merge = self._decode_work(ctx, cache, N)
            ops.attention_decode_bf16(q, cache.k_pages, cache.v_pages, table, ctx.seq_len, o, work, splits,
                                      self.scale, window, nh, nkv, hd, **terms, **merge)
        else:
            # a step of prompts and single tokens: the prompts' kernel leaves the single tokens out, and the kernel
            # for single tokens takes them (gathered, since it counts one row a sequence)
            singles = ctx.single_token_rows()
            ops.attention_prefill_bf16(q, cache.k_pages, cache.v_pages, table, ctx.seq_start, ctx.seq_past, o,
                                       self.scale, window, nh, nkv, hd, skip_below=2 if singles is not None else 0, **terms)
            if singles is not None:
                rows, seqs = singles
                n1 = rows.numel()
                q1, o1 = q.index_select(0, rows), torch.empty((n1, nh * hd), dtype=act, device=h.device)
                splits = ops.decode_splits(n1, nkv, table.shape[1])
                work = ctx.scratch("attention_decode", n1 * nh * splits * (hd + 2))
                ops.attention_decode_bf16(q1, cache.k_pages, cache.v_pages, table.index_select(0, seqs),
                                          ctx.seq_len.index_select(0, seqs), o1, work, splits, self.scale, window,
                                          nh, nkv, hd, **terms)
                o.index_copy_(0, rows, o1)
        return deferred_product(o, self.w_o)
