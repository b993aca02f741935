"""The kernels' plain C++ twins (csrc/ref/ref_kernels.cpp) as Python functions over float32 CPU tensors.

They take the arguments of their counterparts in `ops` (plain float layouts; V pages as [.., hd, 64]),
check nothing and run on the host: an oracle for tests, in the role of the reference's CPU kernels
(crates/synaptix-kernels-cpu/src/rmsnorm.rs:1-27, attention.rs:3-51)."""
from __future__ import annotations

import ctypes as C

import torch

from .build import load_library

_F32, _I32 = torch.float32, torch.int32


def _f(t):
    if t is None:
        return C.c_void_p(0)
    assert t.dtype in (_F32, _I32) and t.device.type == "cpu" and t.is_contiguous(), "the twins take contiguous float32 / int32 CPU tensors"
    return C.c_void_p(t.data_ptr())


def embed(table, ids, out):
    load_library("ref").ref_embed(_f(table), _f(ids), _f(out), ids.shape[0], table.shape[1])


def add_rmsnorm(resid, delta, gain, eps, out, gain_offset=0.0):
    load_library("ref").ref_add_rmsnorm(_f(resid), _f(delta), _f(gain), C.c_float(gain_offset), C.c_float(eps), _f(out),
                                        resid.shape[0], resid.shape[1])


def swiglu(gate_up, out):
    load_library("ref").ref_swiglu(_f(gate_up), _f(out), gate_up.shape[0], gate_up.shape[1] // 2)


def gemm(x, w, out):
    load_library("ref").ref_gemm(_f(x), _f(w), _f(out), x.shape[0], w.shape[0], x.shape[1])


def qk_norm_rope_kv_write(qkv, q_out, k_pages, v_pages, page_table, tok_seq, tok_pos, q_gain, k_gain, eps, cos, sin,
                          n_heads, n_kv_heads, head_dim, write_kv=True, gain_offset=0.0):
    load_library("ref").ref_qk_norm_rope_kv_write(
        _f(qkv), _f(q_out), _f(k_pages), _f(v_pages), _f(page_table), page_table.shape[1], _f(tok_seq), _f(tok_pos),
        _f(q_gain), _f(k_gain), C.c_float(gain_offset), C.c_float(eps), _f(cos), _f(sin),
        0 if cos is None else 2 * cos.shape[1], qkv.shape[0], n_heads, n_kv_heads, head_dim, 1 if write_kv else 0)


def attention(q, k_pages, v_pages, page_table, tok_seq, tok_pos, out, scale, window, n_heads, n_kv_heads, head_dim):
    load_library("ref").ref_attention(_f(q), _f(k_pages), _f(v_pages), _f(page_table), page_table.shape[1], _f(tok_seq),
                                      _f(tok_pos), _f(out), C.c_float(scale), int(window or 0), q.shape[0], n_heads,
                                      n_kv_heads, head_dim)


def sample_rows(logits, temperature, uniform, out):
    load_library("ref").ref_sample_rows(_f(logits), _f(temperature), _f(uniform), _f(out), logits.shape[0], logits.shape[1])
