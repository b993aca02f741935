"""Stand-ins for the GPU kernels, written with torch CPU ops, for tests that run without a GPU.

They let the engine's own logic (packing of a step, the cache, page tables, the order of layers,
the generation loop) run on the CPU against the plain implementation.  They are test equipment:
nothing in the package imports them, and the package has no CPU path of its own.
Each function has the signature and the meaning of its namesake in synaptix_amd.kernels.ops.
"""
from __future__ import annotations


import numpy as np
import torch

from synaptix_amd.engine.engine import Engine
from synaptix_amd.engine.batch import fill_host_buffer

PAGE = 64
F32 = torch.float32


def _rows(w):
    """A weight in plain rows, whether it comes so or in fragment order (pack_weight: four dimensions)."""
    if w.dim() == 4:
        from synaptix_amd.kernels import ops
        return ops.unpack_weight(w)
    return w


def embed(table, ids, resid):
    resid.copy_(_rows(table)[ids.long()].to(F32))


def add_rmsnorm(resid, delta, gain, eps, out, rows=None, gain_offset=0.0):
    if delta is not None and delta.dim() == 3:
        delta = delta.sum(0)
    if rows is None:
        if delta is not None:
            resid.add_(delta)
        x = resid
    else:
        x = resid[rows.long()]
        if delta is not None:
            x = x + delta[rows.long()]
    inv = torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    out.copy_(((gain_offset + gain.to(F32)) * x * inv).to(out.dtype))


def rmsnorm_rows(x, gain, eps, out, gain_offset=0.0):
    xf = x.to(F32)
    inv = torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
    out.copy_(((gain_offset + gain.to(F32)) * xf * inv).to(out.dtype))


def swiglu(gate_up, out, activation="silu"):
    assert activation in ("silu", "swish")
    I = gate_up.shape[1] // 2
    g, u = gate_up[:, :I].to(F32), gate_up[:, I:].to(F32)
    out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))


def gemm(x, w, out, force_simt=False):
    w = _rows(w)
    if out.dim() == 3:                      # partial sums over slices of K
        S, K = out.shape[0], x.shape[1]
        step = ((K + S - 1) // S + 127) // 128 * 128
        for s in range(S):
            out[s] = x[:, s * step:(s + 1) * step].to(F32) @ w[:, s * step:(s + 1) * step].to(F32).T
        return
    out.copy_((x.to(F32) @ w.to(F32).T).to(out.dtype))


PAIR = 16


def gemm_swiglu(x, w_paired, out, activation="silu"):
    assert activation in ("silu", "swish")
    w_paired = _rows(w_paired)
    N, K = w_paired.shape
    w = w_paired.view(N // (2 * PAIR), 2, PAIR, K)
    g = x.to(F32) @ w[:, 0].reshape(N // 2, K).to(F32).T
    u = x.to(F32) @ w[:, 1].reshape(N // 2, K).to(F32).T
    out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))


def gemm_packed(x, wp, out, paired=False, activation="silu", row_scale=None, resid_norm=None):
    from synaptix_amd.kernels import ops
    w = ops.unpack_weight(wp)
    factor = None
    if row_scale is not None:      # the second half of a norm carried between two products
        ss, dim, eps = row_scale
        factor = torch.rsqrt(ss.sum(1) / torch.tensor(float(dim), dtype=F32) + torch.tensor(eps, dtype=F32))[:, None]
    if resid_norm is not None:     # the first half: sums into the residual rows, the gain, the statistic in groups of 16
        resid, gain, gain_offset, xs, ss_out = resid_norm
        sums = x.to(F32) @ w.to(F32).T
        if factor is not None:
            sums = sums * factor
        resid += sums
        xs.copy_(((gain_offset + gain.to(F32)) * resid).to(xs.dtype))
        ss_out.copy_((resid * resid).view(resid.shape[0], -1, 16).sum(2))
        return
    if paired:
        N, K = w.shape
        wv = w.view(N // (2 * PAIR), 2, PAIR, K)
        g = x.to(F32) @ wv[:, 0].reshape(N // 2, K).to(F32).T
        u = x.to(F32) @ wv[:, 1].reshape(N // 2, K).to(F32).T
        if factor is not None:
            g, u = g * factor, u * factor
        out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))
    elif out.dim() == 3:                    # partial sums over slices of K (whole k-steps of 32)
        S, K = out.shape[0], w.shape[1]
        step = -(-(K // 32) // S) * 32
        for i in range(S):
            part = x[:, i * step:(i + 1) * step].to(F32) @ w[:, i * step:(i + 1) * step].to(F32).T
            out[i] = part if factor is None else part * factor
    else:
        y = x.to(F32) @ w.to(F32).T
        out.copy_((y if factor is None else y * factor).to(out.dtype))


def stream_scope():
    import contextlib
    return contextlib.nullcontext()


def gemm_slices(M, N, K, dtype):
    return 2 if (dtype == torch.bfloat16 and M <= 16 and K >= 64 and K % 8 == 0) else 1


def qk_norm_rope_kv_write(qkv, q_out, k_pages, v_pages, page_table, tok_seq, tok_pos, q_gain, k_gain, eps,
                          cos, sin, n_heads, n_kv_heads, head_dim, write_kv=True, gain_offset=0.0):
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    if qkv.dim() == 3:                      # partial sums over slices of K
        qkv = qkv.sum(0)
    N = qkv.shape[0]
    x = qkv.to(F32).view(N, nh + 2 * nkv, hd)
    q, k, v = x[:, :nh], x[:, nh:nh + nkv], x[:, nh + nkv:]

    def norm(t, g):
        if g is None:
            return t
        return (gain_offset + g.to(F32)) * t * torch.rsqrt((t * t).mean(-1, keepdim=True) + eps)

    def rope(t):
        if cos is None:
            return t
        half = cos.shape[1]
        c, s = cos[tok_pos.long()][:, None, :], sin[tok_pos.long()][:, None, :]
        a, b, rest = t[..., :half], t[..., half:2 * half], t[..., 2 * half:]
        return torch.cat([a * c - b * s, b * c + a * s, rest], -1)

    q_out.copy_(rope(norm(q, q_gain)).reshape(N, nh * hd).to(q_out.dtype))
    if not write_kv:
        return
    k = rope(norm(k, k_gain))
    for n in range(N):
        p = int(tok_pos[n])
        page = int(page_table[int(tok_seq[n]), p // PAGE])
        k_pages[page, :, p % PAGE, :] = k[n].to(k_pages.dtype)
        v_pages[page, :, :, p % PAGE] = v[n].to(v_pages.dtype)


def _attend(qrow, k_pages, v_pages, table_row, pos, scale, window, nh, nkv, hd, slopes=None, softcap=0.0):
    T = pos + 1
    pages = table_row[:(T + PAGE - 1) // PAGE].long()
    K = k_pages[pages].to(F32).permute(1, 0, 2, 3).reshape(nkv, -1, hd)[:, :T]          # [nkv, T, hd]
    V = v_pages[pages].to(F32).permute(1, 2, 0, 3).reshape(nkv, hd, -1)[:, :, :T]       # [nkv, hd, T]
    lo = max(0, pos - window + 1) if window and window > 0 else 0
    g = nh // nkv
    out = torch.empty(nh, hd)
    for h in range(nh):
        s = (K[h // g, lo:] @ qrow[h]) * scale
        if softcap:                      # a soft cap on the scaled scores, then a penalty in the distance to the query
            s = softcap * torch.tanh(s / softcap)
        if slopes is not None:
            s = s - float(slopes[h]) * (pos - torch.arange(lo, T, dtype=F32))
        p = torch.softmax(s, 0)
        out[h] = V[h // g][:, lo:] @ p
    return out


def attention_f32(q, k_pages, v_pages, page_table, tok_seq, tok_pos, out, scale, window, n_heads, n_kv_heads,
                  head_dim, slopes=None, softcap=0.0):
    N = q.shape[0]
    qf = q.to(F32).view(N, n_heads, head_dim)
    for n in range(N):
        o = _attend(qf[n], k_pages, v_pages, page_table[int(tok_seq[n])], int(tok_pos[n]), scale, window,
                    n_heads, n_kv_heads, head_dim, slopes, softcap)
        out[n] = o.reshape(-1).to(out.dtype)


def attention_prefill_bf16(q, k_pages, v_pages, page_table, seq_start, seq_past, out, scale, window, n_heads,
                           n_kv_heads, head_dim, variant=0, slopes=None, softcap=0.0, skip_below=0):
    N = q.shape[0]
    qf = q.to(F32).view(N, n_heads, head_dim)
    for b in range(seq_past.shape[0]):
        if int(seq_start[b + 1]) - int(seq_start[b]) < skip_below:
            continue
        for n in range(int(seq_start[b]), int(seq_start[b + 1])):
            pos = int(seq_past[b]) + n - int(seq_start[b])
            o = _attend(qf[n], k_pages, v_pages, page_table[b], pos, scale, window, n_heads, n_kv_heads, head_dim,
                        slopes, softcap)
            out[n] = o.reshape(-1).to(out.dtype)


def decode_splits(n_seqs, n_kv_heads, max_pages):
    return 1


def attention_decode_bf16(q, k_pages, v_pages, page_table, seq_len, out, workspace, n_splits, scale, window,
                          n_heads, n_kv_heads, head_dim, slopes=None, softcap=0.0, counters=None, items=None):
    B = q.shape[0]
    qf = q.to(F32).view(B, n_heads, head_dim)
    for b in range(B):
        o = _attend(qf[b], k_pages, v_pages, page_table[b], int(seq_len[b]) - 1, scale, window, n_heads,
                    n_kv_heads, head_dim, slopes, softcap)
        out[b] = o.reshape(-1).to(out.dtype)


def attention_decode_fused_bf16(qkv, k_pages, v_pages, page_table, seq_len, out, workspace, n_splits, scale, window,
                                n_heads, n_kv_heads, head_dim, q_gain, k_gain, eps, cos, sin, write_kv=True,
                                gain_offset=0.0, slopes=None, softcap=0.0, counters=None, items=None):
    B = qkv.shape[-2]
    q = torch.empty((B, n_heads * head_dim), dtype=torch.bfloat16)
    tok_seq = torch.arange(B, dtype=torch.int32)
    tok_pos = (seq_len - 1).to(torch.int32)
    qk_norm_rope_kv_write(qkv, q, k_pages, v_pages, page_table, tok_seq, tok_pos, q_gain, k_gain, eps, cos, sin,
                          n_heads, n_kv_heads, head_dim, write_kv=write_kv, gain_offset=gain_offset)
    attention_decode_bf16(q, k_pages, v_pages, page_table, seq_len, out, workspace, n_splits, scale, window,
                          n_heads, n_kv_heads, head_dim, slopes, softcap)


def sample_rows(logits, temperature, uniform, out):
    for r in range(logits.shape[0]):
        x = logits[r]
        T = 0.0 if temperature is None else float(temperature[r])
        if not T > 0:
            m = x.max()
            out[r] = int(torch.nonzero(x == m)[-1])
            continue
        if T != 1.0:
            x = x / torch.tensor(T, dtype=F32)
        p = torch.softmax(x, 0)
        hit = torch.nonzero(float(uniform[r]) < torch.cumsum(p, 0))
        out[r] = int(hit[0]) if hit.numel() else x.numel() - 1


def filter_rows(logits, out, temperature, top_k, top_p, min_p, repetition, presence, frequency,
                ids=None, id_start=None, counts=None):
    R, V = logits.shape
    for r in range(R):
        x = logits[r].clone()
        row_ids = [] if ids is None else [int(t) for t in ids[int(id_start[r]):int(id_start[r + 1])]]
        rep, pres, freq = float(repetition[r]), float(presence[r]), float(frequency[r])
        if row_ids and (rep != 1.0 or pres != 0.0 or freq != 0.0):
            cnt = torch.bincount(torch.tensor([t for t in row_ids if 0 <= t < V], dtype=torch.long), minlength=V).to(F32)
            seen = cnt > 0
            if rep != 1.0:
                f = torch.pow(torch.tensor(rep, dtype=F32), cnt)
                x = torch.where(seen, torch.where(x > 0, x / f, x * f), x)
            if pres != 0.0 or freq != 0.0:
                x = torch.where(seen, x - (pres + freq * cnt), x)
        T = float(temperature[r])
        if T > 0.0 and T != 1.0:
            x = x / torch.tensor(T, dtype=F32)
        k = int(top_k[r])
        if 0 < k < V:
            order = torch.argsort(x, descending=True, stable=True)        # equal values: the first in index order
            x[order[k:]] = float("-inf")
        if float(top_p[r]) < 1.0:
            probs = torch.exp(x - x.max())
            order = torch.argsort(probs, descending=True, stable=True)
            sp = probs[order]
            before = torch.cumsum(sp, 0) - sp
            drop = order[(before > float(top_p[r]) * probs.sum()) & torch.isfinite(x[order])]
            x[drop] = float("-inf")
        if float(min_p[r]) > 0.0:
            e = torch.exp(x - x.max())
            x = torch.where(torch.isfinite(x) & (e < float(min_p[r])), torch.full_like(x, float("-inf")), x)
        out[r] = x


ALL = ["embed", "add_rmsnorm", "rmsnorm_rows", "swiglu", "gemm", "gemm_swiglu", "gemm_packed", "stream_scope", "gemm_slices", "qk_norm_rope_kv_write", "attention_f32",
       "attention_prefill_bf16", "decode_splits", "attention_decode_bf16", "attention_decode_fused_bf16", "sample_rows", "filter_rows"]


def install(monkeypatch):
    """Replace the kernels by the stand-ins for the duration of a test."""
    from synaptix_amd.kernels import ops
    import sys
    me = sys.modules[__name__]
    for name in ALL:
        monkeypatch.setattr(ops, name, getattr(me, name))


class CpuEngine(Engine):
    """The engine with the two places that need a GPU (the device check, the pinned upload) replaced."""

    def __init__(self, *args, **kw):
        super().__init__(*args, **kw)
        self.graph_ok = False            # graphs are a GPU matter

    def _require_gpu(self):
        pass

    def _upload(self, layout, slots, tokens_flat, counts, want_rows):
        host = np.zeros(layout.total, dtype=np.int32)
        fill_host_buffer(layout, host, self.cache, slots, tokens_flat, counts, want_rows)
        return torch.from_numpy(host)
