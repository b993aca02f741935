"""The kernels as Python functions over torch tensors on the GPU.

Every function checks on the host that shapes, types and layouts are what its kernel and grid
assume, then launches on torch's current stream.  There is no other implementation behind
these names: without the built library, or with tensors that are not on the GPU, they raise.
"""
from __future__ import annotations

import contextlib
import ctypes
import threading

import torch

from .build import load_library

PAGE_TOKENS = 64          # tokens in a cache page; the kernels are compiled with the same number
MAX_HEAD_DIM = 256
_F32, _BF16, _I32 = torch.float32, torch.bfloat16, torch.int32


class KernelError(RuntimeError):
    pass


_scope = threading.local()


def _stream():
    held = getattr(_scope, "stream", None)
    return held if held is not None else ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


@contextlib.contextmanager
def stream_scope():
    """Within the scope every kernel of this thread is launched on the stream that is current when the scope
    is entered, asked for once (a model's forward pass launches some 300 kernels and never changes the
    stream; asking torch each time costs more than the launch).  Scopes nest; code that switches streams
    inside one opens a new one."""
    before = getattr(_scope, "stream", None)
    _scope.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    try:
        yield
    finally:
        _scope.stream = before


def _ptr(t):
    return ctypes.c_void_p(0) if t is None else ctypes.c_void_p(t.data_ptr())


def _need(t, name, dtypes, shape=None):
    # the checks in the order of their cost; the messages are built only when one fails
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    dt = t.dtype
    if dt is not dtypes and (dtypes.__class__ is torch.dtype or dt not in dtypes):
        want = dtypes if isinstance(dtypes, (tuple, list)) else (dtypes,)
        raise KernelError(f"{name}: dtype {dt}, expected {' or '.join(str(d) for d in want)}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor lies on {t.device}; the kernels of synaptix_amd run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if shape is not None:
        got = t.shape
        ok = len(shape) == len(got)
        if ok:
            for s, g in zip(shape, got):
                if s is not None and s != g:
                    ok = False
                    break
        if not ok:
            raise KernelError(f"{name}: shape {list(got)}, expected {[('*' if s is None else s) for s in shape]}")


def _call(lib, fn, *args):
    if _timing is not None:
        return _timed_call(lib, fn, args)
    rc = getattr(lib, fn)(*args)
    if rc != 0:
        raise KernelError(lib.syn_last_error().decode(errors="replace"))


# ----------------------------------------------------------------------------- per-op times
# The reference can time every op of a forward pass by synchronising the device around it
# (crates/synaptix-models/llm/common/src/model.rs:22-99: prof(name, f), a table of (ms, calls) by name,
# sorted by time, switched on for prefill or decode; off during graph capture).  Here the ops are the
# kernel entry points; op_timing() switches the same thing on for the code inside it.

_timing = None      # None, or {entry point: [milliseconds, calls]}


def _timed_call(lib, fn, args):
    import time
    if torch.cuda.is_current_stream_capturing():
        raise KernelError("op_timing: per-op times need eager steps (synchronising is not allowed while a graph is captured)")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    rc = getattr(lib, fn)(*args)
    torch.cuda.synchronize()
    slot = _timing.setdefault(fn, [0.0, 0])
    slot[0] += (time.perf_counter() - t0) * 1e3
    slot[1] += 1
    if rc != 0:
        raise KernelError(lib.syn_last_error().decode(errors="replace"))


def timing_active() -> bool:
    return _timing is not None


class OpTimes(dict):
    """{entry point: [milliseconds, calls]} with the reference's report: sorted by time, with shares."""

    def report(self) -> str:
        total = sum(v[0] for v in self.values()) or 1.0
        lines = [f"{'op':34s} {'ms':>10s} {'calls':>7s} {'share':>7s}"]
        for name, (ms, calls) in sorted(self.items(), key=lambda kv: -kv[1][0]):
            lines.append(f"{name:34s} {ms:10.3f} {calls:7d} {100 * ms / total:6.1f}%")
        lines.append(f"{'total':34s} {total:10.3f}")
        return "\n".join(lines)


@contextlib.contextmanager
def op_timing():
    """Within the scope every kernel entry point is timed with the device synchronised before and after it
    (so the times include each launch's latency and nothing overlaps); yields the table that fills up.
    Steps inside the scope must be eager: captured steps are refused."""
    global _timing
    before, _timing = _timing, OpTimes()
    try:
        yield _timing
    finally:
        _timing = before


def _is_f32(t):
    return 1 if t.dtype == _F32 else 0


# The activations of a gated feed-forward that the kernels apply (codes of gate_activation in csrc/common.h).
ACTIVATIONS = {"silu": 0, "swish": 0}


def activation_code(name) -> int:
    if name not in ACTIVATIONS:
        raise KernelError(f"activation {name!r}: the kernels apply {sorted(set(ACTIVATIONS))}")
    return ACTIVATIONS[name]


# ----------------------------------------------------------------------------- rows

def embed(table, ids, resid):
    """resid[n, :] = table[ids[n], :] as float.  table [V, H] bf16|f32 (or bf16 in fragment order, pack_weight: four
    dimensions), ids [N] int32, resid [N, H] f32."""
    if isinstance(table, torch.Tensor) and table.dim() == 4:
        _need(table, "embed.table", _BF16, (None, None, 64, 8))
        H, kind = table.shape[1] * 32, 2
    else:
        _need(table, "embed.table", (_BF16, _F32), (None, None))
        H, kind = table.shape[1], _is_f32(table)
    _need(ids, "embed.ids", _I32, (None,))
    _need(resid, "embed.resid", _F32, (ids.shape[0], H))
    _call(load_library("core"), "syn_embed", _ptr(table), kind, _ptr(ids), _ptr(resid), ids.shape[0], H, _stream())


def add_rmsnorm(resid, delta, gain, eps, out, rows=None, gain_offset=0.0):
    """rows is None:  resid += delta (when given), out = RMSNorm(resid) * (gain_offset + gain), for every row.
    rows [n] int32: out[i] = RMSNorm(resid[rows[i]] + delta[rows[i]]) * gain; resid is not written.
    delta may be [S, N, H]: partial sums that are added up on the way."""
    _need(resid, "add_rmsnorm.resid", _F32, (None, None))
    N, H = resid.shape
    n_parts = 1
    if delta is not None:
        if delta.dim() == 3:
            n_parts = delta.shape[0]
            _need(delta, "add_rmsnorm.delta", _F32, (n_parts, N, H))
        else:
            _need(delta, "add_rmsnorm.delta", _F32, (N, H))
    _need(gain, "add_rmsnorm.gain", (_BF16, _F32), (H,))
    n_out = N
    if rows is not None:
        _need(rows, "add_rmsnorm.rows", _I32, (None,))
        n_out = rows.shape[0]
    _need(out, "add_rmsnorm.out", (_BF16, _F32), (n_out, H))
    _call(load_library("core"), "syn_add_rmsnorm", _ptr(resid), _ptr(delta), n_parts, N, _ptr(rows), n_out, _ptr(gain),
          _is_f32(gain), ctypes.c_float(gain_offset), ctypes.c_float(eps), _ptr(out), _is_f32(out), H, _stream())


def rmsnorm_rows(x, gain, eps, out, gain_offset=0.0):
    """out = RMSNorm(x) * (gain_offset + gain) over the last axis; x [..., D] bf16|f32, out like x."""
    _need(x, "rmsnorm_rows.x", (_BF16, _F32))
    D = x.shape[-1]
    _need(gain, "rmsnorm_rows.gain", (_BF16, _F32), (D,))
    _need(out, "rmsnorm_rows.out", x.dtype, tuple(x.shape))
    _call(load_library("core"), "syn_rmsnorm_rows", _ptr(x), _is_f32(x), _ptr(gain), _is_f32(gain),
          ctypes.c_float(gain_offset), ctypes.c_float(eps), _ptr(out), x.numel() // D, D, _stream())


def swiglu(gate_up, out, activation="silu"):
    """out[n, i] = act(gate_up[n, i]) * gate_up[n, I + i]."""
    _need(gate_up, "swiglu.gate_up", (_BF16, _F32), (None, None))
    N, I2 = gate_up.shape
    if I2 % 2:
        raise KernelError(f"swiglu: fused width {I2} is odd")
    _need(out, "swiglu.out", gate_up.dtype, (N, I2 // 2))
    _call(load_library("core"), "syn_swiglu", _ptr(gate_up), _ptr(out), _is_f32(gate_up), N, I2 // 2,
          activation_code(activation), _stream())


# ----------------------------------------------------------------------------- matrix product

def _packed_shape(w, name, K):
    """(N, K) of a weight in fragment order (pack_weight), checked against the rows' width."""
    _need(w, name, _BF16, (None, K // 32 if K % 32 == 0 else -1, 64, 8))
    return w.shape[0] * 16


def gemm(x, w, out, force_simt=False):
    """out[M, N] = x[M, K] . w[N, K]^T with 32-bit accumulation.
    float x float -> float (plain FMA); bf16 x bf16 -> bf16 or float (MFMA).
    A float out of shape [S, M, N] (bf16 operands) receives S partial sums over slices of K
    instead; their sum over S is the product.
    w may be the weight in fragment order (pack_weight: four dimensions): the tiles for 9 rows and more read it
    where K is a multiple of 128; for other K the product runs in blocks of 16 rows through gemm_packed."""
    _need(x, "gemm.x", (_BF16, _F32), (None, None))
    M, K = x.shape
    packed = isinstance(w, torch.Tensor) and w.dim() == 4
    if packed:
        if x.dtype != _BF16 or force_simt:
            raise KernelError("gemm: a weight in fragment order takes bf16 rows and the MFMA kernels")
        N = _packed_shape(w, "gemm.w", K)
        if K % 128:
            if out.dim() == 3 and out.shape[0] != 1:
                raise KernelError(f"gemm: no slices of K = {K} over a weight in fragment order")
            rows = out[0] if out.dim() == 3 else out
            for m0 in range(0, M, PACKED_BLOCK_ROWS):
                gemm_packed(x[m0:m0 + PACKED_BLOCK_ROWS], w, rows[m0:m0 + PACKED_BLOCK_ROWS])
            return
    else:
        _need(w, "gemm.w", x.dtype, (None, K))
        N = w.shape[0]
    slices = 1
    if out.dim() == 3:
        slices = out.shape[0]
        if x.dtype != _BF16 or force_simt or (M > 64 and K % 64):
            raise KernelError("gemm: partial sums over slices of K need bf16 operands (and beyond 64 rows a K "
                              "that is a multiple of 64)")
        _need(out, "gemm.out", _F32, (slices, M, N))
        code = 2
    elif x.dtype == _F32:
        _need(out, "gemm.out", _F32, (M, N))
        code = 0
    else:
        _need(out, "gemm.out", (_BF16, _F32), (M, N))
        code = 2 if out.dtype == _F32 else 1
    _call(load_library("core"), "syn_gemm", _ptr(x), _ptr(w), _ptr(out), code, M, N, K, 1 if force_simt else 0,
          slices, 1 if packed else 0, _stream())


PAIR = 16   # rows of the gate and of the up projection alternate in turns of this many


def pair_rows(gate, up):
    """The weight of gemm_swiglu: rows of `gate` and of `up` [I, K] in turns of 16 -> [2 I, K]."""
    I, K = gate.shape
    if up.shape != gate.shape or I % PAIR:
        raise KernelError(f"pair_rows: shapes {tuple(gate.shape)}, {tuple(up.shape)} (rows in turns of {PAIR})")
    return torch.stack([gate.view(I // PAIR, PAIR, K), up.view(I // PAIR, PAIR, K)], 1).reshape(2 * I, K).contiguous()


def gemm_swiglu(x, w_paired, out, activation="silu"):
    """out[M, I] = act(x . Wg^T) * (x . Wu^T) in bf16 with w_paired = pair_rows(Wg, Wu): the
    activation on the 32-bit sums inside the product, so that the two products are never stored.
    w_paired may be in fragment order (pack_weight of the paired rows), as for gemm."""
    _need(x, "gemm_swiglu.x", _BF16, (None, None))
    M, K = x.shape
    packed = isinstance(w_paired, torch.Tensor) and w_paired.dim() == 4
    if packed:
        N = _packed_shape(w_paired, "gemm_swiglu.w", K)
    else:
        _need(w_paired, "gemm_swiglu.w", _BF16, (None, K))
        N = w_paired.shape[0]
    if N % (2 * PAIR) or K % 8:
        raise KernelError(f"gemm_swiglu: {N} paired rows, K = {K} (multiples of {2 * PAIR} and of 8)")
    _need(out, "gemm_swiglu.out", _BF16, (M, N // 2))
    if packed and K % 128:
        for m0 in range(0, M, PACKED_BLOCK_ROWS):
            gemm_packed(x[m0:m0 + PACKED_BLOCK_ROWS], w_paired, out[m0:m0 + PACKED_BLOCK_ROWS], paired=True,
                        activation=activation)
        return
    _call(load_library("core"), "syn_gemm_swiglu", _ptr(x), _ptr(w_paired), _ptr(out), M, N, K,
          activation_code(activation), 1 if packed else 0, _stream())


PACKED_BLOCK_ROWS = 16   # the most rows that a product of gemm_packed takes
PACKED_MAX_ROWS = 8   # up to this many rows of x the products over packed weights are the faster ones
PACKED_MAX_ROWS_GATED = 16   # the gated product, whose waves take two groups of rows of W for every fragment of x
PACKED_WIDE_N = 32768   # from this many rows of W on (an output head) the products over packed weights stay the faster
                        # ones up to 16 rows of x (151,936 x 4,096 at 16 rows: 222 us on tiles, as at 8 rows in fragments)


def packed_max_rows(n_out: int) -> int:
    """Up to how many rows of x a plain product with a packed weight of n_out rows takes the kernels for few rows."""
    return PACKED_BLOCK_ROWS if n_out >= PACKED_WIDE_N else PACKED_MAX_ROWS


def pack_weight(w):
    """A copy of the bf16 weight w [N, K] in the order of the MFMA fragments that the products for few
    rows take: [N / 16, K / 32, 64, 8] with lane = 16 * (k % 32 // 8) + n % 16 (every load of a wave is then
    1 KB of consecutive bytes).  None if the shape or the type does not allow it (N a multiple of 16, K of 32)."""
    if w.dtype != _BF16 or w.dim() != 2 or w.shape[0] % 16 or w.shape[1] % 32:
        return None
    N, K = w.shape
    return w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).reshape(N // 16, K // 32, 64, 8).contiguous()


def unpack_weight(wp):
    """The inverse of pack_weight: [N, K]."""
    nt, nks = wp.shape[:2]
    return wp.view(nt, nks, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nt * 16, nks * 32).contiguous()


def gemm_packed(x, wp, out, paired=False, activation="silu", row_scale=None, resid_norm=None):
    """out[M, N] (bf16 or float) = x[M, K] . W^T for M <= 16 with wp = pack_weight(W); paired: W holds gate and
    up rows in turns of 16 (pair_rows) and out [M, N / 2] bf16 = act(gate) * up.  A float out of shape
    [S, M, N] receives S partial sums over slices of K instead.

    The two halves of an RMSNorm that lies between two such products (csrc/gemm.hip: RowNorm):
    resid_norm = (resid [M, N] float, gain [N], gain_offset, xs [M, N] bf16, ss [M, N / 16] float) with out None:
    the sums are added into resid, xs = (gain_offset + gain) * resid, ss = sums of resid^2 over groups of 16 columns;
    row_scale = (ss [M, G] float, dim, eps): the sums of row m are multiplied by rsqrt(sum(ss[m]) / dim + eps), which
    makes this the product over the normed rows when x is the xs that came with ss."""
    _need(x, "gemm_packed.x", _BF16, (None, None))
    M, K = x.shape
    if K % 32:
        raise KernelError(f"gemm_packed: K = {K} is no multiple of 32")
    _need(wp, "gemm_packed.wp", _BF16, (None, K // 32, 64, 8))
    N = wp.shape[0] * 16
    if M > 16 or (paired and N % 32):
        raise KernelError(f"gemm_packed: M = {M} (at most 16), N = {N}")
    slices = 1
    ss = resid = xs = ss_out = gain = None
    groups = dim = 0
    eps = gain_offset = 0.0
    if row_scale is not None:
        ss, dim, eps = row_scale
        _need(ss, "gemm_packed.row_scale", _F32, (M, None))
        groups = ss.shape[1]
        if groups < 1 or dim < 1:
            raise KernelError(f"gemm_packed: a row statistic of {groups} groups over {dim} columns")
    if resid_norm is not None:
        resid, gain, gain_offset, xs, ss_out = resid_norm
        if paired or out is not None:
            raise KernelError("gemm_packed: the product before a norm is not gated and has no output beside resid, xs and ss")
        _need(resid, "gemm_packed.resid", _F32, (M, N))
        _need(gain, "gemm_packed.gain", (_BF16, _F32), (N,))
        _need(xs, "gemm_packed.xs", _BF16, (M, N))
        _need(ss_out, "gemm_packed.ss", _F32, (M, N // 16))
        out_code = 2
    elif paired:
        _need(out, "gemm_packed.out", _BF16, (M, N // 2))
        out_code = 1
    elif out.dim() == 3:          # float partial sums over slices of K, which the reader adds
        slices = out.shape[0]
        _need(out, "gemm_packed.out", _F32, (slices, M, N))
        out_code = 2
    else:
        _need(out, "gemm_packed.out", (_BF16, _F32), (M, N))
        out_code = 2 if out.dtype == _F32 else 1
    if row_scale is None and resid_norm is None:
        _call(load_library("core"), "syn_gemm_packed", _ptr(x), _ptr(wp), _ptr(out), out_code,
              M, N, K, 1 if paired else 0, activation_code(activation), slices, _stream())
        return
    _call(load_library("core"), "syn_gemm_packed_norm", _ptr(x), _ptr(wp), _ptr(out), out_code, M, N, K,
          1 if paired else 0, activation_code(activation), slices, _ptr(ss), int(groups), int(dim), ctypes.c_float(eps),
          _ptr(resid), _ptr(xs), _ptr(ss_out), _ptr(gain), _is_f32(gain) if gain is not None else 0,
          ctypes.c_float(gain_offset), _stream())


_compute_units = None


def compute_units() -> int:
    """Compute units of the GPU that the rules below fill: asked of the device once (256 on an MI355X, which is also
    what the rules assume where no GPU is present, as in tests of the rules themselves).  The C side asks the
    device the same question (csrc/gemm.hip: compute_units)."""
    global _compute_units
    if _compute_units is None:
        _compute_units = (torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
                          if torch.cuda.is_available() else 256)
    return _compute_units


def packed_slices(N, K):
    """Into how many slices of K gemm_packed is cut when its reader can add partial sums.  It has a workgroup
    for every 16 rows of W, each with a fixed share of the weight stream; when their number is no
    multiple of the compute units the last round runs half empty (N = 5120: 320 workgroups, two rounds for
    the work of 1.25; N = 2560: 160 compute units of 256).  The smallest cut that fills its rounds to 90 %
    is taken, if one exists among up to 8 slices of at least 1,024."""
    groups, units = -(-N // 16), compute_units()

    def fill(s):
        work = groups * s / units
        return work / -(-groups * s // units)

    best = 1
    for s in (1, 2, 3, 4, 5, 6, 8):
        if s > 1 and K // s < 1024:
            break
        if fill(s) >= 0.9:
            return s
        if fill(s) > fill(best) + 0.05:
            best = s
    return best


def gemm_slices(M, N, K, dtype):
    """Into how many slices of K a product is cut when its reader can add partial sums.  A product
    with few rows of W has too few workgroups (one for every 64 rows) to pull the weights at speed.
    The cut aims at one round of workgroups over the 256 compute units; up to 32 rows of x, where the
    tiles keep three k-tiles in flight, four slices are enough (and leave the reader fewer partial
    sums to add); measured at the shapes of an 8B model (N = 4096 and 6144, K = 4096 and 12288) for
    1, 8, 32 and 64 rows."""
    if dtype != _BF16 or K % 8 != 0 or N > 16384 or K < 2048:
        return 1
    units = compute_units()
    if M > 64:
        # prompts: 256 x 256 tiles are the most efficient, but a narrow product has too few of them for
        # the 256 compute units (128 at 2,048 rows and N = 4096); two or four slices of K fill the chip,
        # at the price of partial sums of M x N floats each
        if K % 128:
            return 1
        if M <= 512:
            # short prompts: still bound by reading W; tiles of 128 rows of W (and of 128 rows of x up to 256 rows,
            # of 256 beyond), cut until they fill the compute units
            tiles = (-(-M // 128) if M <= 256 else -(-M // 256)) * -(-N // 128)
            most, slices = min(8, units // tiles, K // 512), 1
            while slices * 2 <= most:
                slices *= 2
            if slices > 1:
                return slices
        tiles = -(-M // 256) * -(-N // 256)
        return 4 if tiles * 4 <= units and K >= 8192 else (2 if tiles * 2 <= units else 1)
    if M <= 32:
        # 64 rows of W a workgroup, up to three workgroups a compute unit
        most = min(4, 3 * units // -(-N // 64), K // 512)
    else:
        # 128 rows of W a workgroup, one workgroup a compute unit
        most = min(8, units // -(-N // 128), K // 512)
    slices = 1
    while slices * 2 <= most:
        slices *= 2
    return slices


# ----------------------------------------------------------------------------- attention

def v_pages_to_kernel_order(v):
    """V pages [..., kv_heads, hd, 64] as plain (dim, token) rows -> the same shape holding each page
    in the order the bf16 kernels keep it (fragment after fragment of the decode kernel's MFMA: half of
    the tokens, 16 dims, lane group of 8 tokens, dim, token).  Float pages are plain and stay as they are."""
    if v.dtype != _BF16:
        return v
    lead, hd = v.shape[:-2], v.shape[-2]
    x = v.reshape(*lead, hd // 16, 16, 2, 4, 8)            # [dt, r, h, g, e]
    n = len(lead)
    x = x.permute(*range(n), n + 2, n + 0, n + 3, n + 1, n + 4)   # [h, dt, g, r, e]
    return x.reshape(*lead, hd, 64).contiguous()


def v_pages_from_kernel_order(v):
    """The inverse of v_pages_to_kernel_order."""
    if v.dtype != _BF16:
        return v
    lead, hd = v.shape[:-2], v.shape[-2]
    x = v.reshape(*lead, 2, hd // 16, 4, 16, 8)            # [h, dt, g, r, e]
    n = len(lead)
    x = x.permute(*range(n), n + 1, n + 3, n + 0, n + 2, n + 4)   # [dt, r, h, g, e]
    return x.reshape(*lead, hd, 64).contiguous()


def _check_pages(k_pages, v_pages, dtype, nkv, hd, name):
    _need(k_pages, name + ".k_pages", dtype, (None, nkv, PAGE_TOKENS, hd))
    _need(v_pages, name + ".v_pages", dtype, (k_pages.shape[0], nkv, hd, PAGE_TOKENS))


def qk_norm_rope_kv_write(qkv, q_out, k_pages, v_pages, page_table, tok_seq, tok_pos, q_gain, k_gain, eps,
                          cos, sin, n_heads, n_kv_heads, head_dim, write_kv=True, gain_offset=0.0):
    """qkv [N, width] in the activation type, or float partial sums [S, N, width] that are added first.
    Split a fused [q | k | v] projection row into heads; RMSNorm q and k heads (if gains are
    given; the gain is gain_offset + its tensor), rotate them at tok_pos (if tables are given; their width is rotary_dim / 2), write q to
    q_out [N, nh*hd], k and v into the cache pages of sequence tok_seq[n] at position tok_pos[n]
    (not with write_kv False: a layer that reads a cache which another layer writes)."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    n_parts = 0
    if qkv.dim() == 3:          # float partial sums [S, N, width] of a product cut along K
        n_parts = qkv.shape[0]
        _need(qkv, "qk_norm_rope_kv_write.qkv", _F32, (n_parts, None, (nh + 2 * nkv) * hd))
        N = qkv.shape[1]
        _need(q_out, "qk_norm_rope_kv_write.q_out", (_BF16, _F32), (N, nh * hd))
    else:
        _need(qkv, "qk_norm_rope_kv_write.qkv", (_BF16, _F32), (None, (nh + 2 * nkv) * hd))
        N = qkv.shape[0]
        _need(q_out, "qk_norm_rope_kv_write.q_out", qkv.dtype, (N, nh * hd))
    _check_pages(k_pages, v_pages, q_out.dtype, nkv, hd, "qk_norm_rope_kv_write")
    _need(page_table, "qk_norm_rope_kv_write.page_table", _I32, (None, None))
    _need(tok_seq, "qk_norm_rope_kv_write.tok_seq", _I32, (N,))
    _need(tok_pos, "qk_norm_rope_kv_write.tok_pos", _I32, (N,))
    if hd > MAX_HEAD_DIM:
        raise KernelError(f"qk_norm_rope_kv_write: head size {hd} exceeds {MAX_HEAD_DIM}")
    gain_f32 = 0
    if (q_gain is None) != (k_gain is None):
        raise KernelError("qk_norm_rope_kv_write: q and k gains come together")
    if q_gain is not None:
        _need(q_gain, "qk_norm_rope_kv_write.q_gain", (_BF16, _F32), (hd,))
        _need(k_gain, "qk_norm_rope_kv_write.k_gain", q_gain.dtype, (hd,))
        gain_f32 = _is_f32(q_gain)
    rot = 0
    if cos is not None:
        _need(cos, "qk_norm_rope_kv_write.cos", _F32, (None, None))
        _need(sin, "qk_norm_rope_kv_write.sin", _F32, tuple(cos.shape))
        rot = 2 * cos.shape[1]
        if rot > hd:
            raise KernelError(f"qk_norm_rope_kv_write: rotary size {rot} exceeds head size {hd}")
    _call(load_library("core"), "syn_qk_norm_rope_kv_write", _ptr(qkv), n_parts, _ptr(q_out), _ptr(k_pages), _ptr(v_pages),
          _is_f32(q_out), _ptr(page_table), page_table.shape[1], _ptr(tok_seq), _ptr(tok_pos), _ptr(q_gain), _ptr(k_gain),
          gain_f32, ctypes.c_float(gain_offset), ctypes.c_float(eps), _ptr(cos), _ptr(sin), rot, N, nh, nkv, hd,
          1 if write_kv else 0, _stream())


def _score_terms(name, slopes, softcap, n_heads):
    """The optional terms on the scores as the entry points take them: (pointer to slopes [n_heads] float or null,
    soft cap as a C float; 0 = none).  score = cap * tanh(score / cap), then - slope[head] * (query position - key
    position); see csrc/common.h: ScoreTerms."""
    if slopes is not None:
        _need(slopes, name + ".slopes", _F32, (n_heads,))
    softcap = float(softcap or 0.0)
    if softcap < 0.0:
        raise KernelError(f"{name}: a soft cap of {softcap}")
    return _ptr(slopes), ctypes.c_float(softcap)


def attention_f32(q, k_pages, v_pages, page_table, tok_seq, tok_pos, out, scale, window, n_heads, n_kv_heads,
                  head_dim, slopes=None, softcap=0.0):
    """True 32-bit attention of every token (prefill and decode alike).  slopes, softcap: see _score_terms."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    _need(q, "attention_f32.q", _F32, (None, nh * hd))
    N = q.shape[0]
    _check_pages(k_pages, v_pages, _F32, nkv, hd, "attention_f32")
    _need(page_table, "attention_f32.page_table", _I32, (None, None))
    _need(tok_seq, "attention_f32.tok_seq", _I32, (N,))
    _need(tok_pos, "attention_f32.tok_pos", _I32, (N,))
    _need(out, "attention_f32.out", _F32, (N, nh * hd))
    _call(load_library("core"), "syn_attention_f32", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
          page_table.shape[1], _ptr(tok_seq), _ptr(tok_pos), _ptr(out), ctypes.c_float(scale), int(window or 0),
          N, nh, nkv, hd, *_score_terms("attention_f32", slopes, softcap, nh), _stream())


def _attn_lib(hd):
    if hd % 16 != 0 or not (16 <= hd <= MAX_HEAD_DIM):
        raise KernelError(f"bf16 attention: head size {hd} is not one of 16, 32, ..., {MAX_HEAD_DIM}")
    return load_library(f"attn_hd{hd}")


def attention_prefill_bf16(q, k_pages, v_pages, page_table, seq_start, seq_past, out, scale, window, n_heads,
                           n_kv_heads, head_dim, variant=0, slopes=None, softcap=0.0, skip_below=0):
    """Causal attention of the new tokens of each sequence over its cache (which already holds them).
    seq_start [B+1]: offsets of the sequences' new tokens in q; seq_past [B]: tokens cached before.
    variant: 0 = the kernel's own choice, 1 = waves of 16 query rows (every head size), 2 = waves of 32
    query rows (head sizes 64 and 128); for comparisons.  slopes, softcap: see _score_terms (they take the kernel
    with waves of 16 rows).  skip_below: sequences with fewer new tokens than this are left out and their rows of
    `out` stay as they are (2: single tokens, which the caller hands to attention_decode_bf16)."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    _need(q, "attention_prefill.q", _BF16, (None, nh * hd))
    N = q.shape[0]
    _check_pages(k_pages, v_pages, _BF16, nkv, hd, "attention_prefill")
    _need(page_table, "attention_prefill.page_table", _I32, (None, None))
    _need(seq_start, "attention_prefill.seq_start", _I32, (None,))
    B = seq_start.shape[0] - 1
    _need(seq_past, "attention_prefill.seq_past", _I32, (B,))
    if page_table.shape[0] < B:
        raise KernelError(f"attention_prefill: page table has {page_table.shape[0]} rows for {B} sequences")
    _need(out, "attention_prefill.out", _BF16, (N, nh * hd))
    _call(_attn_lib(hd), "syn_attention_prefill_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
          page_table.shape[1], _ptr(seq_start), _ptr(seq_past), B, N, _ptr(out), ctypes.c_float(scale),
          int(window or 0), nh, nkv, hd, int(variant), *_score_terms("attention_prefill", slopes, softcap, nh),
          int(skip_below), _stream())


def decode_splits(n_seqs, n_kv_heads, max_pages):
    """How many ways the key blocks of a sequence are split in decode.  A workgroup has up to 8
    waves that take a block each at a time; a wave that takes several blocks one after another
    pays a trip to memory for each, so the keys are split until about 2,048 waves run, but not so
    far that a split holds fewer than four blocks.  Contexts from 6K tokens on are split further,
    up to 1,024 workgroups, while a split keeps eight blocks.  One split needs no merge.
    Measured inside a graph at 1 to 32 sequences of 512 to 32K tokens (32 heads, 8 kv heads of 128):
    8 sequences of 2,100 tokens: 4 splits 19 us, 1 split 29 us, 8 splits 23 us; one sequence: 8
    splits 10.7 us, 4 splits 12.8 us; 8 sequences of 8K tokens: 16 splits 54 us, 4 splits 60 us."""
    groups = max(1, n_seqs * n_kv_heads)
    want = -(-2048 // (groups * 8))
    splits = max(1, min(want, 1 if max_pages <= 8 else max_pages // 4, 64))
    if max_pages >= 96 and groups < 256:             # (with a workgroup for every compute unit more splits only cost merging:
        more = min(64, 1024 // groups)               # 32 sequences of 8K tokens unsplit 160 us, in 4 splits 166 us)
        if more > splits and max_pages // more >= 8:
            splits = more
    return int(splits)


def _decode_work(name, counters, items, B, n_splits, n_heads, n_kv_heads):
    """The optional arguments of the decode kernels.  counters: int32, at least B * kv heads * ceil(group / 16),
    zero (the kernel leaves them zero): with them the splits are merged inside the one launch where its grid is
    small enough for that to pay.  items: int32 [4 * B * n_splits + 2 * B], the work list that hands longer
    sequences more splits (runtime.decode_items lays it out)."""
    n_items = 0
    if items is not None:
        _need(items, f"{name}.items", _I32, (4 * B * n_splits + 2 * B,))
        n_items = B * n_splits
    if counters is not None:
        chunks = -(-(n_heads // n_kv_heads) // 16)
        _need(counters, f"{name}.counters", _I32)
        if counters.numel() < B * n_kv_heads * chunks:
            raise KernelError(f"{name}: {counters.numel()} counters for {B} sequences x {n_kv_heads * chunks}")
    return _ptr(counters), _ptr(items), n_items


def attention_decode_bf16(q, k_pages, v_pages, page_table, seq_len, out, workspace, n_splits, scale, window,
                          n_heads, n_kv_heads, head_dim, slopes=None, softcap=0.0, counters=None, items=None):
    """One query for each sequence (its last token, already in the cache); seq_len [B] counts it.
    workspace: float [B * nh * n_splits * (hd + 2)].  slopes, softcap: see _score_terms; counters,
    items: see _decode_work."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    _need(q, "attention_decode.q", _BF16, (None, nh * hd))
    B = q.shape[0]
    _check_pages(k_pages, v_pages, _BF16, nkv, hd, "attention_decode")
    _need(page_table, "attention_decode.page_table", _I32, (None, None))
    if page_table.shape[0] < B:
        raise KernelError(f"attention_decode: page table has {page_table.shape[0]} rows for {B} sequences")
    _need(seq_len, "attention_decode.seq_len", _I32, (B,))
    _need(out, "attention_decode.out", _BF16, (B, nh * hd))
    _need(workspace, "attention_decode.workspace", _F32)
    if workspace.numel() < B * nh * n_splits * (hd + 2):
        raise KernelError(f"attention_decode: workspace of {workspace.numel()} floats is too small")
    if slopes is None and not softcap and counters is None and items is None:
        _call(_attn_lib(hd), "syn_attention_decode_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
              page_table.shape[1], _ptr(seq_len), B, _ptr(out), _ptr(workspace), int(n_splits), ctypes.c_float(scale),
              int(window or 0), nh, nkv, hd, _stream())
        return
    _call(_attn_lib(hd), "syn_attention_decode_terms_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
          page_table.shape[1], _ptr(seq_len), B, _ptr(out), _ptr(workspace), int(n_splits), ctypes.c_float(scale),
          int(window or 0), nh, nkv, hd, *_score_terms("attention_decode", slopes, softcap, nh),
          *_decode_work("attention_decode", counters, items, B, n_splits, nh, nkv), _stream())


def attention_decode_fused_bf16(qkv, k_pages, v_pages, page_table, seq_len, out, workspace, n_splits, scale, window,
                                n_heads, n_kv_heads, head_dim, q_gain, k_gain, eps, cos, sin, write_kv=True,
                                gain_offset=0.0, slopes=None, softcap=0.0, counters=None, items=None):
    """attention_decode_bf16 for one new token a sequence whose q, k and v come straight from the
    fused projection: qkv [B, (nh + 2 nkv) * hd] in bf16, or float partial sums [S, B, ...] that are
    added first.  The q/k RMSNorm (if gains are given), the rotation at position seq_len - 1 (if
    tables are given) and, with write_kv, the write of the new k and v into the cache pages happen
    inside the attention kernel; seq_len [B] counts the new token.  counters, items: see _decode_work."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    width = (nh + 2 * nkv) * hd
    n_parts = 0
    if qkv.dim() == 3:
        n_parts = qkv.shape[0]
        _need(qkv, "attention_decode_fused.qkv", _F32, (n_parts, None, width))
        B = qkv.shape[1]
    else:
        _need(qkv, "attention_decode_fused.qkv", _BF16, (None, width))
        B = qkv.shape[0]
    _check_pages(k_pages, v_pages, _BF16, nkv, hd, "attention_decode_fused")
    _need(page_table, "attention_decode_fused.page_table", _I32, (None, None))
    if page_table.shape[0] < B:
        raise KernelError(f"attention_decode_fused: page table has {page_table.shape[0]} rows for {B} sequences")
    _need(seq_len, "attention_decode_fused.seq_len", _I32, (B,))
    _need(out, "attention_decode_fused.out", _BF16, (B, nh * hd))
    _need(workspace, "attention_decode_fused.workspace", _F32)
    if workspace.numel() < B * nh * n_splits * (hd + 2):
        raise KernelError(f"attention_decode_fused: workspace of {workspace.numel()} floats is too small")
    gain_f32 = 0
    if (q_gain is None) != (k_gain is None):
        raise KernelError("attention_decode_fused: q and k gains come together")
    if q_gain is not None:
        _need(q_gain, "attention_decode_fused.q_gain", (_BF16, _F32), (hd,))
        _need(k_gain, "attention_decode_fused.k_gain", q_gain.dtype, (hd,))
        gain_f32 = _is_f32(q_gain)
    rot = 0
    if cos is not None:
        _need(cos, "attention_decode_fused.cos", _F32, (None, None))
        _need(sin, "attention_decode_fused.sin", _F32, tuple(cos.shape))
        rot = 2 * cos.shape[1]
        if rot > hd:
            raise KernelError(f"attention_decode_fused: rotary size {rot} exceeds head size {hd}")
    _call(_attn_lib(hd), "syn_attention_decode_fused_bf16", _ptr(qkv), n_parts, _ptr(k_pages), _ptr(v_pages),
          _ptr(page_table), page_table.shape[1], _ptr(seq_len), B, _ptr(out), _ptr(workspace), int(n_splits),
          ctypes.c_float(scale), int(window or 0), nh, nkv, hd, _ptr(q_gain), _ptr(k_gain), gain_f32,
          ctypes.c_float(gain_offset), ctypes.c_float(eps), _ptr(cos), _ptr(sin), rot, 1 if write_kv else 0,
          *_score_terms("attention_decode_fused", slopes, softcap, nh),
          *_decode_work("attention_decode_fused", counters, items, B, n_splits, nh, nkv), _stream())


# ----------------------------------------------------------------------------- sampling

def sample_rows(logits, temperature, uniform, out):
    """out[r] = argmax (last of equal maxima) where temperature[r] <= 0 or temperature is None,
    else a draw from softmax(logits[r] / temperature[r]) by inverse CDF with uniform[r]."""
    _need(logits, "sample_rows.logits", _F32, (None, None))
    R, V = logits.shape
    if temperature is not None:
        _need(temperature, "sample_rows.temperature", _F32, (R,))
        _need(uniform, "sample_rows.uniform", _F32, (R,))
    _need(out, "sample_rows.out", _I32, (R,))
    _call(load_library("core"), "syn_sample_rows", _ptr(logits), _ptr(temperature),
          _ptr(uniform if temperature is not None else None), _ptr(out), R, V, _stream())


def filter_rows(logits, out, temperature, top_k, top_p, min_p, repetition, presence, frequency,
                ids=None, id_start=None, counts=None):
    """The processors in front of the sampler, one workgroup a row of logits [R, V] (float): repetition penalty,
    presence / frequency penalty, temperature, top-k, top-p, min-p, in this order; what is dropped becomes -inf
    in `out` (which may be `logits`).  Every option is an array with one entry a row: temperature (<= 0 or 1:
    the row is not divided), top_k (int32; 0: off), top_p (>= 1: off), min_p (0: off), repetition (1: off),
    presence, frequency (0: off).  ids (int32, flat) and id_start (int32 [R + 1]) give each row the tokens that
    the penalties look at; counts (int32 [R * V], zero) is their scratch memory, left zero."""
    _need(logits, "filter_rows.logits", _F32, (None, None))
    R, V = logits.shape
    _need(out, "filter_rows.out", _F32, (R, V))
    for name, t, dt in (("temperature", temperature, _F32), ("top_k", top_k, _I32), ("top_p", top_p, _F32),
                        ("min_p", min_p, _F32), ("repetition", repetition, _F32), ("presence", presence, _F32),
                        ("frequency", frequency, _F32)):
        _need(t, f"filter_rows.{name}", dt, (R,))
    if (ids is None) != (id_start is None):
        raise KernelError("filter_rows: ids and id_start come together")
    if ids is not None:
        _need(ids, "filter_rows.ids", _I32, (None,))
        _need(id_start, "filter_rows.id_start", _I32, (R + 1,))
        _need(counts, "filter_rows.counts", _I32)
        if counts.numel() < R * V:
            raise KernelError(f"filter_rows: {counts.numel()} counters for {R} rows of {V}")
    _call(load_library("core"), "syn_filter_rows", _ptr(logits), _ptr(out), R, V, _ptr(temperature), _ptr(top_k),
          _ptr(top_p), _ptr(min_p), _ptr(repetition), _ptr(presence), _ptr(frequency), _ptr(ids), _ptr(id_start),
          _ptr(counts), _stream())


# ----------------------------------------------------------------------------- what the machine gives

def measure_ceilings(device="cuda:0", read_bytes=1 << 30, repeats=5):
    """(memory read rate in GB/s, bf16 MFMA rate in TFLOP/s) of kernels that do nothing else: the
    best of `repeats` passes over a buffer of read_bytes, and of a launch that keeps every matrix
    unit busy from registers.  Measurements, to stand beside the vendor's peaks."""
    lib = load_library("core")
    buf = torch.empty(read_bytes // 4, dtype=torch.int32, device=device).zero_()
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    fsink = torch.zeros(4, dtype=torch.float32, device=device)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best(launch):
        launch()
        torch.cuda.synchronize()
        times = []
        for _ in range(repeats):
            start.record()
            launch()
            end.record()
            end.synchronize()
            times.append(start.elapsed_time(end) * 1e-3)
        return min(times)

    t_read = best(lambda: _call(lib, "syn_probe_read", _ptr(buf), ctypes.c_size_t(buf.numel() * 4), _ptr(sink), _stream()))
    groups, iters = 256 * 8, 4096
    t_mfma = best(lambda: _call(lib, "syn_probe_mfma", groups, iters, _ptr(fsink), _stream()))
    flops = groups * 4 * iters * 4 * 2 * 32 * 32 * 16
    return buf.numel() * 4 / t_read / 1e9, flops / t_mfma / 1e12
