"""Each HIP kernel alone against a plain torch float32 statement of the same operation
(tests/cpu_kernels.py), at sizes other than the engine's test models use, with sizes that are
no multiple of any tile.  Tolerances follow the reference's ladder for its CUDA kernels
(crates/synaptix-kernels-cuda/tests/*: float32 1e-5 .. 1e-4, bf16 around 1e-2 on O(1) data)."""
import math

import pytest
import torch

import cpu_kernels as ref
from synaptix_amd.kernels import runtime as rt

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from synaptix_amd.kernels import ops as o
    return o


def rnd(shape, seed, dtype=F32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def close(got, want, atol, rtol=0.0, what=""):
    got, want = got.detach().cpu().to(F32), want.detach().cpu().to(F32)
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    bad = err > bound
    assert not bad.any(), f"{what}: max abs err {err.max():.3e} (allowed {atol:.1e} + {rtol:.1e}|x|), {int(bad.sum())} values off"


# ----------------------------------------------------------------------------- rows

@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("V,H,N", [(100, 24, 7), (1000, 4100, 3)])
def test_embed(ops, dtype, V, H, N):
    table = rnd((V, H), 1, dtype)
    ids = torch.tensor([(i * 37 + V - 1) % V for i in range(N)], dtype=I32)
    out = torch.empty((N, H), dtype=F32, device=DEV)
    ops.embed(table.to(DEV), ids.to(DEV), out)
    assert torch.equal(out.cpu(), table[ids.long()].to(F32))  # a copy: exact


@pytest.mark.parametrize("out_dtype,gain_dtype", [(F32, F32), (BF16, BF16), (BF16, F32)])
@pytest.mark.parametrize("N,H", [(5, 72), (3, 4096), (2, 5000)])
def test_add_rmsnorm(ops, out_dtype, gain_dtype, N, H):
    eps = 1e-5
    resid, delta = rnd((N, H), 2), rnd((N, H), 3)
    gain = (1 + 0.1 * rnd((H,), 4)).to(gain_dtype)
    want_resid = resid.clone()
    want = torch.empty((N, H), dtype=out_dtype)
    ref.add_rmsnorm(want_resid, delta, gain, eps, want)
    r = resid.to(DEV)
    out = torch.empty((N, H), dtype=out_dtype, device=DEV)
    ops.add_rmsnorm(r, delta.to(DEV), gain.to(DEV), eps, out)
    close(r, want_resid, 1e-6, what="residual sum")
    close(out, want, 1e-5 if out_dtype == F32 else 2e-2, 1e-5 if out_dtype == F32 else 1e-2, "normed")
    # without a delta the residual stays; with rows only those rows are normed and nothing is written
    r2 = resid.to(DEV)
    ops.add_rmsnorm(r2, None, gain.to(DEV), eps, out)
    assert torch.equal(r2.cpu(), resid)
    rows = torch.tensor([N - 1, 0], dtype=I32)
    out2 = torch.empty((2, H), dtype=out_dtype, device=DEV)
    want2 = torch.empty((2, H), dtype=out_dtype)
    ref.add_rmsnorm(resid.clone(), delta, gain, eps, want2, rows)
    ops.add_rmsnorm(r2, delta.to(DEV), gain.to(DEV), eps, out2, rows.to(DEV))
    assert torch.equal(r2.cpu(), resid)
    close(out2, want2, 1e-5 if out_dtype == F32 else 2e-2, 1e-5 if out_dtype == F32 else 1e-2, "gathered rows")


def test_norm_gains_stored_as_a_difference_from_one(ops):
    """gain_offset = 1: the gain is 1 + w in every kernel that norms (rows with the residual sum, rows of any
    width, the q/k heads of prompts in both of their kernels, the q/k heads inside decode attention)."""
    eps = 1e-5
    for H, dt in ((72, F32), (4096, BF16)):
        resid, delta = rnd((3, H), 2), rnd((3, H), 3)
        w = (0.1 * rnd((H,), 4)).to(dt)
        want = torch.empty((3, H), dtype=F32)
        ref.add_rmsnorm(resid.clone(), delta, 1 + w.float(), eps, want)
        got = torch.empty((3, H), dtype=F32, device=DEV)
        ops.add_rmsnorm(resid.to(DEV), delta.to(DEV), w.to(DEV), eps, got, gain_offset=1.0)
        close(got, want, 1e-5, 1e-5, "add_rmsnorm with 1 + w")
        x = rnd((5, H), 5)
        ref.rmsnorm_rows(x, 1 + w.float(), eps, want2 := torch.empty((5, H)))
        got2 = torch.empty((5, H), dtype=F32, device=DEV)
        ops.rmsnorm_rows(x.to(DEV), w.to(DEV), eps, got2, gain_offset=1.0)
        close(got2, want2, 1e-5, 1e-5, "rmsnorm_rows with 1 + w")
    # q/k heads: head size 128 takes the 16-byte kernel, 48 the general one
    for nh, nkv, hd in ((4, 2, 128), (6, 2, 48)):
        N, width = 5, (nh + 2 * nkv) * hd
        table = torch.arange(2, dtype=I32).view(1, 2)
        tok_seq, tok_pos = torch.zeros(N, dtype=I32), torch.arange(60, 60 + N, dtype=I32)
        qkv = rnd((N, width), 6, BF16)
        qg, kg = (0.2 * rnd((hd,), 7)).to(BF16), (0.2 * rnd((hd,), 8)).to(BF16)
        ang = torch.arange(80, dtype=F32)[:, None] * (0.3 / (1 + torch.arange(hd // 2, dtype=F32)))[None, :]
        cos, sin = torch.cos(ang), torch.sin(ang)
        k_ref, v_ref = torch.zeros((2, nkv, 64, hd), dtype=BF16), torch.zeros((2, nkv, hd, 64), dtype=BF16)
        q_ref = torch.empty((N, nh * hd), dtype=BF16)
        ref.qk_norm_rope_kv_write(qkv, q_ref, k_ref, v_ref, table, tok_seq, tok_pos, (1 + qg.float()), (1 + kg.float()),
                                  eps, cos, sin, nh, nkv, hd)
        d = lambda t: t.to(DEV)
        kd, vd = torch.zeros_like(k_ref).to(DEV), dv(torch.zeros_like(v_ref))
        q = torch.empty((N, nh * hd), dtype=BF16, device=DEV)
        ops.qk_norm_rope_kv_write(d(qkv), q, kd, vd, d(table), d(tok_seq), d(tok_pos), d(qg), d(kg), eps, d(cos), d(sin),
                                  nh, nkv, hd, gain_offset=1.0)
        close(q, q_ref.float(), 2e-2, 1e-2, f"q heads of size {hd} with 1 + w")
        close(kd, k_ref.float(), 2e-2, 1e-2, f"k heads of size {hd} with 1 + w")
        # one more token through decode attention with the q/k/v intake
        one = rnd((1, width), 9, BF16)
        seq_len = torch.tensor([66], dtype=I32)
        q1 = torch.empty((1, nh * hd), dtype=BF16)
        ref.qk_norm_rope_kv_write(one, q1, k_ref, v_ref, table, torch.zeros(1, dtype=I32), seq_len - 1, 1 + qg.float(),
                                  1 + kg.float(), eps, cos, sin, nh, nkv, hd)
        want = torch.empty((1, nh * hd), dtype=F32)
        ref.attention_f32(q1.float(), k_ref.float(), v_ref.float(), table, torch.zeros(1, dtype=I32), seq_len - 1, want,
                          0.1, 0, nh, nkv, hd)
        # positions 0..59 of the pages hold zeros: they take part in the softmax on both sides alike
        out = torch.empty((1, nh * hd), dtype=BF16, device=DEV)
        work = torch.empty(nh * 2 * (hd + 2), dtype=F32, device=DEV)
        ops.attention_decode_fused_bf16(d(one), kd, vd, d(table), d(seq_len), out, work, 2, 0.1, 0, nh, nkv, hd, d(qg),
                                        d(kg), eps, d(cos), d(sin), gain_offset=1.0)
        close(out, want, 2e-2, 1e-2, f"decode attention, head size {hd}, gains 1 + w")


def test_an_unknown_activation_is_refused_before_any_launch(ops):
    x = torch.zeros((2, 64), dtype=BF16, device=DEV)
    out = torch.zeros((2, 32), dtype=BF16, device=DEV)
    with pytest.raises(Exception, match="activation 'gelu'"):
        ops.swiglu(x, out, "gelu")
    with pytest.raises(Exception, match="activation 'relu'"):
        ops.gemm_swiglu(x, torch.zeros((64, 64), dtype=BF16, device=DEV), out, "relu")
    from synaptix_amd.kernels.build import load_library
    lib = load_library("core")
    assert lib.syn_swiglu(None, None, 0, 2, 32, 7, None) != 0 and b"activation code 7" in lib.syn_last_error()


def test_rmsnorm_eps_sits_inside_the_root(ops):
    # tiny x: sqrt(mean + eps) and sqrt(mean) + eps differ by orders of magnitude
    x = torch.full((1, 64), 1e-4)
    gain = torch.ones(64)
    out = torch.empty((1, 64), device=DEV)
    ops.rmsnorm_rows(x.to(DEV), gain.to(DEV), 1e-6, out)
    want = 1e-4 / math.sqrt(1e-8 + 1e-6)
    close(out, torch.full((1, 64), want), 1e-6, what="eps inside the root")


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("R,D", [(9, 16), (5, 80), (3, 200)])
def test_rmsnorm_rows(ops, dtype, R, D):
    x, gain = rnd((R, D), 5, dtype), (1 + 0.1 * rnd((D,), 6)).to(dtype)
    want = torch.empty_like(x)
    ref.rmsnorm_rows(x, gain, 1e-6, want)
    out = torch.empty((R, D), dtype=dtype, device=DEV)
    ops.rmsnorm_rows(x.to(DEV), gain.to(DEV), 1e-6, out)
    close(out, want, 1e-5 if dtype == F32 else 2e-2, 0 if dtype == F32 else 1e-2)


def test_rmsnorm_reference_vector(ops):
    """The vector of crates/synaptix-ops/tests/rms_norm.rs:76-95, against the float64 closed form."""
    x = torch.tensor([i * 0.1 - 1.0 for i in range(24)], dtype=F32).view(6, 4)
    w = torch.tensor([0.5, -0.25, 1.0, 2.0])
    out = torch.empty((6, 4), device=DEV)
    ops.rmsnorm_rows(x.to(DEV), w.to(DEV), 1e-6, out)
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * w.double()
    close(out, want.float(), 1e-5)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_swiglu(ops, dtype):
    N, I = 7, 176
    gu = rnd((N, 2 * I), 7, dtype, 2.0)
    want = torch.empty((N, I), dtype=dtype)
    ref.swiglu(gu, want)
    out = torch.empty((N, I), dtype=dtype, device=DEV)
    ops.swiglu(gu.to(DEV), out)
    close(out, want, 5e-6 if dtype == F32 else 1.5e-2, 0 if dtype == F32 else 1e-2)
    # swapping gate and up must change the result (a swapped fused layout would not be seen otherwise)
    swapped = torch.cat([gu[:, I:], gu[:, :I]], 1).contiguous()
    out2 = torch.empty((N, I), dtype=dtype, device=DEV)
    ops.swiglu(swapped.to(DEV), out2)
    assert (out2.cpu().float() - want.float()).abs().max() > 0.1


# ----------------------------------------------------------------------------- matrix product

@pytest.mark.parametrize("M,N,K", [(1, 33, 40), (7, 100, 72), (64, 64, 64), (65, 130, 100), (200, 70, 300)])
def test_gemm_f32(ops, M, N, K):
    x, w = rnd((M, K), 8), rnd((N, K), 9)
    out = torch.empty((M, N), device=DEV)
    ops.gemm(x.to(DEV), w.to(DEV), out)
    want = (x.double() @ w.double().T).float()
    close(out, want, 1e-4, 1e-5, f"gemm f32 {M}x{N}x{K}")


@pytest.mark.parametrize("out_dtype", [BF16, F32])
@pytest.mark.parametrize("M,N,K", [
    (1, 48, 64), (3, 1000, 176), (16, 100, 320), (17, 40, 72), (33, 1000, 128), (48, 70, 2048), (64, 4096, 512),
    (65, 130, 104), (128, 128, 32), (200, 300, 1000), (513, 257, 4096),
    (1700, 5120, 128),                  # the 256 x 160 tile: 32 tiles along N where 256 x 192 makes 27
    (5, 30, 20), (70, 50, 36),          # K no multiple of 8: the plain kernel takes them
    (2048, 6144, 512), (1000, 12300, 136),   # large enough for the 256 x 256 tiles with 8 waves, ragged edges
    (1000, 12544, 128), (300, 200, 64),   # K a multiple of 64: loads straight into LDS, every tile shape
    (8, 40000, 256), (40, 33000, 72), (64, 50000, 1000),   # wide
    (1, 9000, 520), (1, 70000, 136),                       # one row: W straight from memory, K over the waves
    (8, 70000, 264), (20, 66000, 72),                      # few rows, very wide: 32-row tiles, 256 deep
    (100, 300, 1024), (256, 520, 256), (129, 4096, 384), (255, 6144, 128),   # short prompts, narrow: 64-row tiles, several of them along M
])
def test_gemm_bf16(ops, out_dtype, M, N, K):
    x, w = rnd((M, K), 10, BF16), rnd((N, K), 11, BF16)
    out = torch.empty((M, N), dtype=out_dtype, device=DEV)
    ops.gemm(x.to(DEV), w.to(DEV), out)
    want = (x.double() @ w.double().T).float()
    # float accumulation of exact bf16 products: the only error is the order of the sum and the last rounding
    atol = 1e-3 * math.sqrt(K)
    close(out, want, atol if out_dtype == F32 else atol + 0.02, 0 if out_dtype == F32 else 1e-2, f"gemm bf16 {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K,S", [(1, 48, 4096, 4), (8, 4096, 4096, 4), (8, 100, 1000, 3), (16, 64, 12288, 8),
                                     (40, 70, 2048, 2), (64, 130, 520, 5), (8, 96, 1536, 5), (50, 200, 3072, 7),
                                     (300, 520, 1024, 2), (130, 260, 640, 3), (65, 33, 4096, 4),
                                     (200, 4096, 1024, 2), (256, 1000, 2048, 4),
                                     # short prompts cut along K: tiles of 128 x 128 up to 256 rows, of 256 x 128 beyond
                                     (66, 6144, 4096, 4), (128, 200, 4096, 8), (129, 4100, 1024, 2), (256, 1000, 2560, 4),
                                     (257, 520, 4096, 8), (400, 2000, 1152, 2), (512, 4096, 1024, 2)])
def test_gemm_bf16_partial_sums_over_slices_of_k(ops, M, N, K, S):
    """[S, M, N]: slice s holds the sum over its part of K; the slices add up to the product, also
    when K is no multiple of the slice and the last slices are short or empty."""
    x, w = rnd((M, K), 14, BF16), rnd((N, K), 15, BF16)
    out = torch.full((S, M, N), float("nan"), dtype=F32, device=DEV)
    ops.gemm(x.to(DEV), w.to(DEV), out)
    want = (x.double() @ w.double().T).float()
    close(out.sum(0), want, 1e-3 * math.sqrt(K), what=f"sum of {S} slices")
    step = ((K + S - 1) // S + 127) // 128 * 128
    first = (x[:, :step].double() @ w[:, :step].double().T).float()
    close(out[0], first, 1e-3 * math.sqrt(step), what="first slice")
    # the consumer adds the slices: resid + sum(delta) normed
    H = N
    resid = rnd((M, H), 16)
    gain = (1 + 0.1 * rnd((H,), 17)).to(BF16)
    r = resid.to(DEV)
    normed = torch.empty((M, H), dtype=BF16, device=DEV)
    ops.add_rmsnorm(r, out, gain.to(DEV), 1e-6, normed)
    want_resid = resid + out.sum(0).cpu()
    close(r, want_resid, 1e-4, 1e-5, "residual + slices")
    want_n = torch.empty((M, H), dtype=BF16)
    ref.add_rmsnorm(want_resid.clone(), None, gain, 1e-6, want_n)
    close(normed, want_n, 2e-2, 1e-2, "norm of residual + slices")
    rows = torch.tensor([M - 1, 0], dtype=I32)
    got2 = torch.empty((2, H), dtype=F32, device=DEV)
    ops.add_rmsnorm(resid.to(DEV), out, gain.to(DEV), 1e-6, got2, rows.to(DEV))
    want2 = torch.empty((2, H), dtype=F32)
    ref.add_rmsnorm(resid.clone(), out.cpu(), gain, 1e-6, want2, rows)
    close(got2, want2, 1e-4, 1e-4, "gathered rows of residual + slices")


@pytest.mark.parametrize("M,I,K", [(1, 48, 64), (1, 2560, 4096), (1, 1008, 1096), (8, 2560, 4096), (7, 112, 1000), (33, 80, 136), (64, 1024, 512),
                                   (300, 400, 264), (2048, 3072, 256), (1000, 6272, 136), (8, 32784, 72),
                                   (1000, 6272, 128), (300, 400, 192),
                                   # 65 to 256 rows: all of x in one tile of 128, 192 or 256 rows and 96 or 128 rows of W
                                   (65, 48, 64), (100, 1040, 448), (128, 12288, 512), (129, 400, 192), (192, 2000, 320),
                                   (193, 80, 1024), (256, 4864, 640), (200, 400, 72), (1700, 2560, 192)])
def test_gemm_with_the_gated_activation_inside(ops, M, I, K):
    """silu(x . Wg^T) * (x . Wu^T) from one product over the rows of Wg and Wu in turns of 16,
    against the two products and the activation in 64-bit; every tile shape of the kernel."""
    x, wg, wu = rnd((M, K), 18, BF16), rnd((I, K), 19, BF16), rnd((I, K), 20, BF16)
    paired = ops.pair_rows(wg.to(DEV), wu.to(DEV))
    assert paired.shape == (2 * I, K)
    assert torch.equal(paired[16:32].cpu(), wu[:16]) and torch.equal(paired[32:48].cpu(), wg[16:32])
    out = torch.full((M, I), float("nan"), dtype=BF16, device=DEV)
    ops.gemm_swiglu(x.to(DEV), paired, out)
    g, u = x.double() @ wg.double().T, x.double() @ wu.double().T
    want = (g / (1 + torch.exp(-g)) * u).float()
    # products of standard deviation sqrt(K); one bf16 rounding of the result
    close(out, want, 2e-3 * K + 0.02, 1e-2, f"gated product {M}x{I}x{K}")
    with pytest.raises(Exception, match="turns of 16"):
        ops.pair_rows(wg[:24].to(DEV), wu[:24].to(DEV))
    with pytest.raises(Exception, match="paired rows"):
        ops.gemm_swiglu(x.to(DEV), paired[:48], torch.empty((M, 24), dtype=BF16, device=DEV))


@pytest.mark.parametrize("out_dtype", [BF16, F32])
@pytest.mark.parametrize("M,N,K", [(1, 16, 32), (1, 4096, 4096), (8, 6144, 4096), (3, 48, 96), (5, 1008, 1120), (8, 16400, 160),
                                   (16, 64, 12288), (7, 80, 2080),
                                   (8, 32784, 96), (5, 40000, 4096), (13, 32784, 96)])   # very wide from 5 rows on: two groups of rows a wave, an odd number of groups
def test_gemm_over_weights_in_fragment_order(ops, out_dtype, M, N, K):
    """The products for few rows over pack_weight(W): every k-step and every row tile lands where the
    plain product has it, also where K is no multiple of the waves' turns and N of the workgroup's rows."""
    x, w = rnd((M, K), 26, BF16), rnd((N, K), 27, BF16)
    wp = ops.pack_weight(w.to(DEV))
    assert wp.shape == (N // 16, K // 32, 64, 8)
    assert torch.equal(ops.unpack_weight(wp).cpu(), w)
    # lane = 16 * (k % 32 // 8) + n % 16, element k % 8
    assert wp[N // 16 - 1, K // 32 - 1, 16 * 2 + 5, 3] == w[N - 16 + 5, K - 32 + 2 * 8 + 3]
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
    ops.gemm_packed(x.to(DEV), wp, out)
    want = (x.double() @ w.double().T).float()
    atol = 1e-3 * math.sqrt(K)
    close(out, want, atol if out_dtype == F32 else atol + 0.02, 0 if out_dtype == F32 else 1e-2, f"packed {M}x{N}x{K}")
    if out_dtype == F32:
        # partial sums over slices of K: each slice its own part, the slices add up, also when the last ones are short or empty
        for S in (2, 3, 7):
            parts = torch.full((S, M, N), float("nan"), dtype=F32, device=DEV)
            ops.gemm_packed(x.to(DEV), wp, parts)
            close(parts.sum(0), want, atol, what=f"packed {M}x{N}x{K} in {S} slices")
            step = -(-(K // 32) // S) * 32
            first = (x[:, :step].double() @ w[:, :step].double().T).float()
            close(parts[0], first, atol, what=f"first of {S} slices")
    assert ops.pack_weight(w[:N - 3].to(DEV)) is None and ops.pack_weight(w[:, :K - 8].to(DEV)) is None
    with pytest.raises(Exception, match="at most 16"):
        ops.gemm_packed(torch.zeros((17, K), dtype=BF16, device=DEV), wp, torch.empty((17, N), dtype=out_dtype, device=DEV))


@pytest.mark.parametrize("M,I,K", [(1, 16, 32), (1, 2560, 4096), (8, 2560, 4096), (7, 112, 992), (4, 16400, 64),
                                   (9, 2560, 4096), (13, 48, 992), (16, 12288, 512)])       # up to 16 rows: the engine's limit for this product
def test_gated_product_over_weights_in_fragment_order(ops, M, I, K):
    x, wg, wu = rnd((M, K), 28, BF16), rnd((I, K), 29, BF16), rnd((I, K), 30, BF16)
    wp = ops.pack_weight(ops.pair_rows(wg.to(DEV), wu.to(DEV)))
    out = torch.full((M, I), float("nan"), dtype=BF16, device=DEV)
    ops.gemm_packed(x.to(DEV), wp, out, paired=True)
    g, u = x.double() @ wg.double().T, x.double() @ wu.double().T
    want = (g / (1 + torch.exp(-g)) * u).float()
    close(out, want, 2e-3 * K + 0.02, 1e-2, f"packed gated product {M}x{I}x{K}")


@pytest.mark.parametrize("gain_dtype,gain_offset", [(BF16, 0.0), (F32, 1.0)])
@pytest.mark.parametrize("M,H,K,N2", [(1, 64, 96, 48), (8, 4096, 4096, 6144), (5, 224, 1120, 80), (8, 4096, 12288, 24576),
                                      (3, 10240, 64, 32), (16, 96, 32, 16400)])
def test_norm_carried_between_two_products_over_packed_weights(ops, gain_dtype, gain_offset, M, H, K, N2):
    """The two halves of an RMSNorm between two products for few rows.  First half, as the epilogue of the product
    before it: resid += x . W^T, xs = gain * resid, ss = sums of resid^2 over groups of 16 columns.  Second half, as
    the epilogue of the product after it: sums of row m times rsqrt(sum(ss[m]) / H + eps), plain, gated, and in
    slices of K.  Together they equal the product over the normed rows."""
    eps = 1e-5
    x, w = rnd((M, K), 41, BF16), rnd((H, K), 42, BF16, 0.05)
    resid0 = rnd((M, H), 43)
    resid0[0] *= 30.0                    # rows of unequal size: a factor applied to the wrong row would show
    gain = (1 + 0.2 * rnd((H,), 44) - gain_offset).to(gain_dtype)
    wp = ops.pack_weight(w.to(DEV))
    resid = resid0.to(DEV)
    xs = torch.full((M, H), float("nan"), dtype=BF16, device=DEV)
    ss = torch.full((M, H // 16), float("nan"), dtype=F32, device=DEV)
    ops.gemm_packed(x.to(DEV), wp, None, resid_norm=(resid, gain.to(DEV), gain_offset, xs, ss))
    r = resid0.double() + x.double() @ w.double().T
    close(resid, r.float(), 1e-3 * math.sqrt(K) * 0.05 + 1e-5, 1e-6, "residual rows")
    r32 = resid.cpu()                    # what the kernel kept: the rest is computed from it
    g_all = gain_offset + gain.double()
    close(xs, (g_all * r32.double()).float(), 1e-6, 2 ** -8, "rows with the gain")
    close(ss, (r32.double() ** 2).view(M, H // 16, 16).sum(2).float(), 1e-6, 1e-5, "row statistic in groups")
    inv = torch.rsqrt((r32.double() ** 2).sum(1) / H + eps)[:, None]
    xs64 = xs.cpu().double()
    scale = (ss, H, eps)
    # plain product after the norm, bf16 and float, and in slices
    w2 = rnd((N2, H), 45, BF16, 0.05)
    wp2 = ops.pack_weight(w2.to(DEV))
    want = ((xs64 @ w2.double().T) * inv).float()
    atol = 2e-3 * float(want.abs().max()) + 1e-6
    out = torch.full((M, N2), float("nan"), dtype=F32, device=DEV)
    ops.gemm_packed(xs, wp2, out, row_scale=scale)
    close(out, want, atol, 1e-5, "product after the norm")
    parts = torch.full((3, M, N2), float("nan"), dtype=F32, device=DEV)
    ops.gemm_packed(xs, wp2, parts, row_scale=scale)
    close(parts.sum(0), want, atol, 1e-5, "product after the norm in slices")
    outb = torch.full((M, N2), float("nan"), dtype=BF16, device=DEV)
    ops.gemm_packed(xs, wp2, outb, row_scale=scale)
    close(outb, want, atol, 2 ** -7, "product after the norm, bf16")
    # it equals the product over the normed rows up to the rounding of those rows
    normed = (g_all * r32.double() * inv).to(BF16)
    direct = (normed.double() @ w2.double().T).float()
    assert float((want - direct).abs().max()) <= 0.02 * float(direct.abs().max()) + 1e-6
    # gated product after the norm
    if N2 % 32 == 0:
        I = N2 // 2
        wg, wu = w2[:I], w2[I:]
        wpg = ops.pack_weight(ops.pair_rows(wg.to(DEV), wu.to(DEV)))
        outg = torch.full((M, I), float("nan"), dtype=BF16, device=DEV)
        ops.gemm_packed(xs, wpg, outg, paired=True, row_scale=scale)
        gg, uu = (xs64 @ wg.double().T) * inv, (xs64 @ wu.double().T) * inv
        wantg = (gg / (1 + torch.exp(-gg)) * uu).float()
        close(outg, wantg, 2e-3 * float(wantg.abs().max()) + 1e-6, 2 ** -7, "gated product after the norm")
    with pytest.raises(Exception, match="not gated"):
        ops.gemm_packed(x.to(DEV), wp, xs, resid_norm=(resid, gain.to(DEV), gain_offset, xs, ss))


def _sampled(M, N, n, seed):
    g = torch.Generator().manual_seed(seed)
    rows = torch.cat([torch.tensor([0, M - 1, 0, M - 1]), torch.randint(0, M, (n,), generator=g)])
    cols = torch.cat([torch.tensor([0, 0, N - 1, N - 1]), torch.randint(0, N, (n,), generator=g)])
    return rows, cols


def test_products_of_a_prompt_at_the_sizes_of_an_8b_layer(ops):
    """The large-tile products at full size: 2,048 rows through gate+up with the activation inside
    (24,576 paired rows, K = 4096), and through down_proj (N = 4096, K = 12288) in the two slices
    of K that the engine asks for; some hundred sampled outputs, the corners among them, against
    64-bit dot products."""
    M, H, I = 2048, 4096, 12288
    x = rnd((M, H), 70, BF16)
    wg, wu = rnd((I, H), 71, BF16, 0.02), rnd((I, H), 72, BF16, 0.02)
    out = torch.full((M, I), float("nan"), dtype=BF16, device=DEV)
    ops.gemm_swiglu(x.to(DEV), ops.pair_rows(wg.to(DEV), wu.to(DEV)), out)
    rows, cols = _sampled(M, I, 400, 73)
    g = (x[rows].double() * wg[cols].double()).sum(1)
    u = (x[rows].double() * wu[cols].double()).sum(1)
    want = (g / (1 + torch.exp(-g)) * u).float()
    assert torch.isfinite(out).all()
    close(out[rows.to(DEV), cols.to(DEV)], want, 0.02, 1e-2, "gate+up at 8B sizes")
    del wg, wu
    assert ops.gemm_slices(M, H, I, BF16) == 2
    m = rnd((M, I), 74, BF16)
    wd = rnd((H, I), 75, BF16, 0.02)
    parts = torch.full((2, M, H), float("nan"), dtype=F32, device=DEV)
    ops.gemm(m.to(DEV), wd.to(DEV), parts)
    rows, cols = _sampled(M, H, 400, 76)
    want = (m[rows].double() * wd[cols].double()).sum(1).float()
    assert torch.isfinite(parts).all()
    close(parts.sum(0)[rows.to(DEV), cols.to(DEV)], want, 2e-3, 1e-4, "down_proj at 8B sizes, two slices")
    first = (m[rows, :I // 2].double() * wd[cols, :I // 2].double()).sum(1).float()
    close(parts[0][rows.to(DEV), cols.to(DEV)], first, 2e-3, 1e-4, "its first slice")
    # and the plain large product, bf16 out (q/k/v of a prompt: N = 6144)
    wq = rnd((6144, H), 77, BF16, 0.02)
    q = torch.full((M, 6144), float("nan"), dtype=BF16, device=DEV)
    ops.gemm(x.to(DEV), wq.to(DEV), q)
    rows, cols = _sampled(M, 6144, 400, 78)
    want = (x[rows].double() * wq[cols].double()).sum(1).float()
    close(q[rows.to(DEV), cols.to(DEV)], want, 0.02, 1e-2, "q/k/v at 8B sizes")


def test_slices_fill_the_compute_units(ops):
    """The host-side rule for the products over packed weights: one slice where the workgroups fill their
    rounds, more where they would leave the last round half empty."""
    assert ops.packed_slices(4096, 4096) == 1 and ops.packed_slices(151936, 4096) == 1
    assert ops.packed_slices(5120, 25600) == 3 and ops.packed_slices(6144, 4096) == 2
    assert ops.packed_slices(2560, 4096) == 3
    assert ops.packed_slices(2560, 1024) == 1          # no slice shorter than 1,024
    for N in range(16, 12000, 16):
        s = ops.packed_slices(N, 8192)
        assert 1 <= s <= 8


@pytest.mark.parametrize("M,N,K,S", [
    (9, 48, 128, 1), (16, 4096, 4096, 1), (33, 208, 256, 1), (64, 6144, 4096, 1), (64, 144, 384, 3),
    (100, 4112, 384, 1), (128, 208, 4096, 8), (130, 6144, 1024, 1), (200, 4096, 1024, 2), (256, 1008, 2560, 4),
    (257, 528, 4096, 8), (300, 96, 128, 1), (512, 4096, 1024, 2), (700, 272, 640, 1),
    (1700, 5120, 128, 1),               # the 256 x 160 tile
    (2053, 528, 256, 1), (1000, 12304, 128, 1), (2048, 6144, 512, 1),   # the large tiles, ragged edges
    (8, 70000 // 16 * 16, 256, 1), (20, 66000 // 16 * 16, 128, 1),      # few rows, very wide
    (40, 80, 96, 1), (300, 48, 160, 1),                                   # K no multiple of 128: in blocks of 16 rows
])
def test_tiled_gemm_reads_weights_in_fragment_order(ops, M, N, K, S):
    """The tiles for 9 rows and more over pack_weight(W): the same sums in the same order as over plain rows
    (bit for bit where both run the same tile), for every tile shape, with ragged edges in M and N, and as
    partial sums over slices of K."""
    x, w = rnd((M, K), 16, BF16), rnd((N, K), 17, BF16)
    wd = w.to(DEV)
    wp = ops.pack_weight(wd)
    assert wp is not None
    want = (x.double() @ w.double().T).float()
    atol = 1e-3 * math.sqrt(K)
    for out_dtype in ((F32,) if S > 1 else (BF16, F32)):
        shape = (S, M, N) if S > 1 else (M, N)
        got = torch.full(shape, float("nan"), dtype=out_dtype, device=DEV)
        ops.gemm(x.to(DEV), wp, got)
        total = got.float().sum(0) if S > 1 else got
        close(total, want, atol if out_dtype == F32 else atol + 0.02, 0 if out_dtype == F32 else 1e-2,
              f"gemm over fragment order {M}x{N}x{K}")
        if K % 128 == 0 and not (N >= 65536 and K % 256):   # (very wide and K no multiple of 256: plain rows take another tile)
            plain = torch.full(shape, float("nan"), dtype=out_dtype, device=DEV)
            ops.gemm(x.to(DEV), wd, plain)
            assert torch.equal(plain, got), "the same tiles over both layouts must give the same bits"


@pytest.mark.parametrize("M,I,K", [(9, 48, 128), (16, 2560, 4096), (33, 80, 128), (64, 1024, 512), (100, 176, 384),
                                   (128, 12288, 4096), (192, 1040, 256), (256, 2560, 1024), (300, 112, 128),
                                   (1000, 6160, 256), (2048, 1024, 512), (20, 40000, 128), (40, 48, 96)])
def test_tiled_gated_gemm_reads_weights_in_fragment_order(ops, M, I, K):
    x = rnd((M, K), 18, BF16)
    wg, wu = rnd((I, K), 19, BF16, 0.5), rnd((I, K), 20, BF16, 0.5)
    paired = ops.pair_rows(wg.to(DEV), wu.to(DEV))
    wp = ops.pack_weight(paired)
    g = x.double() @ wg.double().T
    want = (g / (1 + torch.exp(-g)) * (x.double() @ wu.double().T)).float()
    got = torch.full((M, I), float("nan"), dtype=BF16, device=DEV)
    ops.gemm_swiglu(x.to(DEV), wp, got)
    close(got, want, 0.03 + 2e-3 * math.sqrt(K), 2e-2, f"gated gemm over fragment order {M}x{I}x{K}")
    if K % 128 == 0 and 2 * I < 65536:
        plain = torch.empty((M, I), dtype=BF16, device=DEV)
        ops.gemm_swiglu(x.to(DEV), paired, plain)
        assert torch.equal(plain, got)


def test_embedding_from_a_table_in_fragment_order(ops):
    V, H = 1008, 4128
    table = rnd((V, H), 21, BF16)
    ids = torch.tensor([0, 15, 16, 17, V - 1, 500, 31], dtype=I32)
    out = torch.full((ids.numel(), H), float("nan"), dtype=F32, device=DEV)
    ops.embed(ops.pack_weight(table.to(DEV)), ids.to(DEV), out)
    assert torch.equal(out.cpu(), table[ids.long()].to(F32))


def test_gemm_bf16_paths_agree(ops):
    """The MFMA kernels and the plain kernel compute the same sums."""
    for M in (4, 40, 300):
        x, w = rnd((M, 256), 12, BF16).to(DEV), rnd((96, 256), 13, BF16).to(DEV)
        a = torch.empty((M, 96), dtype=F32, device=DEV)
        b = torch.empty((M, 96), dtype=F32, device=DEV)
        ops.gemm(x, w, a)
        ops.gemm(x, w, b, force_simt=True)
        close(a, b, 2e-4, what=f"mfma vs plain, M={M}")


# ----------------------------------------------------------------------------- cache write + attention

def dv(v):
    """V pages as plain (dim, token) rows on the CPU -> on the device in the kernels' own order."""
    from synaptix_amd.kernels import ops as real_ops
    return real_ops.v_pages_to_kernel_order(v).to(DEV)


def hv(v):
    """V pages from the device back to plain (dim, token) rows on the CPU."""
    from synaptix_amd.kernels import ops as real_ops
    return real_ops.v_pages_from_kernel_order(v.cpu())


def make_cache(n_pages, nkv, hd, dtype, seed, fill="garbage"):
    """Pages filled with large values: whatever a kernel reads beyond a sequence's end shows."""
    k = rnd((n_pages, nkv, 64, hd), seed, dtype, 50.0)
    v = rnd((n_pages, nkv, hd, 64), seed + 1, dtype, 50.0)
    if fill == "nan":
        k[:], v[:] = float("nan"), float("nan")
    return k, v


def step_arrays(past, new):
    tok_seq, tok_pos, starts = [], [], [0]
    for i, (p, n) in enumerate(zip(past, new)):
        tok_seq += [i] * n
        tok_pos += list(range(p, p + n))
        starts.append(starts[-1] + n)
    t = lambda a: torch.tensor(a, dtype=I32)
    return t(tok_seq), t(tok_pos), t(starts), t(past), t([p + n for p, n in zip(past, new)])


def shuffled_table(n_seqs, width, seed):
    """Each sequence's pages lie scattered over the pool."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_seqs * width, generator=g).to(I32)
    return perm.view(n_seqs, width).contiguous()


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("nh,nkv,hd,rot,norm", [(4, 2, 16, 16, True), (6, 3, 48, 32, True), (8, 1, 128, 128, False),
                                                (3, 3, 80, 0, True)])
def test_qk_norm_rope_kv_write(ops, dtype, nh, nkv, hd, rot, norm):
    past, new = [3, 70, 0], [5, 1, 66]
    tok_seq, tok_pos, _, _, _ = step_arrays(past, new)
    N = len(tok_seq)
    table = shuffled_table(3, 3, 1)
    qkv = rnd((N, (nh + 2 * nkv) * hd), 20, dtype)
    qg = (1 + 0.1 * rnd((hd,), 21)).to(dtype) if norm else None
    kg = (1 + 0.1 * rnd((hd,), 22)).to(dtype) if norm else None
    cos = sin = None
    if rot:
        ang = torch.arange(200, dtype=F32)[:, None] * (10000.0 ** (-torch.arange(rot // 2, dtype=F32) * 2 / rot))[None]
        cos, sin = torch.cos(ang), torch.sin(ang)
    k0, v0 = make_cache(9, nkv, hd, dtype, 23)
    kw, vw, qw = k0.clone(), v0.clone(), torch.empty((N, nh * hd), dtype=dtype)
    ref.qk_norm_rope_kv_write(qkv, qw, kw, vw, table, tok_seq, tok_pos, qg, kg, 1e-5, cos, sin, nh, nkv, hd)
    d = lambda t: None if t is None else t.to(DEV)
    kd, vd, qd = k0.to(DEV), dv(v0), torch.empty((N, nh * hd), dtype=dtype, device=DEV)
    ops.qk_norm_rope_kv_write(d(qkv), qd, kd, vd, d(table), d(tok_seq), d(tok_pos), d(qg), d(kg), 1e-5, d(cos), d(sin),
                              nh, nkv, hd)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == F32 else dict(atol=3e-2, rtol=1e-2)
    close(qd, qw, what="q", **tol)
    close(kd, kw, what="k pages", **tol)
    assert torch.equal(hv(vd), vw), "v is a copy"
    # untouched places of the pages stay as they were
    untouched = (kw == k0)
    assert torch.equal(kd.cpu()[untouched], k0[untouched])
    # the same from float partial sums [S, N, width] (a product cut along K): they are added first
    if dtype == BF16:
        parts = rnd((3, N, (nh + 2 * nkv) * hd), 24)
        parts[2] = qkv.float() - parts[0] - parts[1]
        kd3, vd3, qd3 = k0.to(DEV), dv(v0), torch.empty((N, nh * hd), dtype=dtype, device=DEV)
        ops.qk_norm_rope_kv_write(d(parts), qd3, kd3, vd3, d(table), d(tok_seq), d(tok_pos), d(qg), d(kg), 1e-5, d(cos),
                                  d(sin), nh, nkv, hd)
        close(qd3, qw, what="q from partial sums", **tol)
        close(kd3, kw, what="k pages from partial sums", **tol)
        close(hv(vd3), vw, 2e-2, 1e-2, what="v pages from partial sums")
    # a reader of another layer's cache writes nothing
    kd2, vd2 = k0.to(DEV), dv(v0)
    ops.qk_norm_rope_kv_write(d(qkv), qd, kd2, vd2, d(table), d(tok_seq), d(tok_pos), d(qg), d(kg), 1e-5, d(cos), d(sin),
                              nh, nkv, hd, write_kv=False)
    assert torch.equal(kd2.cpu(), k0) and torch.equal(hv(vd2), v0)
    close(qd, qw, what="q without cache write", **tol)


def fill_sequences(k, v, table, lens, nkv, hd, dtype, seed):
    """Write O(1) keys and values for positions below each length; the rest stays garbage."""
    for b, T in enumerate(lens):
        kk = rnd((T, nkv, hd), seed + 10 * b, dtype)
        vv = rnd((T, nkv, hd), seed + 10 * b + 1, dtype)
        for t in range(T):
            page = int(table[b, t // 64])
            k[page, :, t % 64, :] = kk[t]
            v[page, :, :, t % 64] = vv[t]


ATTN_SHAPES = [
    # nh, nkv, hd, past, new, window
    (4, 2, 16, [0, 0, 0], [5, 17, 70], 0),
    (8, 1, 32, [0, 100, 63], [130, 1, 2], 0),
    (6, 3, 48, [10, 0], [40, 200], 0),
    (8, 2, 64, [600, 0], [1, 8], 0),            # the reference's decode shape (2,8,2,1,600,64) beside a short one
    (32, 8, 128, [0], [300], 0),
    (4, 4, 128, [0, 40], [33, 1], 0),
    (4, 2, 96, [0, 5], [150, 100], 37),          # a window that ends inside pages
    (5, 5, 16, [200], [1], 64),
    (8, 2, 64, [100, 64, 127], [70, 64, 2], 0),   # chunks of a prompt that start inside a page, at its edge, before its end
    (32, 8, 128, [100, 1000], [150, 130], 0),     # the same at the head size and group of the large models
    (6, 2, 48, [33], [300], 50),                  # a chunk over several pages with a window
    (8, 4, 64, [5, 0, 190], [260, 129, 3], 70),   # head size 64 with a window, sequences that end inside pages
    (16, 2, 128, [0, 77], [513, 200], 0),         # eight heads a group, several tiles of 128 rows
    (32, 8, 128, [5, 190], [260, 131], 70),       # the head size of the large models with a window whose edge lies inside pages
]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("nh,nkv,hd,past,new,window", ATTN_SHAPES)
def test_attention_prefill(ops, dtype, nh, nkv, hd, past, new, window):
    B = len(past)
    lens = [p + n for p, n in zip(past, new)]
    width = max((T + 63) // 64 for T in lens) + 1
    table = shuffled_table(B, width, 3)
    # what lies in the pages behind a sequence's end is NaN for the head sizes of the kernel with 32 query rows a
    # wave (and finite garbage elsewhere): a value that leaked from there, times a weight of zero, would show
    k, v = make_cache(B * width, nkv, hd, dtype, 30, fill="nan" if (hd in (64, 128) and dtype == BF16) else "garbage")
    fill_sequences(k, v, table, lens, nkv, hd, dtype, 31)
    tok_seq, tok_pos, starts, past_t, len_t = step_arrays(past, new)
    N = len(tok_seq)
    q = rnd((N, nh * hd), 32, dtype)
    scale = 1 / math.sqrt(hd)
    want = torch.empty((N, nh * hd), dtype=F32)
    ref.attention_f32(q.float(), torch.nan_to_num(k.float()), torch.nan_to_num(v.float()), table, tok_seq, tok_pos, want,
                      scale, window, nh, nkv, hd)
    d = lambda t: t.to(DEV)
    out = torch.empty((N, nh * hd), dtype=dtype, device=DEV)
    if dtype == F32:
        ops.attention_f32(d(q), d(k), dv(v), d(table), d(tok_seq), d(tok_pos), out, scale, window, nh, nkv, hd)
        close(out, want, 1e-4, what="attention f32")
    else:
        ops.attention_prefill_bf16(d(q), d(k), dv(v), d(table), d(starts), d(past_t), out, scale, window, nh, nkv, hd)
        close(out, want, 2e-2, 1e-2, what="attention prefill bf16")
        # both kernels where the head size allows both: waves of 16 and of 32 query rows
        for variant in (1, 2):
            out.fill_(float("nan"))
            if variant == 2 and hd not in (64, 128):
                with pytest.raises(Exception, match="waves of 32 rows"):
                    ops.attention_prefill_bf16(d(q), d(k), dv(v), d(table), d(starts), d(past_t), out, scale, window,
                                               nh, nkv, hd, variant=variant)
                continue
            ops.attention_prefill_bf16(d(q), d(k), dv(v), d(table), d(starts), d(past_t), out, scale, window, nh, nkv,
                                       hd, variant=variant)
            close(out, want, 2e-2, 1e-2, what=f"attention prefill bf16, variant {variant}")
            # sequences with a single new token left out (a step of prompts and single tokens hands them to the
            # kernel for single tokens): their rows stay as they were, the others are computed as before
            if 1 in new and any(n > 1 for n in new):
                out.fill_(7.0)
                ops.attention_prefill_bf16(d(q), d(k), dv(v), d(table), d(starts), d(past_t), out, scale, window, nh, nkv,
                                           hd, variant=variant, skip_below=2)
                single = torch.tensor([n == 1 for n in new])[tok_seq.long()]
                assert bool((out.cpu()[single] == 7.0).all()), "a single token's row was written"
                close(out.cpu()[~single], want[~single], 2e-2, 1e-2, what=f"prompts beside skipped single tokens, variant {variant}")


@pytest.mark.parametrize("nh,nkv,hd,past,new,window,softcap,sloped", [
    (4, 2, 16, [0, 0], [40, 130], 0, 0.0, True),          # a penalty in the distance alone
    (8, 2, 64, [100, 0], [70, 129], 0, 2.0, False),       # a soft cap alone (head size 64: the kernel with 16 rows a wave takes it)
    (32, 8, 128, [30], [300], 0, 1.0, True),              # both, at the head size and group of the large models
    (6, 3, 48, [10, 0], [40, 200], 50, 3.0, True),        # with a window
])
def test_attention_with_terms_on_the_scores(ops, nh, nkv, hd, past, new, window, softcap, sloped):
    """score = cap * tanh(score / cap) - slope[head] * (query position - key position) before mask and softmax, in
    every attention kernel: 32-bit, prompt (bf16), single tokens in splits (bf16), against the plain statement."""
    B = len(past)
    lens = [p + n for p, n in zip(past, new)]
    width = max((T + 63) // 64 for T in lens) + 1
    table = shuffled_table(B, width, 5)
    slopes = torch.tensor([0.5 ** (1 + h % 5) for h in range(nh)], dtype=F32) if sloped else None
    tok_seq, tok_pos, starts, past_t, len_t = step_arrays(past, new)
    N = len(tok_seq)
    scale = 1 / math.sqrt(hd)
    d = lambda t: None if t is None else t.to(DEV)
    for dtype in (F32, BF16):
        k, v = make_cache(B * width, nkv, hd, dtype, 50)
        fill_sequences(k, v, table, lens, nkv, hd, dtype, 51)
        q = rnd((N, nh * hd), 52, dtype, 2.0)              # scores large enough that the cap bends them
        want = torch.empty((N, nh * hd), dtype=F32)
        ref.attention_f32(q.float(), torch.nan_to_num(k.float()), torch.nan_to_num(v.float()), table, tok_seq, tok_pos, want,
                          scale, window, nh, nkv, hd, slopes, softcap)
        plain = torch.empty_like(want)
        ref.attention_f32(q.float(), torch.nan_to_num(k.float()), torch.nan_to_num(v.float()), table, tok_seq, tok_pos, plain,
                          scale, window, nh, nkv, hd)
        assert float((want - plain).abs().max()) > 0.1     # the terms matter at these sizes
        out = torch.empty((N, nh * hd), dtype=dtype, device=DEV)
        if dtype == F32:
            ops.attention_f32(d(q), d(k), dv(v), d(table), d(tok_seq), d(tok_pos), out, scale, window, nh, nkv, hd,
                              slopes=d(slopes), softcap=softcap)
            close(out, want, 2e-4, what="attention f32 with terms")
            continue
        ops.attention_prefill_bf16(d(q), d(k), dv(v), d(table), d(starts), d(past_t), out, scale, window, nh, nkv, hd,
                                   slopes=d(slopes), softcap=softcap)
        close(out, want, 2e-2, 1e-2, what="attention prefill bf16 with terms")
        if hd in (64, 128):
            with pytest.raises(Exception, match="no terms on the scores"):
                ops.attention_prefill_bf16(d(q), d(k), dv(v), d(table), d(starts), d(past_t), out, scale, window, nh, nkv,
                                           hd, variant=2, slopes=d(slopes), softcap=softcap)
        # single tokens: the last token of each sequence as a decode step over the same cache
        last = torch.tensor([int(starts[b + 1]) - 1 for b in range(B)])
        outd = torch.empty((B, nh * hd), dtype=BF16, device=DEV)
        for splits in (1, 3):
            work = torch.empty(B * nh * splits * (hd + 2), dtype=F32, device=DEV)
            ops.attention_decode_bf16(d(q[last].contiguous()), d(k), dv(v), d(table), d(torch.tensor(lens, dtype=I32)), outd,
                                      work, splits, scale, window, nh, nkv, hd, slopes=d(slopes), softcap=softcap)
            close(outd, want[last], 2e-2, 1e-2, what=f"attention decode bf16 with terms, {splits} splits")


def merged_in_kernel(run, two_kernels, want, lens, splits, window, nh, nkv, work):
    """The same call with the merge of the splits inside the one launch, by the workgroup that finishes last:
    first with every sequence in `splits` splits, then with the host's work list, which gives long sequences
    more of them; twice each with the same counters, which the kernel has to leave at zero.  Before every run
    the partial results' memory is filled with NaN by another kernel: a workgroup that merged what an earlier
    launch left in its cache, and not what the other workgroups of this launch have written, would show it."""
    if splits == 1:
        return
    chunks = -(-(nh // nkv) // 16)
    counters = torch.zeros(len(lens) * nkv * chunks, dtype=I32, device=DEV)
    items = torch.tensor(rt.decode_items(lens, splits, window or None), dtype=I32, device=DEV)
    for what, kw in (("merged in the kernel", dict(counters=counters)),
                     ("with a work list", dict(counters=counters, items=items)),
                     ("with a work list, merged by the second kernel", dict(items=items))):
        outs = []
        for _ in range(2):
            got = torch.full_like(two_kernels, float("nan"))
            work.fill_(float("nan"))
            run(got, **kw)
            close(got, want, 2e-2, 1e-2, what=f"decode attention {what}")
            outs.append(got.cpu())
            assert int(counters.abs().sum()) == 0, f"{what}: counters are not back at zero"
        assert torch.equal(outs[0], outs[1]), f"{what}: two runs differ"
    # the same splits merged by either way: the same sums in another order
    got = torch.empty_like(two_kernels)
    run(got, counters=counters)
    close(got, two_kernels.float().cpu(), 1e-2, 1e-2, what="merge in the kernel against the merge kernel")


@pytest.mark.parametrize("nh,nkv,hd,lens,window,splits", [
    (8, 2, 64, [600, 3], 0, 4),                 # crates/synaptix-kernels-cuda/tests/cuda_flash_decode.rs:101 GQA, Tkv=600
    (4, 4, 128, [40], 0, 8),                    # more splits than pages (empty splits), ibid. 130-183
    (40, 2, 32, [129, 64, 65, 1], 0, 3),        # 20 heads a group: two chunks of 16
    (8, 1, 16, [1000, 77], 0, 16),
    (4, 2, 96, [500, 30], 100, 5),
    (32, 8, 128, [2100] * 3, 0, 11),
    (6, 2, 48, [35], 0, 1),                     # head sizes that are no multiple of 32, three heads a group
    (6, 2, 48, [200, 35, 64], 0, 3),
    (5, 1, 80, [100, 300], 0, 2),
    (4, 4, 112, [70], 0, 1),
    (8, 2, 256, [130, 700], 0, 4),
    (32, 8, 128, [7000, 40], 0, 32),            # long contexts: 32 and 64 splits, most of them empty for the short sequence
    (8, 2, 64, [6500, 130, 7000], 0, 64),
    (4, 1, 32, [4100], 0, 24),
    (32, 8, 128, [3000, 500, 2600, 100, 1500], 0, 16),   # 640 workgroups: more than two a compute unit, merged by the second kernel
])
def test_attention_decode_bf16(ops, nh, nkv, hd, lens, window, splits):
    B = len(lens)
    width = max((T + 63) // 64 for T in lens) + 2
    table = shuffled_table(B, width, 4)
    k, v = make_cache(B * width, nkv, hd, BF16, 40, fill="nan" if hd == 64 else "garbage")
    fill_sequences(k, v, table, lens, nkv, hd, BF16, 41)
    tok_seq = torch.arange(B, dtype=I32)
    tok_pos = torch.tensor([T - 1 for T in lens], dtype=I32)
    q = rnd((B, nh * hd), 42, BF16)
    scale = 1 / math.sqrt(hd)
    want = torch.empty((B, nh * hd), dtype=F32)
    kf, vf = torch.nan_to_num(k.float()), torch.nan_to_num(v.float())
    ref.attention_f32(q.float(), kf, vf, table, tok_seq, tok_pos, want, scale, window, nh, nkv, hd)
    d = lambda t: t.to(DEV)
    out = torch.empty((B, nh * hd), dtype=BF16, device=DEV)
    work = torch.empty(B * nh * splits * (hd + 2), dtype=F32, device=DEV)
    ops.attention_decode_bf16(d(q), d(k), dv(v), d(table), d(torch.tensor(lens, dtype=I32)), out, work, splits, scale,
                              window, nh, nkv, hd)
    close(out, want, 2e-2, 1e-2, what="attention decode bf16")
    merged_in_kernel(lambda out2, **kw: ops.attention_decode_bf16(
        d(q), d(k), dv(v), d(table), d(torch.tensor(lens, dtype=I32)), out2, work, splits, scale, window, nh, nkv, hd, **kw),
        out, want, lens, splits, window, nh, nkv, work)


@pytest.mark.parametrize("lens,splits", [([2061] * 8, 4), ([2061], 16), ([3908, 457, 1200, 2500], 8)])
def test_merge_inside_the_launch_reads_what_this_launch_wrote(ops, lens, splits):
    """The workgroup that merges the splits reads partial results that workgroups on other XCDs, each with a
    second-level cache of its own, wrote within the same launch.  200 launches at a decode step's shapes, the
    memory of the partial results filled with NaN by another kernel before each and the keys of other launches
    read in between: every output equals the first, none is NaN."""
    nh, nkv, hd = 32, 8, 128
    B = len(lens)
    width = max((T + 63) // 64 for T in lens) + 1
    table = shuffled_table(B, width, 6)
    k, v = make_cache(B * width, nkv, hd, BF16, 70)
    fill_sequences(k, v, table, lens, nkv, hd, BF16, 71)
    q = rnd((B, nh * hd), 72, BF16)
    d = lambda t: t.to(DEV)
    qd, kd, vd, td, ld = d(q), d(k), dv(v), d(table), d(torch.tensor(lens, dtype=I32))
    work = torch.empty(B * nh * splits * (hd + 2), dtype=F32, device=DEV)
    counters = torch.zeros(B * nkv, dtype=I32, device=DEV)
    items = torch.tensor(rt.decode_items(lens, splits), dtype=I32, device=DEV)
    other = torch.randn(64 << 20, device=DEV)          # 256 MB that a kernel in between reads
    first = None
    for i in range(200):
        out = torch.full((B, nh * hd), float("nan"), dtype=BF16, device=DEV)
        work.fill_(float("nan"))
        if i % 3 == 0:
            other.sum()
        ops.attention_decode_bf16(qd, kd, vd, td, ld, out, work, splits, 1 / math.sqrt(hd), 0, nh, nkv, hd,
                                  counters=counters, items=items if i % 2 else None)
        if first is None:
            first = {}
        key = i % 2
        if key not in first:
            assert torch.isfinite(out.float()).all()
            first[key] = out.clone()
        else:
            assert torch.equal(out, first[key]), f"launch {i} differs from the first of its kind"
    assert int(counters.abs().sum()) == 0


@pytest.mark.parametrize("nh,nkv,hd,rot,norm,lens,window,splits,parts,own", [
    (4, 2, 16, 16, True, [1, 5, 64, 65, 200], 0, 1, 0, True),        # a first token, page edges
    (8, 2, 128, 128, True, [700, 33, 129], 0, 4, 8, True),           # float partial sums, splits
    (6, 2, 48, 32, True, [300, 64], 0, 3, 3, True),                  # partial rotation, head size 48
    (4, 1, 64, 64, False, [500, 2], 100, 2, 0, True),                # no q/k norm, a window
    (40, 2, 32, 0, True, [90, 300], 0, 2, 2, True),                  # no rotation, 20 heads a group (two chunks)
    (8, 4, 128, 128, True, [257, 1000], 0, 8, 4, False),             # reads a cache that another layer wrote
    (32, 8, 128, 128, True, [7000, 33], 0, 32, 4, True),             # long contexts: 32 and 64 splits
    (4, 1, 64, 64, True, [6500, 100, 6401], 0, 64, 0, True),
])
def test_attention_decode_with_qkv_intake(ops, nh, nkv, hd, rot, norm, lens, window, splits, parts, own):
    """Decode attention that makes q, k and v from the fused projection itself equals the q/k kernel
    followed by plain decode attention: the same outputs and the same cache contents afterwards."""
    B, heads = len(lens), nh + 2 * nkv
    width = max((T + 63) // 64 for T in lens) + 2
    table = shuffled_table(B, width, 5)
    k, v = make_cache(B * width, nkv, hd, BF16, 60)
    fill_sequences(k, v, table, lens, nkv, hd, BF16, 61)
    qkv_full = rnd((B, heads * hd), 62, F32)
    if parts:
        cut = torch.rand((parts, 1, 1), generator=torch.Generator().manual_seed(63)) + 0.1
        qkv = (qkv_full[None] * (cut / cut.sum())).contiguous()       # float partial sums that add up to it
    else:
        qkv = qkv_full.to(BF16)
    qg = (1 + 0.2 * rnd((hd,), 64)).to(BF16) if norm else None
    kg = (1 + 0.2 * rnd((hd,), 65)).to(BF16) if norm else None
    cos = sin = None
    if rot:
        ang = torch.arange(max(lens) + 1, dtype=F32)[:, None] * (0.3 / (1 + torch.arange(rot // 2, dtype=F32)))[None, :]
        cos, sin = torch.cos(ang), torch.sin(ang)
    seq_len = torch.tensor(lens, dtype=I32)
    tok_seq, tok_pos = torch.arange(B, dtype=I32), seq_len - 1
    scale = 1 / math.sqrt(hd)
    # the two-kernel way, on the CPU reference
    k_ref, v_ref = k.clone(), v.clone()
    q_ref = torch.empty((B, nh * hd), dtype=BF16)
    ref.qk_norm_rope_kv_write(qkv, q_ref, k_ref, v_ref, table, tok_seq, tok_pos, qg, kg, 1e-5, cos, sin, nh, nkv, hd,
                              write_kv=own)
    want = torch.empty((B, nh * hd), dtype=F32)
    ref.attention_f32(q_ref.float(), k_ref.float(), v_ref.float(), table, tok_seq, tok_pos, want, scale, window, nh, nkv, hd)
    d = lambda t: None if t is None else t.to(DEV)
    kd, vd = d(k), dv(v)
    out = torch.empty((B, nh * hd), dtype=BF16, device=DEV)
    work = torch.empty(B * nh * splits * (hd + 2), dtype=F32, device=DEV)
    ops.attention_decode_fused_bf16(d(qkv), kd, vd, d(table), d(seq_len), out, work, splits, scale, window, nh, nkv, hd,
                                    d(qg), d(kg), 1e-5, d(cos), d(sin), write_kv=own)
    close(out, want, 2e-2, 1e-2, what="decode attention with q/k/v intake")
    merged_in_kernel(lambda out2, **kw: ops.attention_decode_fused_bf16(
        d(qkv), kd, vd, d(table), d(seq_len), out2, work, splits, scale, window, nh, nkv, hd, d(qg), d(kg), 1e-5, d(cos),
        d(sin), write_kv=own, **kw), out, want, lens, splits, window, nh, nkv, work)
    # the cache afterwards: the new rows written (or nothing touched)
    close(kd, k_ref.float(), 2e-2, 1e-2, what="k pages after the step")
    close(hv(vd), v_ref.float(), 2e-2, 1e-2, what="v pages after the step")
    if not own:
        assert torch.equal(kd.cpu(), k) and torch.equal(hv(vd), v)


def test_attention_far_key_stands_out(ops):
    """One key among hundreds is made to dominate: the output must be that key's value, in every
    kernel.  A kernel that loses a page, a split or the cache's start would not show it with
    random data."""
    nh, nkv, hd, T = 4, 2, 64, 700
    scale = 1 / math.sqrt(hd)
    for far in (0, 63, 64, 350, T - 1):
        table = shuffled_table(1, 12, far)
        k, v = make_cache(12, nkv, hd, BF16, 50)
        fill_sequences(k, v, table, [T], nkv, hd, BF16, 51)
        q = rnd((1, nh * hd), 52, BF16)
        page = int(table[0, far // 64])
        for h in range(nkv):   # the far key is 20 x the query of the group's first head
            k[page, h, far % 64, :] = (q.view(nh, hd)[h * 2] * 20).to(BF16)
        want = v[page, :, :, far % 64].float()            # [nkv, hd]
        d = lambda t: t.to(DEV)
        lens = torch.tensor([T], dtype=I32)
        out = torch.empty((1, nh * hd), dtype=BF16, device=DEV)
        work = torch.empty(nh * 6 * (hd + 2), dtype=F32, device=DEV)
        ops.attention_decode_bf16(d(q), d(k), dv(v), d(table), d(lens), out, work, 6, scale, 0, nh, nkv, hd)
        got = out.cpu().float().view(nh, hd)
        for h in range(nkv):
            close(got[h * 2], want[h], 3e-2, 2e-2, f"decode, far key {far}")
        outp = torch.empty((1, nh * hd), dtype=BF16, device=DEV)
        ops.attention_prefill_bf16(d(q), d(k), dv(v), d(table), d(torch.tensor([0, 1], dtype=I32)),
                                   d(torch.tensor([T - 1], dtype=I32)), outp, scale, 0, nh, nkv, hd)
        gotp = outp.cpu().float().view(nh, hd)
        for h in range(nkv):
            close(gotp[h * 2], want[h], 3e-2, 2e-2, f"prefill, far key {far}")
        o32 = torch.empty((1, nh * hd), dtype=F32, device=DEV)
        ops.attention_f32(d(q.float()), d(k.float()), d(v.float()), d(table), d(torch.zeros(1, dtype=I32)),
                          d(torch.tensor([T - 1], dtype=I32)), o32, scale, 0, nh, nkv, hd)
        got32 = o32.cpu().view(nh, hd)
        for h in range(nkv):
            close(got32[h * 2], want[h], 1e-3, 1e-3, f"f32, far key {far}")


def test_attention_window_edge(ops):
    """The key just outside the window dominates if it is seen: it must not be."""
    nh, nkv, hd, T, W = 2, 1, 32, 300, 100
    scale = 1 / math.sqrt(hd)
    table = shuffled_table(1, 6, 9)
    k, v = make_cache(6, nkv, hd, BF16, 60)
    fill_sequences(k, v, table, [T], nkv, hd, BF16, 61)
    q = rnd((1, nh * hd), 62, BF16)
    edge = T - 1 - W          # the last key outside: visible keys are j > T-1-W
    page = int(table[0, edge // 64])
    k[page, 0, edge % 64, :] = (q.view(nh, hd)[0] * 20).to(BF16)
    tok_seq, tok_pos = torch.zeros(1, dtype=I32), torch.tensor([T - 1], dtype=I32)
    want = torch.empty((1, nh * hd), dtype=F32)
    ref.attention_f32(q.float(), k.float(), v.float(), table, tok_seq, tok_pos, want, scale, W, nh, nkv, hd)
    seen = torch.empty((1, nh * hd), dtype=F32)
    ref.attention_f32(q.float(), k.float(), v.float(), table, tok_seq, tok_pos, seen, scale, W + 1, nh, nkv, hd)
    assert (want - seen).abs().max() > 1.0, "the test's key does not dominate"
    d = lambda t: t.to(DEV)
    out = torch.empty((1, nh * hd), dtype=BF16, device=DEV)
    work = torch.empty(nh * 3 * (hd + 2), dtype=F32, device=DEV)
    ops.attention_decode_bf16(d(q), d(k), dv(v), d(table), d(torch.tensor([T], dtype=I32)), out, work, 3, scale, W, nh,
                              nkv, hd)
    close(out, want, 2e-2, 1e-2, "decode at the window's edge")
    ops.attention_prefill_bf16(d(q), d(k), dv(v), d(table), d(torch.tensor([0, 1], dtype=I32)),
                               d(torch.tensor([T - 1], dtype=I32)), out, scale, W, nh, nkv, hd)
    close(out, want, 2e-2, 1e-2, "prefill at the window's edge")
    o32 = torch.empty((1, nh * hd), dtype=F32, device=DEV)
    ops.attention_f32(d(q.float()), d(k.float()), d(v.float()), d(table), d(tok_seq), d(tok_pos), o32, scale, W, nh, nkv,
                      hd)
    close(o32, want, 1e-4, what="f32 at the window's edge")


# ----------------------------------------------------------------------------- sampling

@pytest.mark.parametrize("V", [1000, 999, 40004])
def test_sample_rows_greedy_and_ties(ops, V):
    x = rnd((5, V), 70)
    x[1, 17] = x[1, 900] = 9.0           # the last of equal maxima wins
    x[2, :] = 0.0                        # all equal: the last index
    out = torch.empty(5, dtype=I32, device=DEV)
    ops.sample_rows(x.to(DEV), None, None, out)
    want = [int(x[0].argmax()), 900, V - 1, int(x[3].argmax()), int(x[4].argmax())]
    assert out.cpu().tolist() == want


def test_sample_rows_temperature(ops):
    V, R = 333, 64
    x = rnd((R, V), 71, scale=3.0)
    temps = torch.tensor([0.7, 1.0, 0.0, 1.5] * (R // 4))
    g = torch.Generator().manual_seed(5)
    u = torch.rand(R, generator=g)
    want = torch.empty(R, dtype=I32)
    ref.sample_rows(x, temps, u, want)
    out = torch.empty(R, dtype=I32, device=DEV)
    ops.sample_rows(x.to(DEV), temps.to(DEV), u.to(DEV), out)
    got = out.cpu()
    # a draw falls on the other side of a boundary only if u is within rounding of the CDF there
    differ = int((got != want).sum())
    assert differ <= 1, f"{differ} of {R} draws differ"
    # u = 1 can never be below the last cumulative sum of rounded probabilities: the last index
    ops.sample_rows(x.to(DEV), torch.ones(R).to(DEV), torch.full((R,), 1.5).to(DEV), out)
    assert out.cpu().tolist() == [V - 1] * R


def test_sample_rows_frequencies(ops):
    """Frequencies of many draws lie within 0.01 of the probabilities
    (as crates/synaptix-infer/tests/ref_infer.rs:114-166, with fewer draws)."""
    V, R = 50, 20000
    logits = rnd((1, V), 72, scale=1.5)
    x = logits.expand(R, V).contiguous()
    g = torch.Generator().manual_seed(6)
    u = torch.rand(R, generator=g)
    out = torch.empty(R, dtype=I32, device=DEV)
    ops.sample_rows(x.to(DEV), torch.full((R,), 0.8).to(DEV), u.to(DEV), out)
    freq = torch.bincount(out.cpu().long(), minlength=V).float() / R
    p = torch.softmax(logits[0] / 0.8, 0)
    assert (freq - p).abs().max() < 0.012


def test_products_of_random_shapes(ops):
    """Shapes drawn at random over every kind of product (plain, as partial sums for a reader that adds them, gated)
    through the entry points that the parts use (parts.linear): each lands in whichever kernel the sizes select, in
    fragment order where the sizes allow it and in plain rows where they do not, and equals the 64-bit product."""
    import random
    from synaptix_amd.parts.linear import Matrix, linear, linear_for_sum
    r = random.Random(11)
    done = 0
    while done < 48:
        M = r.choice([1, 2, 5, 8, 9, 13, 16, 17, 32, 33, 64, 65, 100, 128, 129, 255, 257, 300, 513, 700])
        K = r.choice([8, 24, 32, 40, 64, 96, 128, 136, 192, 256, 264, 512, 1000, 1024, 2080, 4096])
        N = r.choice([8, 16, 24, 32, 48, 80, 96, 128, 160, 200, 384, 400, 1000, 1008, 2048, 4096, 6144, 32784])
        kind = r.choice(["plain", "sum", "gated"])
        if kind == "gated":
            N = max(32, N // 32 * 32)
        if M * N * K > 6e9:
            continue
        done += 1
        x, w = rnd((M, K), 300 + done, BF16), rnd((N, K), 400 + done, BF16, 0.05)
        full = x.double() @ w.double().T
        atol = 4e-4 * math.sqrt(K) + 1e-3
        if kind == "gated":
            m = Matrix(ops.pair_rows(w[:N // 2].contiguous().to(DEV), w[N // 2:].contiguous().to(DEV)))
            out = torch.full((M, N // 2), float("nan"), dtype=BF16, device=DEV)
            ops.gemm_swiglu(x.to(DEV), m.data, out)
            g, u = full[:, :N // 2], full[:, N // 2:]
            close(out, (g / (1 + torch.exp(-g)) * u).float(), atol + 0.02, 1e-2, f"gated {M}x{N}x{K}")
        else:
            m = Matrix(w.to(DEV))
            got = linear(x.to(DEV), m, F32) if kind == "plain" else linear_for_sum(x.to(DEV), m)
            close(got.sum(0) if got.dim() == 3 else got, full.float(), atol, what=f"{kind} {M}x{N}x{K}")


def test_attention_of_random_shapes(ops):
    """The attention tests above at shapes drawn at random: head sizes 16 to 256, groups of 1 to 20 heads, sequences that
    begin, end or are cut at page edges, windows down to one key, any number of splits."""
    import random
    r = random.Random(12)
    for _ in range(10):
        hd = r.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
        nkv = r.choice([1, 2, 3, 4, 8])
        nh = nkv * r.choice([1, 2, 3, 4, 7, 8, 17, 20])
        if nh * hd > 8192:
            continue
        B = r.randint(1, 4)
        past = [r.choice([0, 0, 1, 63, 64, 65, 100, 200, 500]) for _ in range(B)]
        new = [r.choice([1, 2, 31, 32, 33, 64, 100, 128, 129, 200, 300]) for _ in range(B)]
        window = r.choice([0, 0, 0, 1, 37, 64, 70, 200])
        lens = [r.choice([1, 2, 63, 64, 65, 130, 300, 700, 2100, 5000]) for _ in range(B)]
        splits = r.choice([1, 2, 3, 4, 8, 16, 32])
        rot = r.choice([0, hd, hd, hd // 2 if (hd // 2) % 2 == 0 else hd])
        test_attention_prefill(ops, BF16, nh, nkv, hd, past, new, window)
        test_attention_decode_bf16(ops, nh, nkv, hd, lens, window, splits)
        test_attention_decode_with_qkv_intake(ops, nh, nkv, hd, rot, r.random() < 0.7, lens, window, splits,
                                              r.choice([0, 0, 2, 4, 8]), r.random() < 0.8)


def _filter(ops, x, options, ids=None, in_place=False):
    """ops.filter_rows over rows x [R, V] with options = list of dicts (k, p, mp, T, rep, pres, freq) and ids = list of lists."""
    R, V = x.shape
    col = lambda key, default, dt: torch.tensor([o.get(key, default) for o in options], dtype=dt).to(DEV)
    flat, starts = [], [0]
    for r in range(R):
        flat += list(ids[r]) if ids else []
        starts.append(len(flat))
    xd = x.to(DEV).contiguous()
    out = xd if in_place else torch.full_like(xd, float("nan"))
    counts = torch.zeros(R * V, dtype=I32, device=DEV) if flat else None
    ops.filter_rows(xd, out, col("T", 1.0, F32), col("k", 0, I32), col("p", 1.0, F32), col("mp", 0.0, F32),
                    col("rep", 1.0, F32), col("pres", 0.0, F32), col("freq", 0.0, F32),
                    torch.tensor(flat, dtype=I32).to(DEV) if flat else None,
                    torch.tensor(starts, dtype=I32).to(DEV) if flat else None, counts)
    torch.cuda.synchronize()
    if counts is not None:
        assert int(counts.abs().sum()) == 0, "the penalties' counters are not left zero"
    return out.cpu()


def _plain_filter(x, o, ids):
    """The plain processors in the reference's order (tests/plain_qwen3.py)."""
    import plain_qwen3 as P
    want = x.clone()
    if o.get("rep", 1.0) != 1.0:
        want = P.repetition_penalty(want, ids, o["rep"], 0)
    if o.get("pres", 0.0) != 0.0 or o.get("freq", 0.0) != 0.0:
        want = P.presence_frequency(want, ids, o.get("pres", 0.0), o.get("freq", 0.0), 0)
    T = o.get("T", 1.0)
    if T > 0 and T != 1.0:
        want = want / torch.tensor(T, dtype=F32)
    if o.get("k", 0):
        want = P.top_k(want, o["k"])
    if o.get("p", 1.0) < 1.0:
        want = P.top_p(want, o["p"]) if o["p"] <= 0.9 else _top_p_in_64_bit(want, o["p"])
    if o.get("mp", 0.0) > 0.0:
        want = P.min_p(want, o["mp"])
    return want


def _top_p_in_64_bit(x, p):
    """The rule of the plain top_p (a candidate stays while the sum of those before it is at most p * the sum of
    all; sorted by probability, equal ones in index order) with sums in 64-bit.  The reference adds up in 32-bit,
    one candidate after the other (crates/synaptix-infer/src/sampling/top_p.rs:31-40): deep in the tail of a large
    vocabulary a candidate is less than half a unit in the last place of that sum, the sum stands still and the
    cut is never reached; the kernel's sums are exact, so for p near 1 it is held against the rule, not against
    that rounding."""
    probs = torch.exp(x.double() - x.max().double())
    order = torch.argsort(probs, descending=True, stable=True)
    sp = probs[order]
    before = torch.cumsum(sp, 0) - sp
    out = x.clone()
    out[order[(before > p * probs.sum()) & torch.isfinite(x[order])]] = float("-inf")
    return out


@pytest.mark.parametrize("V", [97, 1000, 40000])
def test_filter_rows_against_the_plain_processors(ops, V):
    """Every processor alone and all together, rows with different options in one launch, against the plain
    processors: the same entries dropped, the kept ones equal up to the rounding of the penalty's power."""
    options = [dict(k=1), dict(k=17), dict(k=V - 1), dict(k=V), dict(p=0.9), dict(p=0.3), dict(p=0.999), dict(mp=0.05),
               dict(T=0.7), dict(T=0.0, k=5), dict(rep=1.3), dict(pres=0.4, freq=0.2), dict(rep=0.8, pres=-0.1),
               dict(T=0.8, k=40, p=0.85, mp=0.02, rep=1.2, pres=0.3, freq=0.1), dict(T=1.5, k=300, p=0.5), dict()]
    R = len(options)
    x = rnd((R, V), 90, scale=3.0)
    g = torch.Generator().manual_seed(V)
    ids = [torch.randint(-2, V + 3, (60,), generator=g).tolist() for _ in range(R)]       # some ids lie outside the vocabulary
    for r in range(R):
        ids[r] += ids[r][:20]                                                              # and some come several times
    got = _filter(ops, x, options, ids)
    for r, o in enumerate(options):
        want = _plain_filter(x[r], o, [t for t in ids[r] if t >= 0])
        differ = torch.isinf(got[r]) != torch.isinf(want)
        if o.get("p", 1.0) > 0.9 and bool(differ.any()):
            # deep in the tail neighbours in the sorted order lie 1e-8 of the mass apart, less than the rounding of
            # a 32-bit exponential: an entry may fall on the other side only if it stands that close to the cut
            probs = torch.exp(x[r].double() - x[r].max().double())
            above = torch.stack([probs[probs > probs[j]].sum() for j in differ.nonzero().flatten()]) / probs.sum()
            assert int(differ.sum()) <= 2 and bool(((above - o["p"]).abs() < 1e-6).all()), (r, o, above)
            want = torch.where(differ, got[r], want)
        assert torch.equal(torch.isinf(got[r]), torch.isinf(want)), (r, o, int(differ.sum()))
        keep = ~torch.isinf(want)
        close(got[r][keep], want[keep], 1e-5, 1e-5, what=f"kept logits of row {r}")
    again = _filter(ops, x, options, ids, in_place=True)
    assert torch.equal(torch.nan_to_num(again, neginf=-1e30), torch.nan_to_num(got, neginf=-1e30)), "in place, and the same bits twice"


def test_filter_rows_with_equal_values(ops):
    """Equal values at the k-th place and at the boundary of the probability mass: of equal entries the first in
    index order stay, so that top-k keeps exactly k; rows of one value only; rows that are -inf but for a few."""
    V = 5000
    g = torch.Generator().manual_seed(3)
    coarse = torch.randint(-4, 5, (V,), generator=g).float()              # nine values, hundreds of each
    flat = torch.full((V,), 1.5)
    few = torch.full((V,), float("-inf"))
    few[[7, 4000, 123]] = torch.tensor([2.0, 1.0, 2.0])
    x = torch.stack([coarse, coarse, coarse, flat, flat, few, few, coarse])
    options = [dict(k=50), dict(k=900), dict(p=0.6), dict(k=3), dict(p=0.5), dict(k=2), dict(p=0.7), dict(k=700, p=0.8, mp=0.2)]
    got = _filter(ops, x, options)

    def first_k(row, k):
        order = torch.argsort(row, descending=True, stable=True)
        keep = torch.zeros(V, dtype=torch.bool)
        keep[order[:k]] = True
        return keep

    def first_by_mass(row, p):
        probs = torch.exp(row.double() - row.max().double())
        order = torch.argsort(probs, descending=True, stable=True)
        sp = probs[order]
        before = torch.cumsum(sp, 0) - sp
        keep = torch.zeros(V, dtype=torch.bool)
        keep[order[(before <= p * probs.sum()) & torch.isfinite(row[order])]] = True
        return keep

    kept = ~torch.isinf(got)
    assert torch.equal(kept[0], first_k(coarse, 50)) and int(kept[0].sum()) == 50
    assert torch.equal(kept[1], first_k(coarse, 900)) and int(kept[1].sum()) == 900
    assert torch.equal(kept[2], first_by_mass(coarse, 0.6))
    assert kept[3].nonzero().flatten().tolist() == [0, 1, 2]
    assert torch.equal(kept[4], first_by_mass(flat, 0.5)) and int(kept[4].sum()) == V // 2 + 1
    assert kept[5].nonzero().flatten().tolist() == [7, 123]
    assert kept[6].nonzero().flatten().tolist() == [7, 123]            # 2/(2e^2+e) of the mass before the second, 0.84 before the third
    both = first_k(coarse, 700)
    row = torch.where(both, coarse, torch.full_like(coarse, float("-inf")))
    both &= first_by_mass(row, 0.8)
    both &= torch.exp(coarse - coarse.max()) >= 0.2
    assert torch.equal(kept[7], both)
    assert torch.equal(got[kept], x[kept])                                # what stays is untouched


def test_filter_rows_at_the_vocabulary_of_the_large_models(ops):
    """151,936 logits a row, as the models' output head gives them; a sampled token after the filters lies among
    the entries that were kept."""
    import plain_qwen3 as P
    V = 151936
    x = rnd((3, V), 95, scale=2.5)
    options = [dict(T=0.7, k=50, p=0.9), dict(p=0.95, mp=0.001), dict(T=0.9, k=2000, rep=1.1)]
    ids = [list(range(100, 400)) * 2, [], [5, 5, 5, 9]]
    got = _filter(ops, x, options, ids)
    for r, o in enumerate(options):
        want = _plain_filter(x[r], o, ids[r])
        assert torch.equal(torch.isinf(got[r]), torch.isinf(want)), (r, int((torch.isinf(got[r]) != torch.isinf(want)).sum()))
    out = torch.empty(3, dtype=I32, device=DEV)
    ops.sample_rows(got.to(DEV), torch.ones(3).to(DEV), torch.tensor([0.3, 0.999, 0.0]).to(DEV), out)
    for r, t in enumerate(out.cpu().tolist()):
        assert math.isfinite(float(got[r, t]))


def test_measured_ceilings_are_plausible(ops):
    """The two probes run and report rates of the right order for this kind of machine."""
    read_gbs, mfma_tflops = ops.measure_ceilings(DEV, read_bytes=1 << 28, repeats=2)
    assert 500 < read_gbs < 8000 * 1.05, read_gbs          # below the HBM peak, far above PCIe
    assert 100 < mfma_tflops < 2500 * 1.05, mfma_tflops    # below the bf16 peak


def test_stream_scope_holds_the_stream_that_is_current_when_it_opens(ops):
    """Inside a scope kernels go to the stream that was current at its start; a scope opened under another
    stream takes that one; leaving restores what was held before."""
    def held():
        return ops._stream().value or 0      # the default stream is the null handle

    main = torch.cuda.current_stream().cuda_stream
    side = torch.cuda.Stream()
    assert held() == main
    with ops.stream_scope():
        assert held() == main
        with torch.cuda.stream(side):
            assert held() == main          # the scope's stream, not torch's current one
            with ops.stream_scope():
                assert held() == side.cuda_stream
                x, gain = rnd((3, 64), 50).to(DEV), torch.ones(64, device=DEV)
                out = torch.empty((3, 64), device=DEV)
                ops.rmsnorm_rows(x, gain, 1e-6, out)    # launched on the side stream
            assert held() == main
        side.synchronize()
        want = torch.empty((3, 64))
        ref.rmsnorm_rows(x.cpu(), gain.cpu(), 1e-6, want)
        close(out, want, 1e-5, what="launched under a nested scope")
    assert held() == main
