"""The kernels' plain C++ twins (synaptix_amd/csrc/ref/ref_kernels.cpp): on the CPU against the plain
Python statement of the same formulas (tests/plain_qwen3.py), and, marked gpu, the HIP kernels in
32-bit against the twins: three statements of every operation, written independently."""
import math

import pytest
import torch

import plain_qwen3 as P

F32, I32 = torch.float32, torch.int32


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


@pytest.fixture(scope="module")
def twins():
    from synaptix_amd.kernels import ref
    return ref


def paged(nkv, hd, lens, seed):
    """Pages [n, nkv, 64, hd] / [n, nkv, hd, 64] in a shuffled table, and the keys and values they hold."""
    width = max((t + 63) // 64 for t in lens) + 1
    n_pages = len(lens) * width
    table = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).to(I32).view(len(lens), width)
    k = torch.full((n_pages, nkv, 64, hd), 1e9)
    v = torch.full((n_pages, nkv, hd, 64), 1e9)           # whatever is read beyond a sequence's end shows
    keys, vals = [], []
    for b, T in enumerate(lens):
        kk, vv = rnd((T, nkv, hd), seed + 2 * b + 1), rnd((T, nkv, hd), seed + 2 * b + 2)
        keys.append(kk), vals.append(vv)
        for t in range(T):
            k[int(table[b, t // 64]), :, t % 64, :] = kk[t]
            v[int(table[b, t // 64]), :, :, t % 64] = vv[t]
    return table, k, v, keys, vals


def test_rows(twins):
    table, ids = rnd((50, 24), 1), torch.tensor([3, 49, 0, 3], dtype=I32)
    out = torch.empty(4, 24)
    twins.embed(table, ids, out)
    assert torch.equal(out, P.embed(table, ids.tolist()))
    resid, delta, gain = rnd((5, 72), 2), rnd((5, 72), 3), 0.1 * rnd((72,), 4)
    for offset in (0.0, 1.0):
        r, o = resid.clone(), torch.empty(5, 72)
        twins.add_rmsnorm(r, delta, gain, 1e-5, o, gain_offset=offset)
        assert torch.allclose(r, resid + delta, atol=1e-6)
        assert torch.allclose(o, P.rms_norm(resid + delta, offset + gain, 1e-5), atol=1e-5)
    o = torch.empty(1, 4)
    twins.add_rmsnorm(torch.tensor([[-1.0, -0.9, -0.8, -0.7]]), None, torch.tensor([0.5, -0.25, 1.0, 2.0]), 1e-6, o)
    r = 1 / math.sqrt(0.735 + 1e-6)          # the first row of crates/synaptix-ops/tests/rms_norm.rs:76-95
    assert torch.allclose(o[0], torch.tensor([-0.5 * r, 0.9 * r * 0.25, -0.8 * r, -1.4 * r]), atol=1e-6)
    gu, o = rnd((3, 20), 5), torch.empty(3, 10)
    twins.swiglu(gu, o)
    assert torch.allclose(o, P.silu(gu[:, :10]) * gu[:, 10:], atol=1e-6)
    x, w, o = rnd((7, 33), 6), rnd((11, 33), 7), torch.empty(7, 11)
    twins.gemm(x, w, o)
    assert torch.allclose(o, x @ w.T, atol=1e-5)


@pytest.mark.parametrize("nh,nkv,hd,rot,norm", [(4, 2, 16, 16, True), (6, 3, 48, 32, True), (2, 1, 32, 0, False)])
def test_heads_and_attention(twins, nh, nkv, hd, rot, norm):
    """q/k norm, rotation, cache write and attention of the twins against the plain formulas: a prompt of
    70 tokens behind 30 cached ones, in a shuffled page table."""
    past, new = 30, 70
    T = past + new
    table, k, v, keys, vals = paged(nkv, hd, [T], 10)
    qkv = rnd((new, (nh + 2 * nkv) * hd), 20)
    qg, kg = (1 + 0.2 * rnd((hd,), 21), 1 + 0.2 * rnd((hd,), 22)) if norm else (None, None)
    cos = sin = None
    if rot:
        cos, sin = P.rope_tables(rot, T, 1e4)
    pos = torch.arange(past, T, dtype=I32)
    q_out = torch.empty(new, nh * hd)
    twins.qk_norm_rope_kv_write(qkv, q_out, k, v, table, torch.zeros(new, dtype=I32), pos, qg, kg, 1e-5, cos, sin, nh, nkv, hd)
    x = qkv.view(new, nh + 2 * nkv, hd)
    q, kn, vn = x[:, :nh], x[:, nh:nh + nkv], x[:, nh + nkv:]
    if norm:
        q, kn = P.rms_norm(q, qg, 1e-5), P.rms_norm(kn, kg, 1e-5)
    if rot:
        turn = lambda t: torch.cat([P.apply_rope(t[..., :rot], cos, sin, pos.tolist()), t[..., rot:]], -1)
        q, kn = turn(q), turn(kn)
    assert torch.allclose(q_out.view(new, nh, hd), q, atol=1e-5)
    all_k, all_v = torch.cat([keys[0][:past], kn]), torch.cat([vals[0][:past], vn])
    for t in (past, T - 1):
        page = int(table[0, t // 64])
        assert torch.allclose(k[page, :, t % 64, :], all_k[t], atol=1e-5) and torch.allclose(v[page, :, :, t % 64], all_v[t])
    for window in (0, 37):
        out = torch.empty(new, nh * hd)
        twins.attention(q_out, k, v, table, torch.zeros(new, dtype=I32), pos, out, 0.3, window, nh, nkv, hd)
        want = P.attention(q, all_k, all_v, 0.3, pos.tolist(), window or None)
        assert torch.allclose(out.view(new, nh, hd), want, atol=1e-5)


def test_sampling(twins):
    logits = torch.tensor([[1.0, 3.0, 2.0, 3.0, 0.0], [5.0, 3.0, 1.0, 0.0, -1.0]])
    out = torch.empty(2, dtype=I32)
    twins.sample_rows(logits, None, None, out)
    assert out.tolist() == [P.greedy(logits[0]), P.greedy(logits[1])] == [3, 0]
    x = rnd((6, 50), 30)
    temps = torch.tensor([0.7, 0.0, 1.0, 2.0, 0.3, 1.0])
    us = torch.tensor([0.0, 0.5, 0.999999, 0.37, 0.81, 1.0])
    out = torch.empty(6, dtype=I32)
    twins.sample_rows(x, temps, us, out)
    for r in range(6):
        want = P.greedy(x[r]) if temps[r] <= 0 else P.multinomial(x[r] / temps[r], float(us[r]))
        assert int(out[r]) == want


@pytest.mark.gpu
def test_hip_kernels_in_32_bit_equal_their_twins(twins):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from synaptix_amd.kernels import ops
    dev = "cuda:0"
    d = lambda t: None if t is None else t.to(dev)
    # rows
    table, ids = rnd((300, 136), 40), torch.tensor([5, 299, 0, 17, 5], dtype=I32)
    want, got = torch.empty(5, 136), torch.empty(5, 136, device=dev)
    twins.embed(table, ids, want)
    ops.embed(d(table), d(ids), got)
    assert torch.equal(got.cpu(), want)
    resid, delta, gain = rnd((6, 1000), 41), rnd((6, 1000), 42), 1 + 0.1 * rnd((1000,), 43)
    r_cpu, want = resid.clone(), torch.empty(6, 1000)
    twins.add_rmsnorm(r_cpu, delta, gain, 1e-6, want)
    r_gpu, got = d(resid), torch.empty(6, 1000, device=dev)
    ops.add_rmsnorm(r_gpu, d(delta), d(gain), 1e-6, got)
    assert torch.allclose(r_gpu.cpu(), r_cpu, atol=1e-6) and torch.allclose(got.cpu(), want, atol=1e-5)
    gu, want, got = rnd((4, 2 * 90), 44), torch.empty(4, 90), torch.empty(4, 90, device=dev)
    twins.swiglu(gu, want)
    ops.swiglu(d(gu), got)
    assert torch.allclose(got.cpu(), want, atol=1e-6)
    x, w = rnd((70, 100), 45), rnd((130, 100), 46)
    want, got = torch.empty(70, 130), torch.empty(70, 130, device=dev)
    twins.gemm(x, w, want)
    ops.gemm(d(x), d(w), got)
    assert torch.allclose(got.cpu(), want, atol=1e-4)
    # heads, cache write and attention: two sequences, one with cached tokens, a window
    nh, nkv, hd, rot = 6, 2, 48, 32
    past, new = [0, 40], [70, 3]
    lens = [p + n for p, n in zip(past, new)]
    table, k, v, _, _ = paged(nkv, hd, lens, 50)
    N = sum(new)
    tok_seq = torch.tensor([0] * new[0] + [1] * new[1], dtype=I32)
    tok_pos = torch.tensor(list(range(new[0])) + list(range(past[1], lens[1])), dtype=I32)
    qkv = rnd((N, (nh + 2 * nkv) * hd), 51)
    qg, kg = 1 + 0.2 * rnd((hd,), 52), 1 + 0.2 * rnd((hd,), 53)
    cos, sin = P.rope_tables(rot, max(lens), 1e4)
    k_cpu, v_cpu, q_cpu = k.clone(), v.clone(), torch.empty(N, nh * hd)
    twins.qk_norm_rope_kv_write(qkv, q_cpu, k_cpu, v_cpu, table, tok_seq, tok_pos, qg, kg, 1e-5, cos, sin, nh, nkv, hd)
    k_gpu, v_gpu, q_gpu = d(k), d(v), torch.empty(N, nh * hd, device=dev)
    ops.qk_norm_rope_kv_write(d(qkv), q_gpu, k_gpu, v_gpu, d(table), d(tok_seq), d(tok_pos), d(qg), d(kg), 1e-5, d(cos),
                              d(sin), nh, nkv, hd)
    assert torch.allclose(q_gpu.cpu(), q_cpu, atol=1e-5)
    assert torch.allclose(k_gpu.cpu(), k_cpu, atol=1e-5) and torch.allclose(v_gpu.cpu(), v_cpu, atol=1e-6)
    for window in (0, 50):
        want, got = torch.empty(N, nh * hd), torch.empty(N, nh * hd, device=dev)
        twins.attention(q_cpu, k_cpu, v_cpu, table, tok_seq, tok_pos, want, 0.2, window, nh, nkv, hd)
        ops.attention_f32(q_gpu, k_gpu, v_gpu, d(table), d(tok_seq), d(tok_pos), got, 0.2, window, nh, nkv, hd)
        assert torch.allclose(got.cpu(), want, atol=1e-5)
    # sampling
    logits = rnd((5, 999), 54, 3.0)
    temps, us = torch.tensor([0.0, 0.8, 1.0, 0.0, 1.5]), torch.tensor([0.0, 0.3, 0.77, 0.0, 0.05])
    want, got = torch.empty(5, dtype=I32), torch.empty(5, dtype=I32, device=dev)
    twins.sample_rows(logits, temps, us, want)
    ops.sample_rows(d(logits), d(temps), d(us), got)
    assert got.cpu().tolist() == want.tolist()
