"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes as a foreign caller
would: decode attention whose partial results lie in the library's own device array, against the entry
point that takes a workspace, on two calls in a row, the second smaller; and its refusal of a call that
does not fit the array; and the same entry point recorded into a graph."""
import ctypes
import gc
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF16, F32, I32 = torch.bfloat16, torch.float32, torch.int32


def _inputs(n_seqs, lens, nh, nkv, hd, seed):
    g = torch.Generator().manual_seed(seed)
    width = max((t + 63) // 64 for t in lens) + 1
    n_pages = n_seqs * width
    table = torch.randperm(n_pages, generator=g).to(I32).view(n_seqs, width)
    k = torch.randn((n_pages, nkv, 64, hd), generator=g).to(BF16)
    v = torch.randn((n_pages, nkv, hd, 64), generator=g).to(BF16)     # any contents do: both entry points read the same
    q = torch.randn((n_seqs, nh * hd), generator=g).to(BF16)
    return [t.to(DEV) for t in (q, k, v, table, torch.tensor(lens, dtype=I32))], width


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _entry(hd):
    from synaptix_amd.kernels.build import load_library
    lib = load_library(f"attn_hd{hd}")              # a ctypes.CDLL
    lib.syn_attention_decode_bf16_noalloc.restype = ctypes.c_int
    lib.syn_attention_decode_noalloc_init.restype = ctypes.c_int
    return lib


def test_decode_attention_without_allocation_equals_the_one_with_a_workspace():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    nh, nkv, hd = 8, 2, 64
    lib = _entry(hd)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = ctypes.c_float(1 / math.sqrt(hd))
    # what a first call on a device does besides launching (the array's address, the kernels' LDS limit)
    assert lib.syn_attention_decode_noalloc_init() == 0, lib.syn_last_error()
    # two calls in a row on the same array: the first with more sequences, more splits and longer
    # contexts than the second, so that the second finds the first one's partial results beside its own
    for lens, splits in (([700, 130, 64, 1], 6), ([200, 3], 2)):
        n = len(lens)
        (q, k, v, table, seq_len), width = _inputs(n, lens, nh, nkv, hd, 11 + n)
        want = torch.full((n, nh * hd), float("nan"), dtype=BF16, device=DEV)
        got = torch.full((n, nh * hd), float("nan"), dtype=BF16, device=DEV)
        work = torch.empty(n * nh * splits * (hd + 2), dtype=F32, device=DEV)
        rc = lib.syn_attention_decode_bf16(_p(q), _p(k), _p(v), _p(table), width, _p(seq_len), n, _p(want), _p(work),
                                           splits, scale, 0, nh, nkv, hd, stream)
        assert rc == 0, lib.syn_last_error()
        torch.cuda.synchronize()
        # Free device memory as the driver counts it: any allocation in this process moves it, torch's or the
        # library's own.  Nothing else may free or allocate meanwhile: dead engines of earlier tests lie in
        # reference cycles, and a collection in the middle would give their tensors back.
        gc.collect()
        gc.disable()
        try:
            free_before = torch.cuda.mem_get_info()[0]
            rc = lib.syn_attention_decode_bf16_noalloc(_p(q), _p(k), _p(v), _p(table), width, _p(seq_len), n, _p(got),
                                                       splits, scale, 0, nh, nkv, hd, stream)
            torch.cuda.synchronize()
            free_after = torch.cuda.mem_get_info()[0]
        finally:
            gc.enable()
        assert rc == 0, lib.syn_last_error()
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want), f"{lens}: the two entry points differ by {(got.float() - want.float()).abs().max()}"
        assert free_after >= free_before, f"{lens}: {free_before - free_after} bytes of device memory were taken during the call"
    # a call beyond the array: 8 MiB hold 2 Mi floats; 64 sequences x 8 heads x 64 splits x 66 do not fit
    rc = lib.syn_attention_decode_bf16_noalloc(_p(q), _p(k), _p(v), _p(table), width, _p(seq_len), 64, _p(got), 64,
                                               scale, 0, nh, nkv, hd, stream)
    assert rc != 0 and b"need" in lib.syn_last_error() and b"keeps" in lib.syn_last_error()
    torch.cuda.synchronize()


def test_decode_attention_without_allocation_inside_a_captured_graph():
    """After the init call the entry point is stream work only: captured, replayed several times with eager work
    between the replays, and equal to the entry point with a workspace every time."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    nh, nkv, hd = 8, 2, 64
    lib = _entry(hd)
    assert lib.syn_attention_decode_noalloc_init() == 0, lib.syn_last_error()
    scale = ctypes.c_float(1 / math.sqrt(hd))
    lens, splits = [300, 70, 5], 3
    n = len(lens)
    (q, k, v, table, seq_len), width = _inputs(n, lens, nh, nkv, hd, 5)
    got = torch.zeros((n, nh * hd), dtype=BF16, device=DEV)
    want = torch.zeros_like(got)
    work = torch.empty(n * nh * splits * (hd + 2), dtype=F32, device=DEV)

    def with_workspace():
        s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.syn_attention_decode_bf16(_p(q), _p(k), _p(v), _p(table), width, _p(seq_len), n, _p(want), _p(work),
                                           splits, scale, 0, nh, nkv, hd, s)
        assert rc == 0, lib.syn_last_error()

    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()          # a finalizer that frees device memory is refused while a stream is captured
    try:
        with torch.cuda.graph(graph):
            s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            rc = lib.syn_attention_decode_bf16_noalloc(_p(q), _p(k), _p(v), _p(table), width, _p(seq_len), n, _p(got),
                                                       splits, scale, 0, nh, nkv, hd, s)
    finally:
        gc.enable()
    assert rc == 0, lib.syn_last_error()
    for turn in range(3):
        q.copy_(torch.randn(q.shape, generator=torch.Generator().manual_seed(turn)).to(BF16))   # eager work between replays
        with_workspace()
        got.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {turn}: differs by {(got.float() - want.float()).abs().max()}"
