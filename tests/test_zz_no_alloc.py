"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes as a foreign caller
would: decode attention whose partial results lie in the library's own device array, against the entry
point that takes a workspace, on two calls in a row, the second smaller; and its refusal of a call that
does not fit the array."""
import ctypes
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


def test_decode_attention_without_allocation_equals_the_one_with_a_workspace():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from synaptix_amd.kernels.build import load_library
    nh, nkv, hd = 8, 2, 64
    lib = load_library(f"attn_hd{hd}")              # a ctypes.CDLL
    lib.syn_attention_decode_bf16_noalloc.restype = ctypes.c_int
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = ctypes.c_float(1 / math.sqrt(hd))
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
        before = torch.cuda.memory_allocated()
        rc = lib.syn_attention_decode_bf16_noalloc(_p(q), _p(k), _p(v), _p(table), width, _p(seq_len), n, _p(got),
                                                   splits, scale, 0, nh, nkv, hd, stream)
        assert rc == 0, lib.syn_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want), f"{lens}: the two entry points differ by {(got.float() - want.float()).abs().max()}"
    # a call beyond the array: 8 MiB hold 2 Mi floats; 64 sequences x 8 heads x 64 splits x 66 do not fit
    rc = lib.syn_attention_decode_bf16_noalloc(_p(q), _p(k), _p(v), _p(table), width, _p(seq_len), 64, _p(got), 64,
                                               scale, 0, nh, nkv, hd, stream)
    assert rc != 0 and b"need" in lib.syn_last_error() and b"keeps" in lib.syn_last_error()
    torch.cuda.synchronize()
