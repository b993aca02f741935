// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory
// around a call: code that runs under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc.  Such a caller has nowhere to get the decode attention's workspace from (the
// partial results of the splits, which the merge kernel reads), so this variant keeps it in a
// file-scope device array of the library itself.
//
//   syn_attention_decode_bf16_noalloc: syn_attention_decode_bf16 without the workspace argument.
//
// Limits and rules:
//   * n_seqs * nh * n_splits * (hd + 2) floats must fit SYN_NOALLOC_SCRATCH_BYTES (8 MiB for each
//     GPU that the library runs on, held until the process ends); a larger call is refused with an
//     error text and launches nothing.
//   * The call allocates and frees nothing, on the device or through any library.  The address of
//     the array is looked up once per device (and the decode kernels' LDS limit raised there), by
//     syn_attention_decode_noalloc_init or else at the first call on that device.  Neither is stream
//     work and neither may happen while a stream is captured: a caller that captures calls the init
//     (or the entry point once) on that device beforehand.
//   * All calls on one GPU share that GPU's array, which keeps the last call's contents.  Nothing
//     in it has to start at zero: every split of every (sequence, head) writes its maximum, its sum
//     and its values before the merge reads them, an empty split writes a maximum of -inf.  Two
//     calls that overlap on one GPU (different streams, or different threads) race on it: callers
//     order them.
#pragma once
#include <hip/hip_runtime.h>

#define SYN_NOALLOC_SCRATCH_BYTES (8u << 20)

// 0, or a code after an error text (syn_last_error): with the device current, before any capture
extern "C" __attribute__((visibility("default"))) int syn_attention_decode_noalloc_init();

extern "C" __attribute__((visibility("default"))) int syn_attention_decode_bf16_noalloc(
    const void* q, const void* k_pages, const void* v_pages, const int* page_table, int table_stride,
    const int* seq_len, int n_seqs, void* out, int n_splits, float scale, int window, int nh, int nkv, int hd,
    hipStream_t stream);
