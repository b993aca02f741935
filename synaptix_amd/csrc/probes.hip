// Two measurements of what this machine gives, against which the kernels' rates are reported beside
// the vendor's peaks: how fast a kernel that does nothing else reads memory, and how fast the
// matrix units multiply when nothing feeds them from memory.
#include "common.h"

// every workgroup streams its own contiguous piece with 16-byte non-temporal loads, four in flight a lane
__global__ void __launch_bounds__(256)
probe_read_kernel(const f32x4* __restrict__ src, size_t n_vec, int* __restrict__ sink) {
  const size_t per = (n_vec + gridDim.x - 1) / gridDim.x;
  const size_t lo = per * blockIdx.x, hi = lo + per < n_vec ? lo + per : n_vec;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (size_t i = lo + threadIdx.x; i < hi; i += 4 * 256) {
    f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      v[u] = i + u * 256 < hi ? __builtin_nontemporal_load(src + i + u * 256) : (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 4; ++u) acc += v[u];
  }
  if (acc[0] + acc[1] + acc[2] + acc[3] == 1.2345678f) sink[0] = 1;  // keeps the loads alive
}

// bytes: a multiple of 16.  One pass over the buffer.
SYN_EXPORT int syn_probe_read(const void* src, size_t bytes, int* sink, hipStream_t stream) {
  SYN_CHECK(bytes >= 16 && bytes % 16 == 0 && (uintptr_t)src % 16 == 0, "probe_read: %zu bytes", bytes);
  probe_read_kernel<<<256 * 16, 256, 0, stream>>>((const f32x4*)src, bytes / 16, sink);
  SYN_LAUNCH_CHECK("probe_read");
  return 0;
}

// four independent accumulation chains of v_mfma_f32_32x32x16_bf16 a wave, operands in registers
__global__ void __launch_bounds__(256)
probe_mfma_kernel(int iters, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) a[e] = (bf16)(0.001f * (threadIdx.x % 7 + e)), b[e] = (bf16)(0.002f * (threadIdx.x % 5 + e));
  f32x16 acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[c][e] = 0.f;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) s += acc[c][0];
  if (s == 1.2345678f) sink[0] = s;
}

// flops of the launch: workgroups * 4 waves * iters * 4 chains * 2 * 32 * 32 * 16
SYN_EXPORT int syn_probe_mfma(int workgroups, int iters, float* sink, hipStream_t stream) {
  SYN_CHECK(workgroups > 0 && iters > 0, "probe_mfma: empty launch");
  probe_mfma_kernel<<<workgroups, 256, 0, stream>>>(iters, sink);
  SYN_LAUNCH_CHECK("probe_mfma");
  return 0;
}
