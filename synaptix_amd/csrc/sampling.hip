// Sampling on the device: one block a row of logits [rows, V] (32-bit).
//   temperature <= 0: argmax, the last of equal maxima
//                     (crates/synaptix-infer/src/sampling/greedy.rs:7-13: Rust's max_by keeps the last)
//   temperature  > 0: x = logit / T (skipped for T == 1), p = softmax(x), the first i with u < cumsum_i,
//                     else the last index (crates/synaptix-infer/src/sampling/multinomial.rs:7-28,
//                     logit_processor.rs:8-18)
// The uniform number u comes from the host (a Philox stream per sequence).
// The reference samples on the host from a downloaded vector; the arithmetic is the same,
// only the order of the two sums differs (parallel instead of sequential).
#include "common.h"

#define SAMPLE_THREADS 1024

struct ArgBest {
  float v;
  int i;
};

__device__ __forceinline__ ArgBest arg_better(ArgBest a, ArgBest b) {
  // larger value wins; of equal values the larger index wins
  if (b.v > a.v || (b.v == a.v && b.i > a.i)) return b;
  return a;
}

__device__ __forceinline__ ArgBest block_argmax(ArgBest best, ArgBest* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    ArgBest o;
    o.v = __shfl_xor(best.v, off, SYN_WAVE);
    o.i = __shfl_xor(best.i, off, SYN_WAVE);
    best = arg_better(best, o);
  }
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, nw = blockDim.x / SYN_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = best;
  __syncthreads();
  ArgBest r = red[0];
  for (int w = 1; w < nw; ++w) r = arg_better(r, red[w]);
  return r;
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_rows_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                   const float* __restrict__ uniform, int* __restrict__ out, int V) {
  __shared__ ArgBest red_arg[16];
  __shared__ float red[16];
  __shared__ float chunk_sum[SAMPLE_THREADS];
  __shared__ int found[16];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * V;
  const float T = temperature ? temperature[row] : 0.f;

  ArgBest best = {-INFINITY, -1};
  if (V % 4 == 0 && (uintptr_t)logits % 16 == 0) {
    // 16-byte loads, four of them in flight: the row is read once, at memory speed
    const float4* x4 = (const float4*)x;
    const int V4 = V / 4, step = blockDim.x;
    for (int i0 = tid; i0 < V4; i0 += 4 * step) {
      float4 v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
        v[q] = i0 + q * step < V4 ? x4[i0 + q * step] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int i = 4 * (i0 + q * step);
        if (i0 + q * step < V4) {
          best = arg_better(best, ArgBest{v[q].x, i});
          best = arg_better(best, ArgBest{v[q].y, i + 1});
          best = arg_better(best, ArgBest{v[q].z, i + 2});
          best = arg_better(best, ArgBest{v[q].w, i + 3});
        }
      }
    }
  } else {
    for (int i = tid; i < V; i += blockDim.x) {
      ArgBest c = {x[i], i};
      best = arg_better(best, c);
    }
  }
  best = block_argmax(best, red_arg);
  if (!(T > 0.f)) {
    if (tid == 0) out[row] = best.i < 0 ? V - 1 : best.i;
    return;
  }
  const bool scale = T != 1.f;
  const float m = scale ? best.v / T : best.v;  // T > 0: the largest logit stays the largest

  // each thread owns one contiguous chunk, so that prefix sums follow the index order
  const int per = (V + blockDim.x - 1) / blockDim.x;
  const int lo = tid * per, hi = min(V, lo + per);
  float s = 0.f;
  for (int i = lo; i < hi; ++i) s += expf((scale ? x[i] / T : x[i]) - m);
  const float total = block_sum(s, red);
  float ps = 0.f;
  for (int i = lo; i < hi; ++i) ps += expf((scale ? x[i] / T : x[i]) - m) / total;
  chunk_sum[tid] = ps;
  __syncthreads();
  float prefix = 0.f;
  for (int t = 0; t < tid; ++t) prefix += chunk_sum[t];
  const float u = uniform[row];
  int hit = V;  // none
  float c = prefix;
  for (int i = lo; i < hi; ++i) {
    c += expf((scale ? x[i] / T : x[i]) - m) / total;
    if (u < c) {
      hit = i;
      break;
    }
  }
  // smallest hit of the block
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) hit = min(hit, __shfl_xor(hit, off, SYN_WAVE));
  if (tid % SYN_WAVE == 0) found[tid / SYN_WAVE] = hit;
  __syncthreads();
  if (tid == 0) {
    int r = V;
    for (int w = 0; w < (int)blockDim.x / SYN_WAVE; ++w) r = min(r, found[w]);
    out[row] = r >= V ? V - 1 : r;
  }
}

SYN_EXPORT int syn_sample_rows(const float* logits, const float* temperature, const float* uniform, int* out,
                               int n_rows, int V, hipStream_t stream) {
  SYN_CHECK(n_rows > 0 && V > 0, "sample_rows: empty input (%d rows, vocabulary %d)", n_rows, V);
  SYN_CHECK(temperature == nullptr || uniform != nullptr, "sample_rows: temperatures need uniform numbers");
  sample_rows_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, temperature, uniform, out, V);
  SYN_LAUNCH_CHECK("sample_rows");
  return 0;
}
