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

// ------------------------------------------------------------------ the processors in front of the sampler
// One workgroup a row of logits, in the reference's order (crates/synaptix-models/llm/common/src/generate.rs:304-340):
//   repetition penalty   once for each occurrence of a token in the row's list: a positive logit is divided,
//                        any other multiplied (crates/synaptix-infer/src/sampling/repetition.rs:27-45)
//   presence, frequency  logit -= presence + frequency * occurrences (repetition.rs:59-77)
//   temperature          logit /= T where T > 0 and T != 1 (logit_processor.rs:8-18)
//   top-k                the k largest stay (sampling/top_k.rs:8-24; of equal values at the k-th place the
//                        first in index order, where the reference's selection keeps arbitrary ones)
//   top-p                sorted by probability, a candidate stays while the sum of those before it is at most
//                        p * the sum of all (sampling/top_p.rs:8-44; equal probabilities in index order)
//   min-p                those below min_p * the largest probability go (sampling/min_p.rs:8-24)
// What is dropped becomes -inf.  The reference sorts on the host; here the k-th value and the boundary of the
// probability mass are found by selection on the float's bit pattern, a byte at a time from the top (four
// passes over the row with a histogram of 256 bins in LDS), and the sums are integers (probabilities in 44-bit
// fixed point), so that a row gives the same result whatever the order in which threads arrive.
#define FILTER_THREADS 1024
#define FILTER_LIST 2048
typedef unsigned long long u64;

// the float's bits as an unsigned number that grows with the float
__device__ __forceinline__ unsigned order_key(float x) {
  const unsigned b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ bool is_finite(float x) { return x > -INFINITY && x < INFINITY; }
__device__ __forceinline__ u64 mass_of(float x, float m) { return (u64)(expf(x - m) * 17592186044416.f); }   // * 2^44: up to 2^20 entries

struct FilterShared {
  unsigned cnt[256];
  u64 sum[256];
  u64 red64[FILTER_THREADS / SYN_WAVE];
  float redf[FILTER_THREADS / SYN_WAVE];
  int wave_n[FILTER_THREADS / SYN_WAVE];
  int bin;
  unsigned need;
  u64 above;
  // what top-k has left, if that is little: the processors behind it then walk this list, not the row
  int cand_j[FILTER_LIST];
  int n_cand;
};

__device__ __forceinline__ float block_max_all(float v, float* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, SYN_WAVE));
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, nw = blockDim.x / SYN_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = red[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
  return t;
}
__device__ __forceinline__ u64 block_sum_all(u64 v, u64* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, SYN_WAVE);
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, nw = blockDim.x / SYN_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  u64 t = 0;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}

// For the lanes of one wave, lane l holding bins 4 l .. 4 l + 3 of a histogram: above[i] = the sum of all bins above
// bin 4 l + i.
template <typename T>
__device__ __forceinline__ void sums_above(const T* hist, int lane, T (&mine)[4], T (&above)[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) mine[i] = hist[4 * lane + i];
  const T own = mine[0] + mine[1] + mine[2] + mine[3];
  T from_here = own;   // becomes the sum over this lane and all higher ones
#pragma unroll
  for (int off = 1; off < SYN_WAVE; off <<= 1) {
    const T o = __shfl_down(from_here, off, SYN_WAVE);
    if (lane + off < SYN_WAVE) from_here += o;
  }
  above[3] = from_here - own;
  above[2] = above[3] + mine[3];
  above[1] = above[2] + mine[2];
  above[0] = above[1] + mine[1];
}

// A thread's additions to the histogram go through one bin kept in registers: logits share their top bytes, and
// a thousand threads adding to the same few LDS words one by one would take longer than the pass itself.
struct BinCache {
  int bin = -1;
  unsigned n = 0;
  u64 s = 0;
  __device__ __forceinline__ void flush(FilterShared& sh, bool with_sums) {
    if (n) {
      atomicAdd(&sh.cnt[bin], n);
      if (with_sums) atomicAdd(&sh.sum[bin], s);
    }
    n = 0, s = 0;
  }
  __device__ __forceinline__ void add(FilterShared& sh, int b, u64 mass, bool with_sums) {
    if (b != bin) {
      flush(sh, with_sums);
      bin = b;
    }
    ++n, s += mass;
  }
};

// A pass over a row: f(j, x[j]) for every entry, 16 bytes a load and eight loads of a thread under way where the row
// allows it (one entry at a time, a pass of one workgroup over 150,000 entries waits 150 times for memory).
template <typename F>
__device__ __forceinline__ void for_each_entry(const float* x, int V, F f) {
  const int tid = threadIdx.x, nt = blockDim.x;
  if (V % 4 == 0 && (uintptr_t)x % 16 == 0) {
    const float4* x4 = (const float4*)x;
    const int V4 = V / 4;
    for (int i0 = tid; i0 < V4; i0 += 8 * nt) {
      float4 v[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) v[q] = i0 + q * nt < V4 ? x4[i0 + q * nt] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int q = 0; q < 8; ++q)
        if (i0 + q * nt < V4) {
          const int j = 4 * (i0 + q * nt);
          f(j, v[q].x), f(j + 1, v[q].y), f(j + 2, v[q].z), f(j + 3, v[q].w);
        }
    }
  } else {
    for (int j = tid; j < V; j += nt) f(j, x[j]);
  }
}
// The same with a new value for every entry: dst[j] = f(j, src[j]) (dst may be src).
template <typename F>
__device__ __forceinline__ void map_entries(const float* src, float* dst, int V, F f) {
  const int tid = threadIdx.x, nt = blockDim.x;
  if (V % 4 == 0 && (uintptr_t)src % 16 == 0 && (uintptr_t)dst % 16 == 0) {
    const float4* s4 = (const float4*)src;
    float4* d4 = (float4*)dst;
    const int V4 = V / 4;
    for (int i0 = tid; i0 < V4; i0 += 4 * nt) {
      float4 v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = i0 + q * nt < V4 ? s4[i0 + q * nt] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (i0 + q * nt < V4) {
          const int j = 4 * (i0 + q * nt);
          d4[i0 + q * nt] = make_float4(f(j, v[q].x), f(j + 1, v[q].y), f(j + 2, v[q].z), f(j + 3, v[q].w));
        }
    }
  } else {
    for (int j = tid; j < V; j += nt) dst[j] = f(j, src[j]);
  }
}

// Of the entries whose key is `key`, those from the keep-th on in index order become -inf.
__device__ void drop_later_ties(float* x, int V, unsigned key, unsigned keep, FilterShared& sh) {
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE, nw = blockDim.x / SYN_WAVE;
  unsigned before = 0;   // ties in earlier chunks; the same in every thread
  for (int base = 0; base < V; base += blockDim.x) {
    const int j = base + tid;
    const bool tie = j < V && order_key(x[j]) == key;
    const u64 votes = __ballot(tie);
    __syncthreads();
    if (lane == 0) sh.wave_n[wave] = __popcll(votes);
    __syncthreads();
    unsigned rank = before + __popcll(votes & ((1ull << lane) - 1ull)), all = 0;
    for (int w = 0; w < nw; ++w) {
      if (w < wave) rank += sh.wave_n[w];
      all += sh.wave_n[w];
    }
    if (tie && rank >= keep) x[j] = -INFINITY;
    before += all;
  }
  __syncthreads();
}

__global__ void __launch_bounds__(FILTER_THREADS)
filter_rows_kernel(const float* __restrict__ in, float* __restrict__ out, int V, const float* __restrict__ temperature,
                   const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ min_p,
                   const float* __restrict__ repetition, const float* __restrict__ presence,
                   const float* __restrict__ frequency, const int* __restrict__ ids, const int* __restrict__ id_start,
                   int* __restrict__ counts) {
  __shared__ FilterShared sh;
  const int row = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  float* x = out + (size_t)row * V;
  const float* src = in + (size_t)row * V;    // the row as it comes, until the first pass that writes has copied it

  // ---- penalties: occurrences counted in the row's scratch counters, which are zero before and after
  const int n_ids = id_start ? id_start[row + 1] - id_start[row] : 0;
  const float rep = repetition[row], pres = presence[row], freq = frequency[row];
  if (n_ids > 0 && (rep != 1.f || pres != 0.f || freq != 0.f)) {
    if (src != x) {
      map_entries(src, x, V, [](int, float v) { return v; });
      src = x;
      __syncthreads();
    }
    int* cnt = counts + (size_t)row * V;
    const int* mine = ids + id_start[row];
    for (int i = tid; i < n_ids; i += nt) {
      const int t = mine[i];
      if (t >= 0 && t < V) atomicAdd(&cnt[t], 1);
    }
    __syncthreads();
    for (int i = tid; i < n_ids; i += nt) {
      const int t = mine[i];
      if (t < 0 || t >= V) continue;
      const int c = __hip_atomic_load(&cnt[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (c > 0 && atomicCAS(&cnt[t], c, -c) == c) {   // one of the token's occurrences does the work
        float v = x[t];
        if (rep != 1.f) {
          const float f = powf(rep, (float)c);
          v = v > 0.f ? v / f : v * f;
        }
        if (pres != 0.f || freq != 0.f) v -= pres + freq * (float)c;
        x[t] = v;
      }
    }
    __syncthreads();
    for (int i = tid; i < n_ids; i += nt) {
      const int t = mine[i];
      if (t >= 0 && t < V) cnt[t] = 0;
    }
    __syncthreads();
  }

  // ---- temperature, and the largest logit (which every later step keeps)
  const float T = temperature[row];
  const bool scale = T > 0.f && T != 1.f;
  float m = -INFINITY;
  if (scale || src != x) {
    map_entries(src, x, V, [&](int, float v) {
      if (scale) v = v / T;
      m = fmaxf(m, v);
      return v;
    });
  } else {
    for_each_entry(x, V, [&](int, float v) { m = fmaxf(m, v); });
  }
  m = block_max_all(m, sh.redf);   // (its barriers also stand between the writes above and the reads below)

  // ---- top-k: the key of the k-th largest, a byte at a time
  const int k = top_k[row];
  bool listed = false;
  if (k > 0 && k < V) {
    unsigned prefix = 0, need = (unsigned)k, ties = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
      const unsigned himask = shift == 24 ? 0u : 0xffffffffu << (shift + 8);
      for (int b = tid; b < 256; b += nt) sh.cnt[b] = 0;
      __syncthreads();
      BinCache cache;
      for_each_entry(x, V, [&](int, float v) {
        const unsigned key = order_key(v);
        if ((key & himask) == prefix) cache.add(sh, (key >> shift) & 255, 0, false);
      });
      cache.flush(sh, false);
      __syncthreads();
      if (tid < SYN_WAVE) {
        // the bin in which the need-th largest of the matching entries lies (there are at least `need` of them)
        unsigned mine[4], above[4];
        sums_above(sh.cnt, tid, mine, above);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (above[i] < need && need <= above[i] + mine[i]) sh.bin = 4 * tid + i, sh.need = need - above[i];
      }
      __syncthreads();
      prefix |= (unsigned)sh.bin << shift, need = sh.need, ties = sh.cnt[sh.bin];
      __syncthreads();
    }
    // below the k-th key everything goes; of its equals the first `need` stay.  If processors follow and little is
    // left, what stays is listed in LDS (in no order) for them.
    const bool list = (top_p[row] < 1.f || min_p[row] > 0.f) && (unsigned)k - need + ties <= FILTER_LIST;
    if (tid == 0) sh.n_cand = 0;
    __syncthreads();
    map_entries(x, x, V, [&](int j, float v) {
      if (order_key(v) < prefix) return -INFINITY;
      if (list) {
        const int i = atomicAdd(&sh.n_cand, 1);
        sh.cand_j[i] = j;
      }
      return v;
    });
    __syncthreads();
    if (need < ties) drop_later_ties(x, V, prefix, need, sh);
    listed = list;
  }
  // a pass over what is left: f(j, value) for the listed entries or for the whole row
  const int n_listed = listed ? sh.n_cand : 0;
  auto each_left = [&](auto f) {
    if (listed) {
      for (int i = tid; i < n_listed; i += nt) f(sh.cand_j[i], x[sh.cand_j[i]]);
    } else {
      for_each_entry(x, V, f);
    }
  };
  auto drop_left = [&](auto gone) {   // gone(value): whether the entry goes
    if (listed) {
      for (int i = tid; i < n_listed; i += nt) {
        const int j = sh.cand_j[i];
        if (gone(x[j])) x[j] = -INFINITY;
      }
    } else {
      map_entries(x, x, V, [&](int, float v) { return gone(v) ? -INFINITY : v; });
    }
  };

  // ---- top-p: the lowest key whose mass above it is at most p * all mass
  const float p = top_p[row], mp = min_p[row];
  bool min_p_done = false;
  if (p < 1.f) {
    u64 limit = 0;       // p * all mass; all mass is what the first histogram adds up to
    unsigned prefix = 0, ties = 0;
    u64 above = 0, tie_mass = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
      const unsigned himask = shift == 24 ? 0u : 0xffffffffu << (shift + 8);
      for (int b = tid; b < 256; b += nt) sh.cnt[b] = 0, sh.sum[b] = 0;
      __syncthreads();
      BinCache cache;
      each_left([&](int, float v) {
        if (!is_finite(v)) return;
        const unsigned key = order_key(v);
        if ((key & himask) == prefix) cache.add(sh, (key >> shift) & 255, mass_of(v, m), true);
      });
      cache.flush(sh, true);
      __syncthreads();
      if (tid < SYN_WAVE) {
        // a bin's largest entry has exactly the mass of the bins above it before it: the lowest bin that holds
        // entries and has at most `limit` above it is where the boundary lies (every such bin above it stays whole)
        u64 mine[4], over[4];
        sums_above(sh.sum, tid, mine, over);
        if (shift == 24) {
          const u64 total = __shfl(over[0] + mine[0], 0, SYN_WAVE);
          limit = (u64)((double)p * (double)total);
          if (tid == 0) sh.red64[0] = limit;
        }
        int lowest = 256;
#pragma unroll
        for (int i = 3; i >= 0; --i)
          if (sh.cnt[4 * tid + i] && above + over[i] <= limit) lowest = 4 * tid + i;
        int first = lowest;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) first = min(first, __shfl_xor(first, off, SYN_WAVE));
        if (first == 256) {
          if (tid == 0) sh.bin = -1;
        } else if (first == lowest) {
          sh.bin = first, sh.above = above + over[first % 4];
        }
      }
      __syncthreads();
      if (sh.bin < 0) break;   // no finite entry at all
      limit = sh.red64[0];
      prefix |= (unsigned)sh.bin << shift, above = sh.above, ties = sh.cnt[sh.bin], tie_mass = sh.sum[sh.bin];
      __syncthreads();
    }
    if (ties > 0) {
      // (min-p looks at each entry alone, so it goes along in this pass)
      drop_left([&](float v) { return is_finite(v) && (order_key(v) < prefix || (mp > 0.f && expf(v - m) < mp)); });
      min_p_done = true;
      __syncthreads();
      // the j-th of equal entries has (j - 1) of them before it as well
      const u64 each = tie_mass / ties;
      const u64 keep = each == 0 ? (u64)ties : (limit - above) / each + 1;
      if (keep < ties) drop_later_ties(x, V, prefix, (unsigned)keep, sh);
    }
  }

  // ---- min-p: the largest probability belongs to the largest logit, exp(0) = 1 before the division by the sum
  if (mp > 0.f && !min_p_done) drop_left([&](float v) { return is_finite(v) && expf(v - m) < mp; });
}

// in, out [n_rows, V] float (may be the same); one entry a row of every option (top_k 0 and top_p >= 1: off);
// ids, id_start [n_rows + 1]: the tokens that the penalties look at, row after row (null: none);
// counts [n_rows * V] int, zero (needed with ids; the kernel leaves them zero)
SYN_EXPORT int syn_filter_rows(const float* in, float* out, int n_rows, int V, const float* temperature, const int* top_k,
                               const float* top_p, const float* min_p, const float* repetition, const float* presence,
                               const float* frequency, const int* ids, const int* id_start, int* counts,
                               hipStream_t stream) {
  SYN_CHECK(n_rows > 0 && V > 0 && V <= (1 << 20), "filter_rows: %d rows, vocabulary %d (1 .. 2^20)", n_rows, V);
  SYN_CHECK(in && out && temperature && top_k && top_p && min_p && repetition && presence && frequency,
            "filter_rows: an option array is missing");
  SYN_CHECK((ids == nullptr) == (id_start == nullptr) && (ids == nullptr || counts != nullptr),
            "filter_rows: the penalties' tokens come with their row offsets and with counters");
  filter_rows_kernel<<<n_rows, FILTER_THREADS, 0, stream>>>(in, out, V, temperature, top_k, top_p, min_p, repetition,
                                                            presence, frequency, ids, id_start, counts);
  SYN_LAUNCH_CHECK("filter_rows");
  return 0;
}
