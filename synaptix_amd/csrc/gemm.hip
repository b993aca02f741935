// out[M, N] = x[M, K] . W[N, K]^T with 32-bit accumulation (both operands K-contiguous).
//
//   gemm_simt      any shape and type; plain FMA.  The whole 32-bit path, and bf16 shapes that
//                  the MFMA kernels refuse (K not a multiple of 8, unaligned rows).
//   gemm_skinny    bf16, M == 1: the weight matrix is streamed once from HBM through
//                  v_mfma_f32_16x16x32_bf16; the waves of a workgroup split K and sum in LDS
//                  (also over paired gate/up rows, with the gated activation as the epilogue).
//   gemm_packed    bf16, M <= 16 (used up to 8): the same over a copy of W kept in the order of the MFMA
//                  fragments, so that every load of a wave is 1 KB of consecutive bytes.
//   gemm_tiled     bf16: tiles of x and W in LDS, double-buffered, v_mfma_f32_32x32x16_bf16.
//                  M > 64: 256x256x64, 256x192x64 or 128x128x64 tiles; when K is a multiple of 64 by
//                  gemm_pipelined, whose loads write LDS without passing through registers and are
//                  issued, like the fragment reads, one behind each MFMA.
//                  M <= 64: 32 or 64 rows of x, 64 (or 32) rows of W, 128 (or 256) deep: the rows of
//                  W arrive as whole 256-byte pieces, which streams them faster than loading MFMA
//                  fragments (64 bytes a row) straight from memory.  K may be cut into slices
//                  whose partial sums the reader adds.  With PAIRED, W holds the rows of a gate and of
//                  an up projection in turns of 16 and the kernel stores act(gate) * up, half
//                  as wide, without the two products ever being stored.
//
// Reference counterparts: crates/synaptix-kernels-cuda/src/best_cu/gemm/gemm_bf16.cu (TN family,
// mma.sync m16n8k16), best_cu/gemv/mma_gemv.cu:19-133 (M == 1), best_cu/gemm/gemm_f32.cu (SIMT).
// The tilings here are made for 64-lane waves and MFMA operand layouts, not translated.
#include <type_traits>

#include "common.h"

// What a kernel does with its 32-bit sums: store them as float or as bf16, or (the kernels over paired
// gate/up rows) store act(gate) * up as bf16 with the activation `act` of gate_activation.
struct Epilogue {
  int out_is_f32;
  int act;
};

// ------------------------------------------------------------------ SIMT, any type
#define SIMT_BM 64
#define SIMT_BN 64
#define SIMT_BK 16

template <typename TIn, typename TOut>
__global__ void __launch_bounds__(256)
gemm_simt_kernel(const TIn* __restrict__ x, const TIn* __restrict__ w, TOut* __restrict__ out, int M, int N, int K) {
  __shared__ float xs[SIMT_BK][SIMT_BM + 1];
  __shared__ float ws[SIMT_BK][SIMT_BN + 1];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * SIMT_BM, n0 = blockIdx.x * SIMT_BN;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += SIMT_BK) {
    // 64 rows x 16 k for each operand: 1024 values, 4 a thread
    for (int e = tid; e < SIMT_BM * SIMT_BK; e += 256) {
      const int r = e / SIMT_BK, kk = e % SIMT_BK;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
      xs[kk][r] = (gm < M && gk < K) ? to_f32<TIn>(x[(size_t)gm * K + gk]) : 0.f;
      ws[kk][r] = (gn < N && gk < K) ? to_f32<TIn>(w[(size_t)gn * K + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < SIMT_BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gm = m0 + tm + i, gn = n0 + tn + j;
      if (gm < M && gn < N) out[(size_t)gm * N + gn] = from_f32<TOut>(acc[i][j]);
    }
}

// ------------------------------------------------------------------ skinny, bf16, one row of x (up to 16)
// MFMA 16x16x32: A = x rows (m), B = W rows (n), D[m = 4*(lane/16)+j][n = lane%16].
// Both operands: lane holds row lane%16, k = 8*(lane/16) .. +8, one 16-byte load.
// A workgroup owns TILES * 16 rows of W, 16 for each group of KWAVES waves; the waves of a group take
// k-chunks of 32 round-robin, so that at any moment the group reads KWAVES*64 contiguous bytes of each
// row, and their partial tiles are summed in LDS in a fixed order.  PAIRED (TILES == 2): the first 16
// rows are gate rows, the second the up rows of the same outputs, and silu(gate) * up is stored.
template <int TILES, int KWAVES, int U, bool PAIRED>
__global__ void __launch_bounds__(TILES * KWAVES * SYN_WAVE)
gemm_skinny_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, void* __restrict__ out, Epilogue ep,
                   int M, int N, int K) {
  static_assert(!PAIRED || TILES == 2, "a pair is two tiles");
  constexpr int WAVES = TILES * KWAVES;
  __shared__ float part[WAVES][4][64];
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int tile = wave / KWAVES, kw = wave % KWAVES;
  const int r16 = lane % 16, kq = (lane / 16) * 8;
  const int n0 = (blockIdx.x * TILES + tile) * 16;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // Rows of W beyond N are read from the last valid row (their results are never stored); rows of x
  // beyond M are not loaded at all: the fewer lanes a load of x has, the less it costs.
  const bf16* wrow = w + (size_t)min(n0 + r16, N - 1) * K + kq;
  const bool xok = r16 < M;
  const bf16* xrow = x + (size_t)min(r16, M - 1) * K + kq;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};

  // U chunks of 32 at a time: all loads of a group are issued before the first product needs them,
  // so that a wave keeps U KiB of the weight stream in flight
  constexpr int GROUP = 32 * U;
  const int k_full = K / (KWAVES * GROUP) * (KWAVES * GROUP);
  for (int k0 = kw * GROUP; k0 < k_full; k0 += KWAVES * GROUP) {
    bf16x8 bw[U], ax[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      bw[u] = __builtin_nontemporal_load((const bf16x8*)(wrow + k0 + u * 32));
      ax[u] = xok ? *(const bf16x8*)(xrow + k0 + u * 32) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[u], bw[u], acc, 0, 0, 0);
  }
  // what is left of K, chunk by chunk; K is a multiple of 8, so a lane's 8 elements lie inside or
  // outside as a whole
  for (int k0 = k_full + kw * 32; k0 < K; k0 += KWAVES * 32) {
    const bool kin = k0 + kq < K;
    const bf16x8 ax = (kin && xok) ? *(const bf16x8*)(xrow + k0) : zero;
    const bf16x8 bw = kin ? *(const bf16x8*)(wrow + k0) : zero;
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax, bw, acc, 0, 0, 0);
  }

#pragma unroll
  for (int j = 0; j < 4; ++j) part[wave][j][lane] = acc[j];
  __syncthreads();
  auto summed = [&](int t, int j, int ln) {
    float s = 0.f;
#pragma unroll
    for (int q = 0; q < KWAVES; ++q) s += part[t * KWAVES + q][j][ln];
    return s;
  };
  if constexpr (PAIRED) {
    for (int idx = threadIdx.x; idx < 4 * 64; idx += WAVES * SYN_WAVE) {
      const int j = idx / 64, ln = idx % 64;
      const int m = 4 * (ln / 16) + j, col = (int)blockIdx.x * 16 + ln % 16;  // N / 2 outputs, 16 a workgroup
      if (m < M && 2 * col < N) {
        const float g = summed(0, j, ln), up = summed(1, j, ln);
        ((bf16*)out)[(size_t)m * (N / 2) + col] = (bf16)gated(ep.act, g, up);
      }
    }
  } else {
    for (int idx = threadIdx.x; idx < TILES * 4 * 64; idx += WAVES * SYN_WAVE) {
      const int t = idx / 256, j = (idx / 64) % 4, ln = idx % 64;
      const int m = 4 * (ln / 16) + j, n = (blockIdx.x * TILES + t) * 16 + ln % 16;
      if (m < M && n < N) {
        const float v = summed(t, j, ln);
        if (ep.out_is_f32)
          ((float*)out)[(size_t)m * N + n] = v;
        else
          ((bf16*)out)[(size_t)m * N + n] = (bf16)v;
      }
    }
  }
}

template <int TILES, int KWAVES, int U, bool PAIRED = false>
static void launch_skinny(const bf16* x, const bf16* w, void* out, Epilogue ep, int M, int N, int K,
                          hipStream_t stream) {
  const int rows = TILES * 16;
  gemm_skinny_kernel<TILES, KWAVES, U, PAIRED>
      <<<(N + rows - 1) / rows, TILES * KWAVES * SYN_WAVE, 0, stream>>>(x, w, out, ep, M, N, K);
}

// ------------------------------------------------------------------ a norm between two products for few rows
// RMSNorm between two products for few rows of x needs every element of a row, which no workgroup of the product
// before it holds; as a kernel of its own it moves a few KB and costs a launch.  The products over packed
// weights therefore carry it between them in two halves:
//   * the product BEFORE the norm (resid != null; one slice of K, float sums) adds its sums into the float residual
//     rows, stores xs[m, n] = bf16((gain_offset + gain[n]) * resid[m, n]) (the norm's input with the gain, without
//     the row's factor) and, for each group of 16 columns, ss_out[m, group] = the sum of resid[m, n]^2 over them;
//   * the product AFTER the norm (ss != null) takes xs as its x and multiplies its finished sums of row m by
//     rsqrt(sum over groups of ss[m, :] / dim + eps): the product is linear in x, so the row's factor can wait.
// A row's statistic is added up in a fixed order (groups in turn over the lanes, then the wave's tree).
struct RowNorm {
  const float* ss;    // [M, ss_groups] of the product before, or null
  int ss_groups;
  float inv_dim;      // 1 / width of the normed rows
  float eps;
  float* resid;       // [M, N] float, or null
  bf16* xs;           // [M, N]
  float* ss_out;      // [M, N / 16]
  const void* gain;   // [N] bf16 or float
  int gain_is_f32;
  float gain_offset;
};

// inv[m] for the rows of x into LDS (16 floats): wave w takes rows w and w + n_waves (up to 16 rows, 8 waves or more).
// The statistic's first 256 groups a row are asked for before the product's loop (row_stat_load) and added up behind
// it (row_stat_finish), so that their way from memory is not the tail of the workgroup.
struct RowStat {
  float v[2][4];
};
__device__ __forceinline__ void row_stat_load(const RowNorm& rn, int M, int wave, int n_waves, int lane, RowStat& st) {
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int m = wave + r * n_waves;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = lane + SYN_WAVE * i;
      st.v[r][i] = (rn.ss && m < M && t < rn.ss_groups) ? rn.ss[(size_t)m * rn.ss_groups + t] : 0.f;
    }
  }
}
__device__ __forceinline__ void row_stat_finish(const RowNorm& rn, int M, int wave, int n_waves, int lane, const RowStat& st,
                                                float* inv) {
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int m = wave + r * n_waves;
    if (m >= M) break;   // the same for the whole wave
    float s = (st.v[r][0] + st.v[r][1]) + (st.v[r][2] + st.v[r][3]);
    for (int t = lane + 4 * SYN_WAVE; t < rn.ss_groups; t += SYN_WAVE) s += rn.ss[(size_t)m * rn.ss_groups + t];
    s = wave_sum(s);
    if (lane == 0) inv[m] = rsqrtf(s * rn.inv_dim + rn.eps);
  }
}

// the epilogue of the product before the norm for output (m, n) with its finished sum v; all 16 lanes of a
// group of columns call it together (rows beyond M with in == false); r0 and g: resid[m, n] and the gain of
// column n, asked for before the product's loop
__device__ __forceinline__ void resid_norm_store(const RowNorm& rn, bool in, int m, int n, int N, float v, float r0, float g) {
  float r = 0.f;
  if (in) {
    const size_t at = (size_t)m * N + n;
    r = r0 + v;
    rn.resid[at] = r;
    rn.xs[at] = (bf16)(g * r);
  }
  float q = r * r;
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) q += __shfl_xor(q, off, SYN_WAVE);
  if (in && (n & 15) == 0) rn.ss_out[(size_t)m * (N / 16) + n / 16] = q;
}

// ------------------------------------------------------------------ few rows of x, W in fragment order
// The same scheme as gemm_skinny (up to 16 rows of x, K split over the waves of a group, partial
// tiles summed in LDS in a fixed order) over a copy of W that is kept in the order of the MFMA
// fragments: wp[N / 16][K / 32][64 lanes][8], lane = 16 * (k % 32 / 8) + n % 16.  A wave's load of a
// fragment is then 1 KB of consecutive bytes, and the fragments of a group of rows follow each other
// along K: the weight stream is read as a kernel that does nothing else reads it (measured 6.2 to
// 6.7 TB/s on the wide products, against 4.5 to 5.3 from rows of W).  The fragments of x come from
// memory for every wave (x stays in the caches); that costs as many requests as W from 16 rows on,
// so the callers use this kernel up to 8 rows.  Wave kw of a group takes the k-steps kw * U .. + U,
// then those KWAVES * U further on.
template <int TILES, int KWAVES, int U, bool PAIRED>
__global__ void __launch_bounds__(TILES * KWAVES * SYN_WAVE)
gemm_packed_kernel(const bf16* __restrict__ x, const bf16* __restrict__ wp, void* __restrict__ out, Epilogue ep,
                   int M, int N, int K, int ks_slice, RowNorm rn) {
  static_assert(!PAIRED || TILES == 2, "a pair is two tiles");
  constexpr int WAVES = TILES * KWAVES;
  __shared__ float part[WAVES][4][64];
  __shared__ float inv[16];
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int tile = wave / KWAVES, kw = wave % KWAVES;
  const int r16 = lane % 16, kq = (lane / 16) * 8;
  const int nt = (int)blockIdx.x * TILES + tile, n_tiles = N / 16;   // 16 rows of W
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int nks = K / 32;
  const bool tile_in = nt < n_tiles;   // the last workgroup may hold a group beyond the end
  const bf16* wt = wp + ((size_t)min(nt, n_tiles - 1) * nks * 64 + lane) * 8;
  const bool xok = r16 < M;
  const bf16* xrow = x + (size_t)min(r16, M - 1) * K + kq;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  // what the epilogue needs of a norm's halves is asked for now, not behind the loop
  RowStat stat;
  if (rn.ss) row_stat_load(rn, M, wave, WAVES, lane, stat);
  float r0 = 0.f, g0 = 0.f;
  static_assert(TILES * 256 <= WAVES * SYN_WAVE, "every thread stores at most one output");
  if (!PAIRED && rn.resid && threadIdx.x < TILES * 256) {
    const int t = threadIdx.x / 256, j = (threadIdx.x / 64) % 4, ln = threadIdx.x % 64;
    const int m = 4 * (ln / 16) + j, n = ((int)blockIdx.x * TILES + t) * 16 + ln % 16;
    if (m < M && n < N) r0 = rn.resid[(size_t)m * N + n], g0 = load_gain(rn.gain, rn.gain_is_f32, n, rn.gain_offset);
  }
  // blockIdx.y = which slice of K (ks_slice k-steps of 32) this workgroup sums; its output is slice blockIdx.y
  // of a float [slices, M, N] that the reader adds up (a product with few rows of W gets more workgroups so)
  const int ks_begin = (int)blockIdx.y * ks_slice, ks_end = min(nks, ks_begin + ks_slice);
  if (tile_in) {
    for (int ks0 = ks_begin + kw * U; ks0 < ks_end; ks0 += KWAVES * U) {
      bf16x8 bw[U], ax[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool in = ks0 + u < ks_end;
        bw[u] = in ? __builtin_nontemporal_load((const bf16x8*)(wt + (size_t)(ks0 + u) * 512)) : zero;
        ax[u] = (in && xok) ? *(const bf16x8*)(xrow + (ks0 + u) * 32) : zero;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[u], bw[u], acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) part[wave][j][lane] = acc[j];
  if (rn.ss) row_stat_finish(rn, M, wave, WAVES, lane, stat, inv);
  __syncthreads();
  auto summed = [&](int t, int j, int ln) {
    float s = 0.f;
#pragma unroll
    for (int q = 0; q < KWAVES; ++q) s += part[t * KWAVES + q][j][ln];
    return s;
  };
  if constexpr (PAIRED) {
    for (int idx = threadIdx.x; idx < 4 * 64; idx += WAVES * SYN_WAVE) {
      const int j = idx / 64, ln = idx % 64;
      const int m = 4 * (ln / 16) + j, col = (int)blockIdx.x * 16 + ln % 16;  // N / 2 outputs, 16 a workgroup
      if (m < M && 2 * col < N) {
        const float f = rn.ss ? inv[m] : 1.f;
        const float g = summed(0, j, ln) * f, up = summed(1, j, ln) * f;
        ((bf16*)out)[(size_t)m * (N / 2) + col] = (bf16)gated(ep.act, g, up);
      }
    }
  } else {
    for (int idx = threadIdx.x; idx < TILES * 4 * 64; idx += WAVES * SYN_WAVE) {
      const int t = idx / 256, j = (idx / 64) % 4, ln = idx % 64;
      const int m = 4 * (ln / 16) + j, n = ((int)blockIdx.x * TILES + t) * 16 + ln % 16;
      const bool in = m < M && n < N;
      float v = summed(t, j, ln);
      if (rn.ss && in) v *= inv[m];
      if (rn.resid) {   // the same for the whole workgroup
        resid_norm_store(rn, in, m, n, N, v, r0, g0);
      } else if (in) {
        if (ep.out_is_f32)
          ((float*)out)[((size_t)blockIdx.y * M + m) * N + n] = v;
        else
          ((bf16*)out)[(size_t)m * N + n] = (bf16)v;
      }
    }
  }
}

template <int TILES, int KWAVES, int U, bool PAIRED = false>
static void launch_packed(const bf16* x, const bf16* wp, void* out, Epilogue ep, int M, int N, int K,
                          hipStream_t stream, int slices, const RowNorm& rn) {
  const int rows = TILES * 16;
  const int ks_slice = (K / 32 + slices - 1) / slices;
  gemm_packed_kernel<TILES, KWAVES, U, PAIRED>
      <<<dim3((N + rows - 1) / rows, slices), TILES * KWAVES * SYN_WAVE, 0, stream>>>(x, wp, out, ep, M, N, K, ks_slice, rn);
}


// The same with two adjacent groups of 16 rows of W for every wave (for PAIRED: the gate rows and the up rows of
// the same 16 outputs): a fragment of x is loaded once for two products, a third fewer loads at 8 rows of x.
template <int KWAVES, int U, bool PAIRED>
__global__ void __launch_bounds__(KWAVES * SYN_WAVE)
gemm_packed2_kernel(const bf16* __restrict__ x, const bf16* __restrict__ wp, void* __restrict__ out, Epilogue ep,
                    int M, int N, int K, int ks_slice, RowNorm rn) {
  __shared__ float part[KWAVES][2][4][64];
  __shared__ float inv[16];
  const int kw = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int r16 = lane % 16, kq = (lane / 16) * 8;
  const int nt = (int)blockIdx.x * 2, n_tiles = N / 16;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int nks = K / 32;
  const bool second = nt + 1 < n_tiles;   // an odd number of groups leaves the last workgroup one
  const bf16* wt0 = wp + ((size_t)nt * nks * 64 + lane) * 8;
  const bf16* wt1 = wp + ((size_t)min(nt + 1, n_tiles - 1) * nks * 64 + lane) * 8;
  const bool xok = r16 < M;
  const bf16* xrow = x + (size_t)min(r16, M - 1) * K + kq;
  f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  RowStat stat;
  if (rn.ss) row_stat_load(rn, M, kw, KWAVES, lane, stat);
  const int ks_begin = (int)blockIdx.y * ks_slice, ks_end = min(nks, ks_begin + ks_slice);
  for (int ks0 = ks_begin + kw * U; ks0 < ks_end; ks0 += KWAVES * U) {
    bf16x8 b0[U], b1[U], ax[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool in = ks0 + u < ks_end;
      b0[u] = in ? __builtin_nontemporal_load((const bf16x8*)(wt0 + (size_t)(ks0 + u) * 512)) : zero;
      b1[u] = in ? __builtin_nontemporal_load((const bf16x8*)(wt1 + (size_t)(ks0 + u) * 512)) : zero;
      ax[u] = (in && xok) ? *(const bf16x8*)(xrow + (ks0 + u) * 32) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[u], b0[u], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[u], b1[u], acc1, 0, 0, 0);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) part[kw][0][j][lane] = acc0[j], part[kw][1][j][lane] = acc1[j];
  if (rn.ss) row_stat_finish(rn, M, kw, KWAVES, lane, stat, inv);
  __syncthreads();
  auto summed = [&](int t, int j, int ln) {
    float s = 0.f;
#pragma unroll
    for (int q = 0; q < KWAVES; ++q) s += part[q][t][j][ln];
    return s;
  };
  if constexpr (PAIRED) {
    for (int idx = threadIdx.x; idx < 4 * 64; idx += KWAVES * SYN_WAVE) {
      const int j = idx / 64, ln = idx % 64;
      const int m = 4 * (ln / 16) + j, col = (int)blockIdx.x * 16 + ln % 16;  // N / 2 outputs, 16 a workgroup
      if (m < M && 2 * col < N) {
        const float f = rn.ss ? inv[m] : 1.f;
        ((bf16*)out)[(size_t)m * (N / 2) + col] = (bf16)gated(ep.act, summed(0, j, ln) * f, summed(1, j, ln) * f);
      }
    }
  } else {
    for (int idx = threadIdx.x; idx < 2 * 4 * 64; idx += KWAVES * SYN_WAVE) {
      const int t = idx / 256, j = (idx / 64) % 4, ln = idx % 64;
      const int m = 4 * (ln / 16) + j, n = (nt + t) * 16 + ln % 16;
      if (m < M && n < N && (t == 0 || second)) {
        float v = summed(t, j, ln);
        if (rn.ss) v *= inv[m];
        if (ep.out_is_f32) ((float*)out)[((size_t)blockIdx.y * M + m) * N + n] = v;
        else ((bf16*)out)[(size_t)m * N + n] = (bf16)v;
      }
    }
  }
}

template <int KWAVES, int U, bool PAIRED = false>
static void launch_packed2(const bf16* x, const bf16* wp, void* out, Epilogue ep, int M, int N, int K,
                           hipStream_t stream, int slices, const RowNorm& rn) {
  const int ks_slice = (K / 32 + slices - 1) / slices;
  gemm_packed2_kernel<KWAVES, U, PAIRED>
      <<<dim3((N + 31) / 32, slices), KWAVES * SYN_WAVE, 0, stream>>>(x, wp, out, ep, M, N, K, ks_slice, rn);
}

// ------------------------------------------------------------------ shared by the tiled kernels
// Which tile: workgroup b runs on XCD b % 8, and each XCD has an L2 of its own.  Tiles are grouped
// into panels of PM x PN (m fastest); a panel goes to one XCD, so the workgroups that run there at
// the same time share rows of x and of W in its L2.  False for the launches that pad the last panels.
// With slices of K (blockIdx.y) the panels of slice s are handed out s * panels XCDs further on, so
// that a product of fewer than 8 panels still reaches every XCD.
__device__ __forceinline__ bool tile_of_workgroup(int M, int N, int BM, int BN, int& tm, int& tn) {
  const int tiles_n = (N + BN - 1) / BN, tiles_m = (M + BM - 1) / BM;
  const int PM = min(8, tiles_m), PN = 4;
  const int panels_m = (tiles_m + PM - 1) / PM, panels = panels_m * ((tiles_n + PN - 1) / PN);
  const int xcd = ((int)blockIdx.x + 8 - (int)((blockIdx.y * panels) % 8)) % 8, local = (int)blockIdx.x / 8;
  const int panel = (local / (PM * PN)) * 8 + xcd, in_panel = local % (PM * PN);
  tm = (panel % panels_m) * PM + in_panel % PM;
  tn = (panel / panels_m) * PN + in_panel / PM;
  return tm < tiles_m && tn < tiles_n;
}

static int tile_grid(int M, int N, int BM, int BN) {
  const int tiles_n = (N + BN - 1) / BN, tiles_m = (M + BM - 1) / BM;
  const int PM = tiles_m < 8 ? tiles_m : 8, PN = 4;
  const int panels = ((tiles_m + PM - 1) / PM) * ((tiles_n + PN - 1) / PN);
  return (panels + 7) / 8 * 8 * PM * PN;
}

// The accumulators of a wave (TM x TN tiles of MFMA 32x32: D[m = 8*(e/4) + 4*(lane/32) + e%4][n = lane%32])
// to memory.  mw, nw: the first row and column of the wave's part.  PAIRED: columns n % 32 < 16 are
// gate rows, the 16 after them the up rows of the same outputs (N is a multiple of 32 then, so a tile of
// 32 columns lies inside or outside as a whole).  Two tiles side by side are stored together: the lanes
// of the first kind take the first tile (their own gate, the partner's up), the others the second (the
// partner's gate, their own up), so that a store covers 32 consecutive outputs of a row (64 bytes, not
// twice 32).  A last tile without a neighbour is stored by the lanes of the first kind alone.
template <int TM, int TN, bool PAIRED>
__device__ __forceinline__ void store_tiles(const f32x16 (&acc)[TM][TN], void* __restrict__ out, Epilogue ep,
                                            size_t slice, int M, int N, int mw, int nw, int lane) {
  if constexpr (PAIRED) {
    const bool first = lane % 32 < 16;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; j += 2)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = mw + i * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
          const float own0 = acc[i][j][e], other0 = __shfl_xor(own0, 16, SYN_WAVE);
          if (j + 1 < TN) {   // known once the loop is unrolled
            const float own1 = acc[i][j + 1 < TN ? j + 1 : j][e], other1 = __shfl_xor(own1, 16, SYN_WAVE);
            const float g = first ? own0 : other1, up = first ? other0 : own1;
            if (m < M && nw + (j + (first ? 0 : 1)) * 32 < N)
              ((bf16*)out)[(size_t)m * (N / 2) + (nw + j * 32) / 2 + lane % 32] = (bf16)gated(ep.act, g, up);
          } else {
            if (m < M && nw + j * 32 < N && first)
              ((bf16*)out)[(size_t)m * (N / 2) + (nw + j * 32) / 2 + lane % 16] = (bf16)gated(ep.act, own0, other0);
          }
        }
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = mw + i * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
          const int n = nw + j * 32 + lane % 32;
          if (m < M && n < N) {
            if (ep.out_is_f32)
              ((float*)out)[(slice * M + m) * N + n] = acc[i][j][e];
            else
              ((bf16*)out)[(size_t)m * N + n] = (bf16)acc[i][j][e];
          }
        }
  }
}

// ------------------------------------------------------------------ tiled, bf16
// Block tile BM (m) x BN (n) x BK (k); WM x WN waves, each (BM/WM) x (BN/WN) of MFMA 32x32x16 tiles.
// MFMA 32x32x16: A = x rows, B = W rows; lane holds row lane%32, k = 8*(lane/32) .. +8;
// D[m = 8*(j/4) + 4*(lane/32) + j%4][n = lane%32], j = 0..15.
// LDS tiles are double-buffered: while one k-tile is multiplied the next is on its way from memory
// into registers, and is stored into the other buffer before the barrier.
template <int BM, int BN, int BK, int WM, int WN, bool KTAIL, bool PAIRED>
__global__ void __launch_bounds__(64 * WM * WN)
gemm_tiled_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, void* __restrict__ out, Epilogue ep,
                  int M, int N, int K, int k_slice) {
  constexpr bool FEW = BM <= 64;                     // the variants for few rows of x: slices of K, absent rows
  constexpr int THREADS = 64 * WM * WN;              // WM x WN waves
  constexpr int LD = BK + 8;                         // padded row of the LDS tiles, in bf16 elements
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;  // 32x32 tiles a wave holds in m and n
  constexpr int CPR = BK / 8;                        // 16-byte chunks in a tile row
  constexpr int RPP = THREADS / CPR;                 // tile rows the workgroup moves in one pass
  constexpr int XL = BM / RPP, WL = BN / RPP;        // passes for x and for W
  static_assert(BM % RPP == 0 && BN % RPP == 0 && TM >= 1 && TN >= 1, "tile shape");
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];  // [2][(BM + BN) * LD]
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE;
  const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
  int tm, tn;
  if (!tile_of_workgroup(M, N, BM, BN, tm, tn)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // global -> LDS: thread t moves chunk t % CPR of rows t / CPR + RPP * i
  const int lrow = tid / CPR, lchunk = (tid % CPR) * 8;
  // rows of x beyond M are not fetched (their LDS rows hold zeros and their results are never
  // stored): with few rows this spares most of the traffic for x
  const bf16* xg[XL];
  const bf16* wg[WL];
  bool xin[XL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    xin[i] = !FEW || m0 + lrow + RPP * i < M;
    xg[i] = x + (size_t)min(m0 + lrow + RPP * i, M - 1) * K + lchunk;
  }
#pragma unroll
  for (int i = 0; i < WL; ++i) wg[i] = w + (size_t)min(n0 + lrow + RPP * i, N - 1) * K + lchunk;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // blockIdx.y = which slice of K (k_slice elements, a multiple of 128) this workgroup sums
  const int k_begin = FEW ? (int)blockIdx.y * k_slice : 0, k_end = FEW ? min(K, k_begin + k_slice) : K;
  const int nk = (k_end - k_begin + BK - 1) / BK;
  bf16x8 rx[XL], rw[WL];
  auto fetch = [&](int kt) {
    // K is a multiple of 8: a chunk lies inside or outside as a whole
    const int k = k_begin + kt * BK;
    const bool kin = !KTAIL || k + lchunk < k_end;
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      rx[i] = (kin && xin[i]) ? *(const bf16x8*)(xg[i] + k) : zero;
    }
#pragma unroll
    for (int i = 0; i < WL; ++i) rw[i] = kin ? *(const bf16x8*)(wg[i] + k) : zero;
  };
  auto stash = [&](int buf) {
    bf16* xs = smem + buf * (BM + BN) * LD;
    bf16* ws = xs + BM * LD;
#pragma unroll
    for (int i = 0; i < XL; ++i) *(bf16x8*)(xs + (lrow + RPP * i) * LD + lchunk) = rx[i];
#pragma unroll
    for (int i = 0; i < WL; ++i) *(bf16x8*)(ws + (lrow + RPP * i) * LD + lchunk) = rw[i];
  };

  fetch(0);
  stash(0);
  __syncthreads();
  const int fr = lane % 32, fk = (lane / 32) * 8;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) fetch(kt + 1);
    const bf16* xs = smem + buf * (BM + BN) * LD;
    const bf16* ws = xs + BM * LD;
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      bf16x8 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = *(const bf16x8*)(xs + (wm + i * 32 + fr) * LD + ks + fk);
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = *(const bf16x8*)(ws + (wn + j * 32 + fr) * LD + ks + fk);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) stash(buf ^ 1);  // the other buffer was last read before the previous barrier
    __syncthreads();
  }

  store_tiles<TM, TN, PAIRED>(acc, out, ep, FEW ? blockIdx.y : 0, M, N, m0 + wm, n0 + wn, lane);
}

template <int BM, int BN, int BK, int WM, int WN, bool PAIRED = false>
static int launch_tiled(const bf16* x, const bf16* w, void* out, Epilogue ep, int M, int N, int K,
                        hipStream_t stream, int slices = 1) {
  SYN_CHECK(slices == 1 || BM <= 64, "gemm: slices of K only with the tiles for few rows");   // (gemm_tiled's own limit)
  const int k_slice = ((K + slices - 1) / slices + 127) / 128 * 128;  // the same cut as launch_direct makes
  const int grid = tile_grid(M, N, BM, BN);
  const size_t lds = (size_t)2 * (BM + BN) * (BK + 8) * sizeof(bf16);
  static OncePerDevice raised;
  if (lds > 65536) {
    const hipError_t e = once_per_device(raised, [&] {
      hipError_t r = hipFuncSetAttribute((const void*)gemm_tiled_kernel<BM, BN, BK, WM, WN, false, PAIRED>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (r == hipSuccess)
        r = hipFuncSetAttribute((const void*)gemm_tiled_kernel<BM, BN, BK, WM, WN, true, PAIRED>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      return r;
    });
    SYN_CHECK(e == hipSuccess, "gemm: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
  }
  // whole k-tiles only, and no slice that begins at or beyond the end of K: then no chunk needs a check
  if (K % BK == 0 && k_slice % BK == 0 && (long)(slices - 1) * k_slice < K)
    gemm_tiled_kernel<BM, BN, BK, WM, WN, false, PAIRED>
        <<<dim3(grid, slices), 64 * WM * WN, lds, stream>>>(x, w, out, ep, M, N, K, k_slice);
  else
    gemm_tiled_kernel<BM, BN, BK, WM, WN, true, PAIRED>
        <<<dim3(grid, slices), 64 * WM * WN, lds, stream>>>(x, w, out, ep, M, N, K, k_slice);
  return 0;
}

// ------------------------------------------------------------------ tiled, loads straight into LDS
// The same tiles with buffer_load_dwordx4 ... lds: a load writes its 16 bytes a lane into LDS without
// passing through registers, so a k-tile on its way costs no registers and no LDS store
// instructions, and the wait for it is the last thing before the barrier.  K (and every slice of
// it) must be a multiple of BK.  An instruction of a wave fills 1 KB of LDS in lane order: 8 rows of
// 64 k-values or 4 rows of 128, unpadded.  To keep the fragment reads free of bank conflicts all the
// same, slot s of row r holds the row's 16-byte chunk s ^ swizzle(r): the swizzle is applied to the
// global address of the lane that fills the slot, and again by the reader.  Measured 10 to 20 %
// faster than staging through registers for prompts, and for single tokens from 16 rows of x on.
template <int BK>
__device__ __forceinline__ int direct_swizzle(int row) {
  // BK = 64: a row is 128 bytes, two rows span the 64 banks; BK = 128: a row spans them all
  return BK == 64 ? (row >> 1) & 7 : row & (BK / 8 - 1);
}

// WP: w is the weight in fragment order (pack_weight: [N / 16][K / 32][64 lanes][8], N a multiple of 16).  A load of a
// wave then moves one fragment (16 rows x 32 k-values, 1 KB of consecutive bytes) into the slot that a load of
// plain rows fills, and a lane's fragment of an MFMA 32x32x16 lies in two of them: rows fr % 16 of fragment
// fr / 16, chunks 2 (ks % 2) + fh of k-fragment ks / 2; 16 lanes read 256 consecutive bytes, without a swizzle.
template <int BM, int BN, int BK, int WM, int WN, bool PAIRED, int STAGES, bool WP>
__global__ void __launch_bounds__(64 * WM * WN)
gemm_direct_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, void* __restrict__ out, Epilogue ep,
                   int M, int N, int K, int k_slice) {
  static_assert((BK == 64 || BK == 128 || BK == 256) && STAGES >= 2, "k-tiles of 64, 128 or 256 in two or more buffers");
  constexpr int WAVES = WM * WN;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int ROWS = BM + BN;
  constexpr int CPR = BK / 8;                    // 16-byte chunks in a row of a k-tile
  constexpr int RPI = 64 / CPR;                  // rows an instruction of a wave fills
  constexpr int PASSES = ROWS / (RPI * WAVES);   // instructions of a wave for one k-tile
  static_assert(ROWS % (RPI * WAVES) == 0 && TM >= 1 && TN >= 1, "tile shape");
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];  // [STAGES][ROWS][BK]
  const int tid = threadIdx.x, lane = tid % SYN_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / SYN_WAVE);   // scalar: LDS addresses of the loads stay scalar
  const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
  int tm, tn;
  if (!tile_of_workgroup(M, N, BM, BN, tm, tn)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  // blockIdx.y = which slice of K (k_slice elements, a multiple of BK) this workgroup sums
  const int k_begin = (int)blockIdx.y * k_slice, k_end = min(K, k_begin + k_slice);
  const int nk = max(0, (k_end - k_begin) / BK);

  // the descriptors begin at the tile's first rows, so a lane's offset stays below 2^32 for any M and N,
  // and end with the last row of x and of W: a lane whose row lies beyond reads nothing from memory
  // (its LDS slot gets zeros, and its results are never stored), which with few rows of x spares
  // most of the requests for x.
  // pass p: the wave fills tile rows (p * WAVES + wave) * RPI .. + RPI (x rows first, then W rows)
  static_assert(BM % (RPI * WAVES) == 0, "a pass lies in x or in W as a whole, for all waves alike");
  const size_t row_bytes = (size_t)K * sizeof(bf16);
  const BufferView vx = buffer_view(x + (size_t)m0 * K, (size_t)(M - m0) * row_bytes);
  // (in fragment order 16 rows of W are K / 32 fragments of 1 KB one after another: as many bytes as 16 plain rows)
  const BufferView vw = buffer_view(w + (size_t)n0 * K, (size_t)(N - n0) * row_bytes);
  constexpr int KF = BK / 32;                    // fragments of a k-tile along K
  unsigned src[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int row0 = (p * WAVES + wave) * RPI, row = row0 + lane / CPR;
    const int chunk = (lane % CPR) ^ direct_swizzle<BK>(row);
    if (WP && row0 >= BM) {
      const int slot = (row0 - BM) / RPI;        // which fragment of the tile: 16 rows slot / KF, k-fragment slot % KF
      src[p] = (unsigned)((size_t)(slot / KF) * 16 * row_bytes + (size_t)(slot % KF) * 1024 + lane * 16);
    } else {
      const int in_tile = row0 < BM ? row : row - BM;
      src[p] = (unsigned)((size_t)in_tile * row_bytes + chunk * 16);
    }
  }
  auto fetch = [&](int kt, int buf) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      bf16* dst = smem + (size_t)buf * ROWS * BK + (size_t)(p * WAVES + wave) * RPI * BK;  // the same for all lanes
      // every wave fills rows of x in the first passes and rows of W in the others; this kernel runs where a
      // row of W has one reader (up to 64 rows of x) or at most four: its loads are marked non-temporal
      if (p * WAVES * RPI < BM)
        buffer_to_lds16(vx, dst, src[p], (k_begin + kt * BK) * (int)sizeof(bf16));
      else
        buffer_to_lds16<true>(vw, dst, src[p], (k_begin + kt * BK) * (int)sizeof(bf16) * (WP ? 16 : 1));
    }
  };
  // Tile kt lies in buffer kt % STAGES; while it is multiplied the STAGES - 1 tiles after it are on their
  // way.  Before the barrier that ends a tile a wave waits until its own loads of the next tile have
  // written LDS (all but the (STAGES - 2) * PASSES youngest have then) and its fragment reads have
  // returned.  The barrier carries no fence: a fence would wait for every load on its way.
  constexpr int YOUNGER = (STAGES - 2) * PASSES;
  auto next_landed = [](bool full_pipeline) {
    if (full_pipeline) __builtin_amdgcn_s_waitcnt(0x0070 | (YOUNGER & 15) | ((YOUNGER >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0)
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int fr = lane % 32, fh = lane / 32;
#pragma unroll
  for (int t = 0; t < STAGES - 1; ++t)
    if (t < nk) fetch(t, t);  // a slice beyond the end of K stores zeros
  next_landed(nk >= STAGES - 1);
  __builtin_amdgcn_s_barrier();
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt % STAGES;
    const bool more = kt + STAGES - 1 < nk;
    if (more) fetch(kt + STAGES - 1, (kt + STAGES - 1) % STAGES);  // that buffer was last read before the previous barrier
    const bf16* xs = smem + (size_t)buf * ROWS * BK;
    const bf16* ws = xs + BM * BK;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 a[TM], b[TN];
      const int c = 2 * ks + fh;  // the 16-byte chunk of a row that this lane multiplies
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wm + i * 32 + fr;
        a[i] = *(const bf16x8*)(xs + row * BK + (c ^ direct_swizzle<BK>(row)) * 8);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int row = wn + j * 32 + fr;
        if constexpr (WP)
          b[j] = *(const bf16x8*)(ws + ((row / 16) * KF + ks / 2) * 512 + ((2 * (ks % 2) + fh) * 16 + row % 16) * 8);
        else
          b[j] = *(const bf16x8*)(ws + row * BK + (c ^ direct_swizzle<BK>(row + BM)) * 8);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    next_landed(more);
    __builtin_amdgcn_s_barrier();
  }
  store_tiles<TM, TN, PAIRED>(acc, out, ep, blockIdx.y, M, N, m0 + wm, n0 + wn, lane);
}

// A weight [N, K] as a product is handed it: plain rows, or in fragment order (pack_weight)
struct Weight {
  const bf16* p;
  bool packed;
};

// slices > 1 only with a float output [slices, M, N]; K must be a multiple of BK
template <int BM, int BN, int BK, int WM, int WN, bool PAIRED = false, int STAGES = 3>
static int launch_direct(const bf16* x, Weight w, void* out, Epilogue ep, int M, int N, int K,
                         hipStream_t stream, int slices = 1) {
  SYN_CHECK(K % BK == 0, "gemm: K = %d is no multiple of the k-tile %d", K, BK);
  const int step = BK > 128 ? BK : 128;
  const int k_slice = ((K + slices - 1) / slices + step - 1) / step * step;  // a multiple of BK
  const size_t lds = (size_t)STAGES * (BM + BN) * BK * sizeof(bf16);
  static OncePerDevice raised;
  if (lds > 65536) {
    const hipError_t e = once_per_device(raised, [&] {
      hipError_t r = hipFuncSetAttribute((const void*)gemm_direct_kernel<BM, BN, BK, WM, WN, PAIRED, STAGES, false>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (r == hipSuccess)
        r = hipFuncSetAttribute((const void*)gemm_direct_kernel<BM, BN, BK, WM, WN, PAIRED, STAGES, true>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      return r;
    });
    SYN_CHECK(e == hipSuccess, "gemm: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
  }
  const dim3 grid(tile_grid(M, N, BM, BN), slices);
  if (w.packed)
    gemm_direct_kernel<BM, BN, BK, WM, WN, PAIRED, STAGES, true><<<grid, 64 * WM * WN, lds, stream>>>(x, w.p, out, ep, M, N, K, k_slice);
  else
    gemm_direct_kernel<BM, BN, BK, WM, WN, PAIRED, STAGES, false><<<grid, 64 * WM * WN, lds, stream>>>(x, w.p, out, ep, M, N, K, k_slice);
  return 0;
}

// ------------------------------------------------------------------ tiled, M > 64: software-pipelined
// The k-tile of 64 is four k-steps of 8 (or more) MFMAs a wave.  What the plain loop above leaves to
// the compiler is laid out by hand here, because each of these was measured to cost matrix-unit time:
//   * the fragments of k-step s + 1 are read from LDS while the MFMAs of step s run (two sets of
//     fragment registers), and the reads are placed one behind each MFMA: a wave issues in order, and
//     an MFMA keeps the matrix unit busy for 32 cycles in which the read behind it costs nothing;
//   * the barrier of a k-tile stands before the MFMAs of its last k-step; behind it the loads of the
//     tile after the next and the first fragments of the next tile are issued, again one behind each MFMA;
//   * the loads go through a buffer descriptor (a base in scalar registers, a 32-bit offset a lane, the
//     k offset as a scalar): a load is then two instructions (LDS address into M0, the load), where a
//     64-bit address a lane costs vector adds and takes longer to issue.
// Counters showed the texture addresser busy about 25 cycles for each 1 KB load of 8 rows x 128 bytes,
// 1,600 of the 2,048 cycles that the MFMAs of a 256x256x64 tile take: loads that arrive in a burst
// hold up the waves that issue them, so their spread matters more than their number.
// WP: w in fragment order, as in gemm_direct_kernel.
template <int BM, int BN, int WM, int WN, bool PAIRED, bool WP>
__global__ void __launch_bounds__(64 * WM * WN)
gemm_pipelined_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, void* __restrict__ out, Epilogue ep,
                      int M, int N, int K, int k_slice) {
  constexpr int BK = 64;
  constexpr int WAVES = WM * WN;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int ROWS = BM + BN;
  constexpr int RPI = 8;                           // rows of 128 bytes that one load of a wave fills
  constexpr int PASSES = ROWS / (RPI * WAVES);     // loads of a wave for one k-tile
  constexpr int NM = TM * TN, NR = TM + TN;        // MFMAs and fragment reads of a wave in one k-step
  static_assert(ROWS % (RPI * WAVES) == 0 && BM % RPI == 0 && NM >= NR, "tile shape");
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];  // [2][ROWS][64], chunks swizzled as in gemm_direct
  const int tid = threadIdx.x, lane = tid % SYN_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / SYN_WAVE);   // scalar: LDS addresses of the loads stay scalar
  const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
  int tm, tn;
  if (!tile_of_workgroup(M, N, BM, BN, tm, tn)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  // blockIdx.y = which slice of K (k_slice elements, a multiple of BK) this workgroup sums; a slice is never empty
  const int k_begin = (int)blockIdx.y * k_slice;
  const int nk = (min(K, k_begin + k_slice) - k_begin) / BK;

  // the descriptors begin at the tile's first rows and the slice's first column, so a lane's offset stays
  // below 2^32 for any M and N
  const size_t row_bytes = (size_t)K * sizeof(bf16);
  const BufferView vx = buffer_view(x + (size_t)m0 * K + k_begin, (size_t)(M - m0) * row_bytes - k_begin * sizeof(bf16));
  const BufferView vw = buffer_view(w + (size_t)n0 * K + (size_t)k_begin * (WP ? 16 : 1),
                                    (size_t)(N - n0) * row_bytes - (size_t)k_begin * sizeof(bf16) * (WP ? 16 : 1));
  // pass p: the wave fills tile rows (p * WAVES + wave) * 8 .. + 8 (x rows first, then W rows; rows beyond M or
  // N repeat the last valid one and their results are never stored)
  unsigned src[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int row0 = (p * WAVES + wave) * RPI, row = row0 + lane / 8;
    const int chunk = (lane % 8) ^ direct_swizzle<BK>(row);
    if (WP && row0 >= BM) {
      // fragment slot of the tile: 16 rows slot / 2 (groups beyond N repeat the last one), k-fragment slot % 2
      const int slot = (row0 - BM) / RPI, group = min(slot / 2, (N - n0) / 16 - 1);
      src[p] = (unsigned)((size_t)group * 16 * row_bytes + (size_t)(slot % 2) * 1024 + lane * 16);
    } else {
      const int in_tile = row0 < BM ? min(row, M - 1 - m0) : min(row - BM, N - 1 - n0);
      src[p] = (unsigned)((size_t)in_tile * row_bytes + chunk * 16);
    }
  }
  auto fetch_pass = [&](int kt, int buf, int p) {
    bf16* dst = smem + (size_t)buf * ROWS * BK + (size_t)(p * WAVES + wave) * RPI * BK;
    const bool of_x = (p * WAVES + wave) * RPI < BM;
    // (a k-tile of 64 is 128 bytes further on in a plain row, two fragments of 1 KB further on in fragment order)
    buffer_to_lds16(of_x ? vx : vw, dst, src[p], kt * (BK * (int)sizeof(bf16)) * (WP && !of_x ? 16 : 1));
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int fr = lane % 32, fh = lane / 32;
  int arow[TM], brow[TN], asw[TM], bsw[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) arow[i] = (wm + i * 32 + fr) * BK, asw[i] = direct_swizzle<BK>(wm + i * 32 + fr);
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int row = wn + j * 32 + fr;
    // (in fragment order: the two fragments of rows row / 16 begin at 1,024 elements a group; k-step ks lies 256 further on)
    brow[j] = WP ? BM * BK + (row / 16) * 1024 + (fh * 16 + row % 16) * 8 : (BM + row) * BK;
    bsw[j] = direct_swizzle<BK>(BM + row);
  }
  bf16x8 a[2][TM], b[2][TN];   // two sets of fragments: one is multiplied while the other is read
  auto read_one = [&](int buf, int ks, int set, int idx) {
    const bf16* base = smem + (size_t)buf * ROWS * BK;
    const int c = 2 * ks + fh;  // the 16-byte chunk of a row that this lane multiplies
    if (idx < TM) a[set][idx] = *(const bf16x8*)(base + arow[idx] + (c ^ asw[idx]) * 8);
    else if constexpr (WP) b[set][idx - TM] = *(const bf16x8*)(base + brow[idx - TM] + ks * 256);
    else b[set][idx - TM] = *(const bf16x8*)(base + brow[idx - TM] + (c ^ bsw[idx - TM]) * 8);
  };
  auto mfmas = [&](int set) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[set][i], b[set][j], acc[i][j], 0, 0, 0);
  };
  // one k-tile.  MORE_LOADS: the tile after the next exists; MORE_TILES: a next tile exists.
  auto tile = [&](int kt, auto more_loads, auto more_tiles) {
    constexpr int NF = decltype(more_loads)::value ? PASSES : 0, NN = decltype(more_tiles)::value ? NR : 0;
    const int buf = kt & 1;
#pragma unroll
    for (int ks = 0; ks < 3; ++ks) {
      __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the fragments read one k-step ago are there
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < NR; ++i) read_one(buf, ks + 1, (ks + 1) & 1, i);
      mfmas(ks & 1);
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA,
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read behind it
      }
      __builtin_amdgcn_sched_group_barrier(0x008, NM - NR, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    // this wave's loads of the next tile have landed and its reads of this tile are done; behind the
    // barrier that holds for every wave.  No fence: this is all the barrier has to order.
    __builtin_amdgcn_s_waitcnt(0x0070);     // vmcnt(0) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // in program order a load into LDS and a fragment read alternate, so that they can be spread
#pragma unroll
    for (int i = 0; i < (NF > NN ? NF : NN); ++i) {
      if (i < NF) fetch_pass(kt + 2, buf, i);
      if (i < NN) read_one(buf ^ 1, 0, 0, i);
    }
    mfmas(1);
#pragma unroll
    for (int i = 0; i < NM; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (i < NF) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);   // one load,
      if (i < NN) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
    }
    __builtin_amdgcn_sched_barrier(0);
  };

#pragma unroll
  for (int p = 0; p < PASSES; ++p) fetch_pass(0, 0, p);
  if (nk > 1) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) fetch_pass(1, 1, p);
    __builtin_amdgcn_s_waitcnt(0x0f70 | (PASSES & 15) | ((PASSES >> 4) << 14));   // vmcnt(PASSES): tile 0 is there
  } else {
    __builtin_amdgcn_s_waitcnt(0x0f70);
  }
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < NR; ++i) read_one(0, 0, 0, i);
  int kt = 0;
  for (; kt + 2 < nk; ++kt) tile(kt, std::true_type{}, std::true_type{});
  if (kt + 1 < nk) tile(kt++, std::false_type{}, std::true_type{});
  tile(kt, std::false_type{}, std::false_type{});
  store_tiles<TM, TN, PAIRED>(acc, out, ep, blockIdx.y, M, N, m0 + wm, n0 + wn, lane);
}

template <int BM, int BN, int WM, int WN, bool PAIRED = false>
static int launch_pipelined(const bf16* x, Weight w, void* out, Epilogue ep, int M, int N, int K,
                            hipStream_t stream, int slices = 1) {
  SYN_CHECK(K % 64 == 0, "gemm: K = %d is no multiple of the k-tile 64", K);
  const int k_slice = ((K + slices - 1) / slices + 127) / 128 * 128;  // the same cut as the tiles for few rows make
  SYN_CHECK((long)(slices - 1) * k_slice < K, "gemm: %d slices of %d leave the last one empty (K = %d)", slices, k_slice, K);
  const size_t lds = (size_t)2 * (BM + BN) * 64 * sizeof(bf16);
  static OncePerDevice raised;
  if (lds > 65536) {
    const hipError_t e = once_per_device(raised, [&] {
      hipError_t r = hipFuncSetAttribute((const void*)gemm_pipelined_kernel<BM, BN, WM, WN, PAIRED, false>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (r == hipSuccess)
        r = hipFuncSetAttribute((const void*)gemm_pipelined_kernel<BM, BN, WM, WN, PAIRED, true>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      return r;
    });
    SYN_CHECK(e == hipSuccess, "gemm: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
  }
  const dim3 grid(tile_grid(M, N, BM, BN), slices);
  if (w.packed)
    gemm_pipelined_kernel<BM, BN, WM, WN, PAIRED, true><<<grid, 64 * WM * WN, lds, stream>>>(x, w.p, out, ep, M, N, K, k_slice);
  else
    gemm_pipelined_kernel<BM, BN, WM, WN, PAIRED, false><<<grid, 64 * WM * WN, lds, stream>>>(x, w.p, out, ep, M, N, K, k_slice);
  return 0;
}

// M > 64: the tile shape by pick_large_tile; loads straight into LDS where K allows it
template <bool PAIRED>
static int launch_large(const bf16* x, Weight w, void* out, Epilogue ep, int M, int N, int K,
                        hipStream_t stream, int slices = 1);

// Which of the large tiles for M > 64: 0 = 256 x 256, 1 = 256 x 192 (one workgroup of four waves a compute
// unit; a fifth less efficient), 2 = 128 x 128 (two workgroups a compute unit, about as much less efficient),
// 3 = 256 x 160 (four waves of 64 x 160; for N = 5120, which it cuts into 32 where 256 x 192 makes 27).
// The estimate is the number of rounds over the 256 compute units times the work of a tile.  Measured
// for N = 6144 and 24576 at 1,024 to 8,192 rows: the narrower tile wins where it fills a round that the
// wide one leaves partly empty (q/k/v at 2,048 and 4,096 rows: 100 against 116 us, 181 against 198) and
// loses over many rounds (gate+up at 3,072, 5,120 and 7,680 rows: 760 against 638 us, 989 against 900,
// 1524 against 1349); its factor came out between 1.15 and 1.3.  A tie goes to the larger tile.
static int pick_large_tile(int M, int N) {
  auto rounds = [](long tiles, long slots) { return (tiles + slots - 1) / slots; };
  auto tiles = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  const long cus = syn_compute_units();
  const double cost[4] = {(double)rounds(tiles(256, 256), cus) * 256 * 256,
                          (double)rounds(tiles(256, 192), cus) * 256 * 192 * 1.2,
                          (double)rounds(tiles(128, 128), 2 * cus) * 2 * 128 * 128 * 1.2,
                          (double)rounds(tiles(256, 160), cus) * 256 * 160 * 1.2};
  int best = 0;
  for (int i = 1; i < 4; ++i)
    if (cost[i] < cost[best]) best = i;
  return best;
}

template <bool PAIRED>
static int launch_large(const bf16* x, Weight w, void* out, Epilogue ep, int M, int N, int K,
                        hipStream_t stream, int slices) {
  // cut along K (the reader adds the partial sums): the largest tile, which the slices multiply
  if (slices > 1) return launch_pipelined<256, 256, 2, 4, PAIRED>(x, w, out, ep, M, N, K, stream, slices);
  const int shape = pick_large_tile(M, N);
  if (K % 64 == 0) {
    if (shape == 0) return launch_pipelined<256, 256, 2, 4, PAIRED>(x, w, out, ep, M, N, K, stream);
    if (shape == 1) return launch_pipelined<256, 192, 2, 2, PAIRED>(x, w, out, ep, M, N, K, stream);
    if (shape == 3) return launch_pipelined<256, 160, 4, 1, PAIRED>(x, w, out, ep, M, N, K, stream);
    return launch_pipelined<128, 128, 2, 2, PAIRED>(x, w, out, ep, M, N, K, stream);
  }
  SYN_CHECK(!w.packed, "gemm: a weight in fragment order needs a K that is a multiple of 64 (K = %d)", K);
  if (shape == 0) return launch_tiled<256, 256, 64, 4, 2, PAIRED>(x, w.p, out, ep, M, N, K, stream);
  if (shape == 1 || shape == 3) return launch_tiled<256, 192, 64, 4, 2, PAIRED>(x, w.p, out, ep, M, N, K, stream);
  return launch_tiled<128, 128, 64, 2, 2, PAIRED>(x, w.p, out, ep, M, N, K, stream);
}

// ------------------------------------------------------------------ entry point
// dtype: 0 = float in, float out; 1 = bf16 in, bf16 out; 2 = bf16 in, float out.
// slices > 1 (bf16 in, float out): out is [slices, M, N], slice s holds the sum over its part of K; the
// reader adds the slices.
// w_packed: w is the weight in fragment order (pack_weight; bf16, N a multiple of 16, K of 128): for the tiles that
// load straight into LDS; the other kernels read plain rows only.
SYN_EXPORT int syn_gemm(const void* x, const void* w, void* out, int dtype, int M, int N, int K, int force_simt,
                        int slices, int w_packed, hipStream_t stream) {
  SYN_CHECK(M > 0 && N > 0 && K > 0, "gemm: empty shape M=%d N=%d K=%d", M, N, K);
  SYN_CHECK(!w_packed || (dtype != 0 && !force_simt && N % 16 == 0 && K % 128 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0),
            "gemm: a weight in fragment order needs bf16 operands, N = %d a multiple of 16 and K = %d of 128", N, K);
  SYN_CHECK(dtype >= 0 && dtype <= 2, "gemm: unknown dtype code %d", dtype);
  SYN_CHECK(slices >= 1 && (slices == 1 || (dtype == 2 && !force_simt && K % 8 == 0 && slices <= 64 && (M <= 64 || K % 64 == 0))),
            "gemm: %d slices of K need bf16 operands and a float output (and beyond 64 rows a K that is a multiple of 64; K = %d)", slices, K);
  const dim3 simt_grid((N + SIMT_BN - 1) / SIMT_BN, (M + SIMT_BM - 1) / SIMT_BM);
  if (dtype == 0) {
    gemm_simt_kernel<float, float><<<simt_grid, 256, 0, stream>>>((const float*)x, (const float*)w, (float*)out, M, N, K);
    SYN_LAUNCH_CHECK("gemm_simt");
    return 0;
  }
  const int out_is_f32 = dtype == 2;
  const Epilogue ep = {out_is_f32, SYN_ACT_SILU};   // (no activation in a plain product)
  const bool aligned = (K % 8 == 0) && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0);
  SYN_CHECK(slices == 1 || aligned, "gemm: slices of K need 16-byte aligned operands");
  if (force_simt || !aligned) {
    if (out_is_f32)
      gemm_simt_kernel<bf16, float><<<simt_grid, 256, 0, stream>>>((const bf16*)x, (const bf16*)w, (float*)out, M, N, K);
    else
      gemm_simt_kernel<bf16, bf16><<<simt_grid, 256, 0, stream>>>((const bf16*)x, (const bf16*)w, (bf16*)out, M, N, K);
    SYN_LAUNCH_CHECK("gemm_simt");
    return 0;
  }
  const bf16* xb = (const bf16*)x;
  const bf16* wb = (const bf16*)w;
  const Weight wt = {wb, w_packed != 0};
  // From sweeps at the shapes of an 8B model (N = 4096 .. 151936, K = 4096 and 12288).
  // Short prompts (65 to 512 rows) of a narrow product: even the smallest of the large tiles would leave
  // most compute units without work (q/k/v at 128 rows: 48 tiles of 128 x 128), and the product is still
  // bound by reading W: the 64 x 64 tiles take it (q/k/v at 128 rows 57 -> 31 us, o_proj in two slices
  // 52 -> 18, down_proj in four 74 -> 34; at 256 rows 59 -> 36, 57 -> 22, 79 -> 62; at 512 rows o_proj
  // 58 -> 39 and q/k/v 63 -> 67; down_proj from 384 rows on and the output head stay on the large tiles).
  const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
  // (cut along K the tiles are 128 x 128 up to 256 rows and 256 x 128 beyond)
  const long tiles_cut = (long)(M <= 256 ? (M + 127) / 128 : (M + 255) / 256) * ((N + 127) / 128);
  const bool few_large_tiles = M > 64 && M <= 512 && K % 128 == 0 && (slices > 1 ? tiles_cut : tiles128) * slices <= syn_compute_units();
  int rc = 0;
  if (M == 1 && slices == 1 && !w_packed) {
    // one row: fragments of W straight from memory, K split over the waves
    if (N <= 8192) launch_skinny<1, 16, 4>(xb, wb, out, ep, M, N, K, stream);
    else launch_skinny<1, 8, 4>(xb, wb, out, ep, M, N, K, stream);
  } else if (M <= 32) {
    // few rows: memory-bound; small tiles (many workgroups), deep in K (long pieces of each row), three
    // k-tiles in flight, straight into LDS where K allows it
    if (N >= 65536 && K % 256 == 0) rc = launch_direct<32, 64, 256, 1, 2>(xb, wt, out, ep, M, N, K, stream, slices);
    else if (N >= 65536 && !w_packed) rc = launch_tiled<32, 32, 256, 1, 1>(xb, wb, out, ep, M, N, K, stream, slices);
    else if (K % 128 == 0) rc = launch_direct<32, 64, 128, 1, 2>(xb, wt, out, ep, M, N, K, stream, slices);
    else rc = launch_tiled<32, 64, 128, 1, 2>(xb, wb, out, ep, M, N, K, stream, slices);
  } else if (M <= 64 && K % 128 == 0) {
    // 33 to 64 rows: 128 rows of W a workgroup, so that the rows of x are fetched half as often (every
    // workgroup reads all of x), three k-tiles in a ring, one workgroup a compute unit.  A decode step of 64
    // sequences: 7.70 -> 7.51 ms with this tile for q/k/v, o_proj and down_proj, 7.26 with it for gate+up
    // as well (though that product then has only 192 workgroups); 64 x 64 tiles in a ring of four: 8.08.
    rc = launch_direct<64, 128, 128, 2, 4, false, 3>(xb, wt, out, ep, M, N, K, stream, slices);
  } else if (few_large_tiles && slices > 1) {
    // short prompts of a narrow product whose reader adds partial sums: k-tiles of 64 in a ring of three, 128 rows
    // of W a workgroup, and as many slices of K as fill the compute units (ops.gemm_slices).  Measured at the
    // shapes of an 8B layer against the tiles of the branch below: 128 rows: q/k/v in 4 slices 17 us (31 uncut),
    // down_proj in 8 slices 26 (30 in 4); 256 rows: q/k/v 26 (32), down_proj 39 (50); 512 rows (256 rows of x a
    // tile): q/k/v in 2 slices 36 (51), o_proj in 4 slices 29 (30), down_proj 57 (55).
    if (M <= 256) rc = launch_direct<128, 128, 64, 2, 4, false, 3>(xb, wt, out, ep, M, N, K, stream, slices);
    else rc = launch_direct<256, 128, 64, 4, 2, false, 3>(xb, wt, out, ep, M, N, K, stream, slices);
  } else if (few_large_tiles && K % 128 == 0) {
    // the same uncut: 64 x 128 up to 256 rows, 128 x 128 beyond (a prompt of 256 tokens
    // 8.91 -> 8.24 ms, of 512 tokens 12.63 -> 11.59 ms against 64 x 64 tiles)
    if (M <= 256) rc = launch_direct<64, 128, 128, 2, 4, false, 3>(xb, wt, out, ep, M, N, K, stream, slices);
    else rc = launch_direct<128, 128, 128, 2, 4, false, 2>(xb, wt, out, ep, M, N, K, stream, slices);
  } else if (M <= 64 || few_large_tiles) {
    if (K % 128 == 0) rc = launch_direct<64, 64, 128, 2, 2, false, 2>(xb, wt, out, ep, M, N, K, stream, slices);
    else rc = launch_tiled<64, 64, 128, 2, 2>(xb, wb, out, ep, M, N, K, stream, slices);
  } else {
    rc = launch_large<false>(xb, wt, out, ep, M, N, K, stream, slices);
  }
  if (rc) return rc;
  SYN_LAUNCH_CHECK("gemm");
  return 0;
}

// out[M, N/2] = silu(x . Wg^T) * (x . Wu^T), bf16, where w [N, K] holds the rows of Wg and of Wu in
// turns of 16: rows 32b .. 32b+15 are rows 16b .. 16b+15 of Wg, rows 32b+16 .. 32b+31 those of Wu.
// The activation is applied to the 32-bit sums and rounded once.
// w_packed: as for syn_gemm
SYN_EXPORT int syn_gemm_swiglu(const void* x, const void* w, void* out, int M, int N, int K, int act, int w_packed,
                               hipStream_t stream) {
  SYN_CHECK(M > 0 && N > 0 && K > 0, "gemm_swiglu: empty shape M=%d N=%d K=%d", M, N, K);
  SYN_CHECK(!w_packed || K % 128 == 0, "gemm_swiglu: a weight in fragment order needs K = %d a multiple of 128", K);
  SYN_CHECK(act >= 0 && act < SYN_ACT_COUNT, "gemm_swiglu: unknown activation code %d", act);
  const Epilogue ep = {0, act};
  SYN_CHECK(N % 32 == 0, "gemm_swiglu: %d paired rows are no multiple of 32", N);
  SYN_CHECK(K % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0,
            "gemm_swiglu: K = %d must be a multiple of 8 and the operands 16-byte aligned", K);
  const bf16* xb = (const bf16*)x;
  const bf16* wb = (const bf16*)w;
  int rc = 0;
  const Weight wt = {wb, w_packed != 0};
  if (M == 1 && !w_packed) {
    // one row: fragments of W straight from memory; eight waves on the gate rows, eight on the up rows
    launch_skinny<2, 8, 4, true>(xb, wb, out, ep, M, N, K, stream);
  } else if (M <= 32) {
    if (N >= 65536 && !w_packed) rc = launch_tiled<32, 32, 256, 1, 1, true>(xb, wb, out, ep, M, N, K, stream);
    else if (K % 128 == 0) rc = launch_direct<32, 64, 128, 1, 2, true>(xb, wt, out, ep, M, N, K, stream);
    else rc = launch_tiled<32, 64, 128, 1, 2, true>(xb, wb, out, ep, M, N, K, stream);
  } else if (M <= 64) {
    if (K % 128 == 0) rc = launch_direct<64, 128, 128, 2, 2, true, 3>(xb, wt, out, ep, M, N, K, stream);
    else rc = launch_tiled<64, 64, 128, 2, 2, true>(xb, wb, out, ep, M, N, K, stream);
  } else if (M <= 256 && K % 64 == 0) {
    // 65 to 256 rows: still bound by reading W.  All of x in one tile, so that W is read once; k-tiles of 64 in a
    // ring of three or four, so that a workgroup has 60 to 80 KB under way.  Measured for gate+up of an 8B layer
    // (N = 24576, K = 4096) against the smallest of the large tiles: 128 rows 66 -> 46 us (96 rows of W a
    // workgroup: 256 workgroups), 192 rows 72 -> 57, 256 rows 80 -> 62; from 320 rows on the large tiles win
    // (98 against 110 us and more).
    if (M <= 128) rc = launch_direct<128, 96, 64, 4, 1, true, 4>(xb, wt, out, ep, M, N, K, stream);
    else if (M <= 192) rc = launch_direct<192, 128, 64, 2, 2, true, 3>(xb, wt, out, ep, M, N, K, stream);
    else rc = launch_direct<256, 128, 64, 4, 2, true, 3>(xb, wt, out, ep, M, N, K, stream);
  } else {
    rc = launch_large<true>(xb, wt, out, ep, M, N, K, stream);
  }
  if (rc) return rc;
  SYN_LAUNCH_CHECK("gemm_swiglu");
  return 0;
}

// The products above for up to 16 rows of x over wp, a copy of W [N, K] in fragment order (see
// gemm_packed_kernel; N a multiple of 16, K of 32).  out_code: 1 = bf16 [M, N], 2 = float [M, N];
// paired: W holds gate and up rows in turns of 16 and out is bf16 [M, N / 2] = act(gate) * up.
// slices > 1 (float out, not paired): out is [slices, M, N], slice s holds the sum over its part of K.
// The norm between two such products (RowNorm above):
//   ss [M, ss_groups] float (or null): the sums of row m are multiplied by rsqrt(sum(ss[m, :]) / norm_dim + eps);
//   resid [M, N] float (or null; then float sums, one slice, not paired, `out` unused): resid += sums,
//   xs [M, N] bf16 = (gain_offset + gain[n]) * resid, ss_out [M, N / 16] = sums of resid^2 over groups of 16 columns.
SYN_EXPORT int syn_gemm_packed_norm(const void* x, const void* wp, void* out, int out_code, int M, int N, int K, int paired,
                                    int act, int slices, const float* ss, int ss_groups, int norm_dim, float eps,
                                    float* resid, void* xs, float* ss_out, const void* gain, int gain_is_f32,
                                    float gain_offset, hipStream_t stream) {
  SYN_CHECK(act >= 0 && act < SYN_ACT_COUNT, "gemm_packed: unknown activation code %d", act);
  SYN_CHECK(slices >= 1 && slices <= 64 && (slices == 1 || (out_code == 2 && !paired)),
            "gemm_packed: %d slices of K need a float output [slices, M, N] and no activation", slices);
  const Epilogue ep = {out_code == 2, act};
  SYN_CHECK(M > 0 && M <= 16 && N > 0 && K > 0, "gemm_packed: M = %d (1 .. 16), N = %d, K = %d", M, N, K);
  SYN_CHECK(N % 16 == 0 && K % 32 == 0 && (!paired || N % 32 == 0),
            "gemm_packed: N = %d must be a multiple of 16 (32 for paired rows), K = %d of 32", N, K);
  SYN_CHECK(out_code == 1 || out_code == 2, "gemm_packed: unknown output code %d", out_code);
  SYN_CHECK(!paired || out_code == 1, "gemm_packed: the gated product is stored as bf16");
  SYN_CHECK((uintptr_t)x % 16 == 0 && (uintptr_t)wp % 16 == 0, "gemm_packed: operands must be 16-byte aligned");
  RowNorm rn = {};
  if (ss) {
    SYN_CHECK(ss_groups > 0 && norm_dim > 0, "gemm_packed: %d groups of a row statistic over %d columns", ss_groups, norm_dim);
    rn.ss = ss, rn.ss_groups = ss_groups, rn.inv_dim = 1.f / (float)norm_dim, rn.eps = eps;
  }
  if (resid) {
    SYN_CHECK(!paired && slices == 1 && out_code == 2 && xs && ss_out && gain,
              "gemm_packed: the product before a norm is one slice of float sums with xs, ss_out and a gain");
    rn.resid = resid, rn.xs = (bf16*)xs, rn.ss_out = ss_out, rn.gain = gain, rn.gain_is_f32 = gain_is_f32;
    rn.gain_offset = gain_offset;
  }
  const bf16* xb = (const bf16*)x;
  const bf16* wb = (const bf16*)wp;
  // from sweeps at N = 4096 .. 151936, K = 4096 and 12288, 1 and 8 rows
  // gate and up rows of the same outputs: from 5 rows of x on a wave takes both (a fragment of x is then loaded
  // once for two products: a decode step of 8 sequences 3.88 -> 3.80 ms; at one row 3.30 -> 3.31 ms, at four
  // within the differences between boxes).  The same for the narrow products (two groups of rows a wave, twice
  // the slices of K) gained under 1 % at 8 sequences and lost as much at 4.
  if (paired && M >= 5) launch_packed2<16, 2, true>(xb, wb, out, ep, M, N, K, stream, 1, rn);
  else if (paired) launch_packed<2, 8, 4, true>(xb, wb, out, ep, M, N, K, stream, 1, rn);
  else if (N <= 8192) launch_packed<1, 16, 2>(xb, wb, out, ep, M, N, K, stream, slices, rn);
  // very wide (the output head): from 5 rows of x on two groups of rows a wave as well (N = 151936, K = 4096 at 8 rows:
  // 193 -> 182 us; at one row 175 -> 179; three or four groups a wave, or deeper, lose again; N = 10240 in two slices
  // of K: 18.9 -> 20.0 us, so only where W is very wide)
  else if (M >= 5 && N >= 32768) launch_packed2<8, 4>(xb, wb, out, ep, M, N, K, stream, slices, rn);
  else launch_packed<1, 8, 8>(xb, wb, out, ep, M, N, K, stream, slices, rn);
  SYN_LAUNCH_CHECK("gemm_packed");
  return 0;
}

SYN_EXPORT int syn_gemm_packed(const void* x, const void* wp, void* out, int out_code, int M, int N, int K, int paired,
                               int act, int slices, hipStream_t stream) {
  return syn_gemm_packed_norm(x, wp, out, out_code, M, N, K, paired, act, slices, nullptr, 0, 0, 0.f, nullptr, nullptr,
                              nullptr, nullptr, 0, 0.f, stream);
}
