// Row kernels that move little data per flop: embedding gather, RMSNorm with the
// residual sum fused in, SwiGLU, and the fused per-head q/k norm + rotation + cache write.
//
// Reference counterparts (one kernel each there, several fused here):
//   crates/synaptix-kernels-cuda/src/cu/embed/embed.cu:18-46
//   crates/synaptix-kernels-cuda/src/cu/reduction/rms_norm.cu:65-98
//   crates/synaptix-kernels-cuda/src/cu/fused/norm/rmsnorm_residual.cu:97-159
//   crates/synaptix-kernels-cuda/src/cu/fused/mlp/silu_and_mul.cu:11-52
//   crates/synaptix-kernels-cuda/src/cu/elementwise/rope.cu:27-70, kv_append.cu:32-78
#include "common.h"

SYN_DEFINE_ERROR_CHANNEL

// ------------------------------------------------------------------ embedding
// resid[n, :] = table[ids[n], :] widened to float.  Ids are checked on the host.
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ resid,
                             int H) {
  const int n = blockIdx.x;
  const T* row = table + (size_t)ids[n] * H;
  float* out = resid + (size_t)n * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_f32<T>(row[i]);
}

// the same from a bf16 table in fragment order ([V / 16][H / 32][64 lanes][8], as the products read the tied
// output head): eight consecutive values of a row are one lane's 16 bytes
__global__ void embed_packed_kernel(const bf16* __restrict__ table, const int* __restrict__ ids, float* __restrict__ resid,
                                    int H) {
  const int n = blockIdx.x, id = ids[n];
  const bf16* group = table + (size_t)(id / 16) * H * 16;   // the 16 rows around row id: H / 32 fragments of 512 values
  float* out = resid + (size_t)n * H;
  for (int c = threadIdx.x; c < H / 8; c += blockDim.x) {   // chunk c: values 8 c .. 8 c + 7 of the row
    const bf16x8 v = *(const bf16x8*)(group + (size_t)(c / 4) * 512 + ((c % 4) * 16 + id % 16) * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[c * 8 + e] = (float)v[e];
  }
}

// table_kind: 0 = bf16 rows, 1 = float rows, 2 = bf16 in fragment order (V a multiple of 16, H of 32)
SYN_EXPORT int syn_embed(const void* table, int table_kind, const int* ids, float* resid, int n_tokens, int H,
                         hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && H > 0, "embed: empty input (%d tokens, width %d)", n_tokens, H);
  SYN_CHECK(table_kind >= 0 && table_kind <= 2, "embed: unknown kind of table %d", table_kind);
  if (table_kind == 1) {
    embed_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)table, ids, resid, H);
  } else if (table_kind == 2) {
    SYN_CHECK(H % 32 == 0, "embed: a table in fragment order has a width that is a multiple of 32, not %d", H);
    embed_packed_kernel<<<n_tokens, 256, 0, stream>>>((const bf16*)table, ids, resid, H);
  } else {
    embed_kernel<bf16><<<n_tokens, 256, 0, stream>>>((const bf16*)table, ids, resid, H);
  }
  SYN_LAUNCH_CHECK("embed");
  return 0;
}

// ------------------------------------------------------------------ residual sum + RMSNorm
// rows == nullptr: for every row r: resid[r] += delta[r] (if delta), out[r] = norm(resid[r]).
// rows != nullptr: out[i] = norm(resid[rows[i]] + delta[rows[i]]); resid stays as it is.
// delta may come as n_parts partial sums [n_parts][n_rows][H] (a product cut along K); they are
// added in order.  The sum, the mean of squares and the scaling are 32-bit; one rounding at the store.
template <typename TOut>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const float* __restrict__ delta, int n_parts,
                                   size_t part_stride, const int* __restrict__ rows, const void* __restrict__ gain,
                                   int gain_is_f32, float gain_offset, float eps, TOut* __restrict__ out, int H) {
  __shared__ float red[16];
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)r * H;
  const float* d = delta ? delta + (size_t)r * H : nullptr;
  TOut* o = out + (size_t)blockIdx.x * H;
  const bool write_back = (rows == nullptr) && (d != nullptr);
  auto summed = [&](int i) {
    float v = x[i];
    if (d)
      for (int p = 0; p < n_parts; ++p) v += d[p * part_stride + i];
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = summed(i);
    if (write_back) x[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = write_back ? x[i] : summed(i);
    o[i] = from_f32<TOut>(load_gain(gain, gain_is_f32, i, gain_offset) * v * inv);
  }
}

// The same for rows whose width is a multiple of 4 and at most 4 * VPT * blockDim: every thread
// keeps its values (float4 loads) in registers between the sum of squares and the scaling.  The
// partial sums are fetched eight at a time, so that their loads are in flight together, and
// added in their order.
__device__ inline float4 load_gain4(const void* gain, int gain_is_f32, int i4) {
  if (gain_is_f32) return ((const float4*)gain)[i4];
  struct alignas(8) bf16x4s { bf16 e[4]; };
  const bf16x4s g = ((const bf16x4s*)gain)[i4];
  return make_float4((float)g.e[0], (float)g.e[1], (float)g.e[2], (float)g.e[3]);
}

__device__ inline void store4(float* o, int i4, const float4 r) { ((float4*)o)[i4] = r; }
__device__ inline void store4(bf16* o, int i4, const float4 r) {
  struct alignas(8) bf16x4s { bf16 e[4]; } t;
  t.e[0] = (bf16)r.x;
  t.e[1] = (bf16)r.y;
  t.e[2] = (bf16)r.z;
  t.e[3] = (bf16)r.w;
  ((bf16x4s*)o)[i4] = t;
}

template <typename TOut, int VPT>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ resid, const float* __restrict__ delta, int n_parts,
                                       size_t part_stride, const int* __restrict__ rows,
                                       const void* __restrict__ gain, int gain_is_f32, float gain_offset, float eps,
                                       TOut* __restrict__ out, int H) {
  __shared__ float red[16];
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float4* x = (float4*)(resid + (size_t)r * H);
  const float4* d = delta ? (const float4*)(delta + (size_t)r * H) : nullptr;
  TOut* o = out + (size_t)blockIdx.x * H;
  const bool write_back = (rows == nullptr) && (d != nullptr);
  const int H4 = H / 4;
  const size_t stride4 = part_stride / 4;
  float4 v[VPT], g[VPT];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i < H4) {
      v[j] = x[i];
      g[j] = load_gain4(gain, gain_is_f32, i);  // fetched here, beside the values, not after the sum
      g[j].x += gain_offset, g[j].y += gain_offset, g[j].z += gain_offset, g[j].w += gain_offset;
      if (d) {
        for (int p0 = 0; p0 < n_parts; p0 += 8) {
          float4 t[8];
#pragma unroll
          for (int q = 0; q < 8; ++q)
            t[q] = p0 + q < n_parts ? d[(size_t)(p0 + q) * stride4 + i] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            v[j].x += t[q].x;
            v[j].y += t[q].y;
            v[j].z += t[q].z;
            v[j].w += t[q].w;
          }
        }
      }
      if (write_back) x[i] = v[j];
      ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    }
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)H + eps);
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i < H4)
      store4(o, i, make_float4(g[j].x * v[j].x * inv, g[j].y * v[j].y * inv, g[j].z * v[j].z * inv,
                               g[j].w * v[j].w * inv));
  }
}

SYN_EXPORT int syn_add_rmsnorm(float* resid, const float* delta, int n_parts, int n_rows, const int* rows, int n_out,
                               const void* gain, int gain_is_f32, float gain_offset, float eps, void* out,
                               int out_is_f32, int H, hipStream_t stream) {
  SYN_CHECK(n_out > 0 && H > 0 && n_rows > 0, "add_rmsnorm: empty input (%d rows, width %d)", n_out, H);
  SYN_CHECK(n_parts >= 1 && n_parts <= 64, "add_rmsnorm: %d partial sums", n_parts);
  const size_t stride = (size_t)n_rows * H;
  const bool vec = H % 4 == 0 && H <= 4 * 4 * 1024 && ((uintptr_t)resid % 16 == 0) && ((uintptr_t)delta % 16 == 0) &&
                   ((uintptr_t)out % 16 == 0) && ((uintptr_t)gain % 16 == 0);
  if (vec) {
    const int H4 = H / 4;
    const int block = H4 <= 256 ? 256 : (H4 <= 512 ? 512 : 1024);
    const int vpt = (H4 + block - 1) / block;  // 1 .. 4
#define SYN_ARN(T, V)                                                                                          \
  add_rmsnorm_vec_kernel<T, V><<<n_out, block, 0, stream>>>(resid, delta, n_parts, stride, rows, gain, gain_is_f32, \
                                                            gain_offset, eps, (T*)out, H)
    if (out_is_f32) {
      if (vpt == 1) SYN_ARN(float, 1); else if (vpt == 2) SYN_ARN(float, 2); else SYN_ARN(float, 4);
    } else {
      if (vpt == 1) SYN_ARN(bf16, 1); else if (vpt == 2) SYN_ARN(bf16, 2); else SYN_ARN(bf16, 4);
    }
#undef SYN_ARN
  } else {
    const int block = H >= 4096 ? 1024 : (H >= 1024 ? 512 : 256);
    if (out_is_f32)
      add_rmsnorm_kernel<float><<<n_out, block, 0, stream>>>(resid, delta, n_parts, stride, rows, gain, gain_is_f32,
                                                            gain_offset, eps, (float*)out, H);
    else
      add_rmsnorm_kernel<bf16><<<n_out, block, 0, stream>>>(resid, delta, n_parts, stride, rows, gain, gain_is_f32,
                                                           gain_offset, eps, (bf16*)out, H);
  }
  SYN_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// ------------------------------------------------------------------ RMSNorm of rows of any width
// One wave a row.
template <typename T>
__global__ void rmsnorm_rows_kernel(const T* __restrict__ x, const void* __restrict__ gain, int gain_is_f32,
                                    float gain_offset, float eps, T* __restrict__ out, int n_rows, int width) {
  const int row = blockIdx.x * (blockDim.x / SYN_WAVE) + threadIdx.x / SYN_WAVE;
  if (row >= n_rows) return;
  const int lane = threadIdx.x % SYN_WAVE;
  const T* xr = x + (size_t)row * width;
  T* o = out + (size_t)row * width;
  float ss = 0.f;
  for (int i = lane; i < width; i += SYN_WAVE) {
    float v = to_f32<T>(xr[i]);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)width + eps);
  for (int i = lane; i < width; i += SYN_WAVE)
    o[i] = from_f32<T>(load_gain(gain, gain_is_f32, i, gain_offset) * to_f32<T>(xr[i]) * inv);
}

SYN_EXPORT int syn_rmsnorm_rows(const void* x, int is_f32, const void* gain, int gain_is_f32, float gain_offset,
                                float eps, void* out, int n_rows, int width, hipStream_t stream) {
  SYN_CHECK(n_rows > 0 && width > 0, "rmsnorm_rows: empty input (%d rows, width %d)", n_rows, width);
  const int wpb = 4;
  const int grid = (n_rows + wpb - 1) / wpb;
  if (is_f32)
    rmsnorm_rows_kernel<float><<<grid, wpb * SYN_WAVE, 0, stream>>>((const float*)x, gain, gain_is_f32, gain_offset,
                                                                    eps, (float*)out, n_rows, width);
  else
    rmsnorm_rows_kernel<bf16><<<grid, wpb * SYN_WAVE, 0, stream>>>((const bf16*)x, gain, gain_is_f32, gain_offset,
                                                                   eps, (bf16*)out, n_rows, width);
  SYN_LAUNCH_CHECK("rmsnorm_rows");
  return 0;
}

// ------------------------------------------------------------------ SwiGLU on a fused [gate | up] row
// out[n, i] = act(gu[n, i]) * gu[n, I + i] in 32-bit (gate_activation; silu(z) = z / (1 + exp(-z))).
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_rows, int I, int act) {
  const size_t total = (size_t)n_rows * I;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t n = idx / I;
    const int i = (int)(idx - n * I);
    const float g = to_f32<T>(gu[n * 2 * I + i]);
    const float u = to_f32<T>(gu[n * 2 * I + I + i]);
    out[idx] = from_f32<T>(gated(act, g, u));
  }
}

// 8 values a thread with 16-byte loads (bf16, width a multiple of 8)
__global__ void swiglu_vec8_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int n_rows, int I, int act) {
  const int I8 = I / 8;
  const size_t total = (size_t)n_rows * I8;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t n = idx / I8;
    const int i = (int)(idx - n * I8) * 8;
    const bf16x8 g = *(const bf16x8*)(gu + n * 2 * I + i);
    const bf16x8 u = *(const bf16x8*)(gu + n * 2 * I + I + i);
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)gated(act, (float)g[e], (float)u[e]);
    *(bf16x8*)(out + n * I + i) = o;
  }
}

SYN_EXPORT int syn_swiglu(const void* gu, void* out, int is_f32, int n_rows, int I, int act, hipStream_t stream) {
  SYN_CHECK(n_rows > 0 && I > 0, "swiglu: empty input (%d rows, width %d)", n_rows, I);
  SYN_CHECK(act >= 0 && act < SYN_ACT_COUNT, "swiglu: unknown activation code %d", act);
  if (!is_f32 && I % 8 == 0 && (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const size_t total = (size_t)n_rows * (I / 8);
    int grid = (int)((total + 255) / 256);
    if (grid > 65536) grid = 65536;
    swiglu_vec8_kernel<<<grid, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, n_rows, I, act);
    SYN_LAUNCH_CHECK("swiglu");
    return 0;
  }
  const size_t total = (size_t)n_rows * I;
  int grid = (int)((total + 255) / 256);
  if (grid > 65536) grid = 65536;
  if (is_f32)
    swiglu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu, (float*)out, n_rows, I, act);
  else
    swiglu_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, n_rows, I, act);
  SYN_LAUNCH_CHECK("swiglu");
  return 0;
}

// ------------------------------------------------------------------ q/k norm + rotation + cache write
// One wave for each (token, head) of the fused projection row [q heads | k heads | v heads].
//   q: optional RMSNorm over the head, rotation at the token's position, stored to q_out[token, head, :]
//   k: the same, stored to the cache page of the token's sequence: k_pages[page, kv_head, pos % 64, :]
//   v: copied as it is, stored transposed inside the page:          v_pages[page, kv_head, :, pos % 64]
// Rotation (half-split layout over the first `rot` dims, the rest passes through):
//   d < rot/2:        o[d] = x[d] cos[p, d]         - x[d + rot/2] sin[p, d]
//   rot/2 <= d < rot: o[d] = x[d] cos[p, d - rot/2] + x[d - rot/2] sin[p, d - rot/2]
// All arithmetic is 32-bit; each value is rounded once when stored.
// TIn = T, or float with n_parts >= 1 partial sums [n_parts][tokens][heads * hd] that are added first.
template <typename T, typename TIn>
__global__ void qk_norm_rope_kv_write_kernel(const TIn* __restrict__ qkv, int n_parts, size_t part_stride,
                                             T* __restrict__ q_out, T* __restrict__ k_pages,
                                             T* __restrict__ v_pages, const int* __restrict__ page_table,
                                             int table_stride, const int* __restrict__ tok_seq,
                                             const int* __restrict__ tok_pos, const void* __restrict__ q_gain,
                                             const void* __restrict__ k_gain, int gain_is_f32, float gain_offset,
                                             float eps, const float* __restrict__ cos_t,
                                             const float* __restrict__ sin_t, int rot, int nh, int nkv, int hd,
                                             int write_kv) {
  extern __shared__ float lds[];  // [waves][hd]
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int heads = nh + 2 * nkv;
  const int tok = blockIdx.x;
  const int head = blockIdx.y * (blockDim.x / SYN_WAVE) + wave;
  // no early return: every wave reaches the barrier; a layer that reads another layer's cache
  // (write_kv == 0) only needs its q heads
  const bool active = head < (write_kv ? heads : nh);
  float* xs = lds + wave * hd;
  const int pos = tok_pos[tok];
  const bool is_q = head < nh, is_k = !is_q && head < nh + nkv;
  const void* gain = is_q ? q_gain : (is_k ? k_gain : nullptr);

  if (active) {
    const TIn* src = qkv + ((size_t)tok * heads + head) * hd;
    float ss = 0.f;
    for (int d = 2 * lane; d < hd; d += 2 * SYN_WAVE) {  // head sizes are even: two values a lane
      float v0 = to_f32<TIn>(src[d]), v1 = to_f32<TIn>(src[d + 1]);
      for (int p = 1; p < n_parts; ++p) {
        v0 += to_f32<TIn>(src[p * part_stride + d]);
        v1 += to_f32<TIn>(src[p * part_stride + d + 1]);
      }
      xs[d] = v0;
      xs[d + 1] = v1;
      ss += v0 * v0 + v1 * v1;
    }
    if (gain) {
      ss = wave_sum(ss);
      const float inv = rsqrtf(ss / (float)hd + eps);
      for (int d = 2 * lane; d < hd; d += 2 * SYN_WAVE) {
        xs[d] = load_gain(gain, gain_is_f32, d, gain_offset) * xs[d] * inv;
        xs[d + 1] = load_gain(gain, gain_is_f32, d + 1, gain_offset) * xs[d + 1] * inv;
      }
    }
  }
  __syncthreads();  // lanes read what other lanes of their wave wrote
  if (!active) return;

  T* dst;
  size_t dst_stride = 1;
  bool v_in_mfma_order = false;   // a bf16 V page is kept in the order of v_page_offset
  if (is_q) {
    dst = q_out + ((size_t)tok * nh + head) * hd;
  } else {
    const int kvh = is_k ? head - nh : head - nh - nkv;
    const int page = page_table[(size_t)tok_seq[tok] * table_stride + pos / SYN_PAGE];
    const size_t base = ((size_t)page * nkv + kvh) * SYN_PAGE * hd;
    if (is_k) {
      dst = k_pages + base + (size_t)(pos % SYN_PAGE) * hd;
    } else {
      dst = v_pages + base + (pos % SYN_PAGE);
      dst_stride = SYN_PAGE;
      if (sizeof(T) == 2) {
        dst = v_pages + base;
        v_in_mfma_order = true;
      }
    }
  }
  const bool rotate = (is_q || is_k) && cos_t != nullptr;
  const int half = rot / 2;
  auto rotated = [&](int d) {
    float o = xs[d];
    if (rotate && d < rot) {
      if (d < half) {
        const float c = cos_t[(size_t)pos * half + d], s = sin_t[(size_t)pos * half + d];
        o = xs[d] * c - xs[d + half] * s;
      } else {
        const float c = cos_t[(size_t)pos * half + d - half], s = sin_t[(size_t)pos * half + d - half];
        o = xs[d] * c + xs[d - half] * s;
      }
    }
    return o;
  };
  for (int d = 2 * lane; d < hd; d += 2 * SYN_WAVE) {
    if (v_in_mfma_order) {
      dst[v_page_offset(hd, d, pos % SYN_PAGE)] = from_f32<T>(rotated(d));
      dst[v_page_offset(hd, d + 1, pos % SYN_PAGE)] = from_f32<T>(rotated(d + 1));
    } else {
      dst[(size_t)d * dst_stride] = from_f32<T>(rotated(d));
      dst[(size_t)(d + 1) * dst_stride] = from_f32<T>(rotated(d + 1));
    }
  }
}

// The same for the q and k heads of bf16 rows whose head size is 8 * LPH with LPH = 2, 4, .. 32 lanes
// a head and whose rotation covers the whole head (or is absent): a lane holds 8 values of a head
// (16-byte load and store), the sum of squares is reduced over the LPH lanes of the head, and the
// partner of a rotated pair sits LPH / 2 lanes away.  A block takes 256 / LPH heads of one token.
// PARTS: the rows come as n_parts float partial sums [n_parts][tokens][heads * HD] of a product cut
// along K (part_stride elements apart), which are added first, in their order.
template <int LPH, bool PARTS>
__device__ __forceinline__ void
qk_heads_part(int block_x, int block_y, const void* __restrict__ qkv_in, int n_parts, size_t part_stride,
              bf16* __restrict__ q_out, bf16* __restrict__ k_pages,
                const int* __restrict__ page_table, int table_stride, const int* __restrict__ tok_seq,
                const int* __restrict__ tok_pos, const void* __restrict__ q_gain, const void* __restrict__ k_gain,
                int gain_is_f32, float gain_offset, float eps, const float* __restrict__ cos_t,
                const float* __restrict__ sin_t, int n_tokens, int nh, int nkv, int n_active) {
  constexpr int HD = LPH * 8, HPB = 256 / LPH, half = HD / 2;
  constexpr int TPB = 4;  // tokens a block takes, their loads in flight together
  const int head_raw = block_y * HPB + threadIdx.x / LPH;  // q heads, then k heads
  const int head = min(head_raw, n_active - 1);                // idle lanes repeat the last head: shuffles need them
  const int c = threadIdx.x % LPH;                             // which 8 values of the head
  const bool is_q = head < nh, low = c < LPH / 2;
  const void* gain = is_q ? q_gain : k_gain;
  float g[8];
  if (gain) {
    if (gain_is_f32) {
      const float4 g0 = ((const float4*)gain)[c * 2], g1 = ((const float4*)gain)[c * 2 + 1];
      g[0] = g0.x, g[1] = g0.y, g[2] = g0.z, g[3] = g0.w, g[4] = g1.x, g[5] = g1.y, g[6] = g1.z, g[7] = g1.w;
    } else {
      const bf16x8 gb = ((const bf16x8*)gain)[c];
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = (float)gb[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] += gain_offset;
  }
  float val[TPB][8];
  int pos[TPB];
  float4 cs[TPB][2], sn[TPB][2];
  if constexpr (PARTS) {
#pragma unroll
    for (int t = 0; t < TPB; ++t) {
#pragma unroll
      for (int e = 0; e < 8; ++e) val[t][e] = 0.f;
      pos[t] = tok_pos[min(block_x * TPB + t, n_tokens - 1)];
    }
    for (int p = 0; p < n_parts; ++p) {
      float4 lo4[TPB], hi4[TPB];     // the tokens' loads of one part in flight together
#pragma unroll
      for (int t = 0; t < TPB; ++t) {
        const int tok = min(block_x * TPB + t, n_tokens - 1);
        const float4* src = (const float4*)((const float*)qkv_in + (size_t)p * part_stride +
                                            ((size_t)tok * (nh + 2 * nkv) + head) * HD + c * 8);
        lo4[t] = src[0], hi4[t] = src[1];
      }
#pragma unroll
      for (int t = 0; t < TPB; ++t) {
        val[t][0] += lo4[t].x, val[t][1] += lo4[t].y, val[t][2] += lo4[t].z, val[t][3] += lo4[t].w;
        val[t][4] += hi4[t].x, val[t][5] += hi4[t].y, val[t][6] += hi4[t].z, val[t][7] += hi4[t].w;
      }
    }
  } else {
    bf16x8 raw[TPB];
#pragma unroll
    for (int t = 0; t < TPB; ++t) {
      const int tok = min(block_x * TPB + t, n_tokens - 1);
      raw[t] = *(const bf16x8*)((const bf16*)qkv_in + ((size_t)tok * (nh + 2 * nkv) + head) * HD + c * 8);
      pos[t] = tok_pos[tok];
    }
#pragma unroll
    for (int t = 0; t < TPB; ++t)
#pragma unroll
      for (int e = 0; e < 8; ++e) val[t][e] = (float)raw[t][e];
  }
  if (cos_t) {
#pragma unroll
    for (int t = 0; t < TPB; ++t) {
      const float4* c4 = (const float4*)(cos_t + (size_t)pos[t] * half + (low ? c : c - LPH / 2) * 8);
      const float4* s4 = (const float4*)(sin_t + (size_t)pos[t] * half + (low ? c : c - LPH / 2) * 8);
      cs[t][0] = c4[0], cs[t][1] = c4[1], sn[t][0] = s4[0], sn[t][1] = s4[1];
    }
  }
#pragma unroll
  for (int t = 0; t < TPB; ++t) {
    const int tok = block_x * TPB + t;
    float v[8];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[e] = val[t][e];
      ss += v[e] * v[e];
    }
    if (gain) {
#pragma unroll
      for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, SYN_WAVE);
      const float inv = rsqrtf(ss / (float)HD + eps);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = g[e] * v[e] * inv;
    }
    if (cos_t) {
      const float cc[8] = {cs[t][0].x, cs[t][0].y, cs[t][0].z, cs[t][0].w, cs[t][1].x, cs[t][1].y, cs[t][1].z, cs[t][1].w};
      const float sc[8] = {sn[t][0].x, sn[t][0].y, sn[t][0].z, sn[t][0].w, sn[t][1].x, sn[t][1].y, sn[t][1].z, sn[t][1].w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float partner = __shfl_xor(v[e], LPH / 2, SYN_WAVE);
        v[e] = low ? v[e] * cc[e] - partner * sc[e] : v[e] * cc[e] + partner * sc[e];
      }
    }
    if (head_raw >= n_active || tok >= n_tokens) continue;
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)v[e];
    if (is_q) {
      *(bf16x8*)(q_out + ((size_t)tok * nh + head) * HD + c * 8) = o;
    } else {
      const int page = page_table[(size_t)tok_seq[tok] * table_stride + pos[t] / SYN_PAGE];
      *(bf16x8*)(k_pages + (((size_t)page * nkv + (head - nh)) * SYN_PAGE + pos[t] % SYN_PAGE) * HD + c * 8) = o;
    }
  }
}

// The v heads of the same rows: 64 tokens x 32 dims a block go through LDS and are written in the
// order of v_page_offset, in which 8 consecutive positions of one dim are one 16-byte piece and the
// 16 dims of a fragment follow each other at 16 bytes.
#define V_DIMS 32
template <bool PARTS>   // as for qk_heads_part
__device__ __forceinline__ void
v_block_write_part(int block_x, int block_y, int block_z, const void* __restrict__ qkv_in, int n_parts,
                   size_t part_stride, bf16* __restrict__ v_pages, const int* __restrict__ page_table,
                     int table_stride, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, int n_tokens,
                     int nh, int nkv, int hd) {
  constexpr int LD = V_DIMS + 2, PAIRS = V_DIMS / 2;
  __shared__ __attribute__((aligned(16))) bf16 vtile[64 * LD];
  __shared__ size_t dst_base[SYN_PAGE];
  __shared__ int dst_slot[SYN_PAGE];
  const int tid = threadIdx.x, t0 = block_x * 64, kvh = block_y, d0 = block_z * V_DIMS;
  const int heads = nh + 2 * nkv;
  for (int idx = tid; idx < 64 * PAIRS; idx += 256) {
    const int j = idx / PAIRS, pr = idx % PAIRS;
    if (t0 + j < n_tokens && d0 + 2 * pr < hd) {   // head sizes are even
      const size_t at = ((size_t)(t0 + j) * heads + nh + nkv + kvh) * hd + d0 + 2 * pr;
      if constexpr (PARTS) {
        float2 sum = make_float2(0.f, 0.f);
        for (int p = 0; p < n_parts; ++p) {
          const float2 v = *(const float2*)((const float*)qkv_in + (size_t)p * part_stride + at);
          sum.x += v.x, sum.y += v.y;
        }
        vtile[j * LD + 2 * pr] = (bf16)sum.x, vtile[j * LD + 2 * pr + 1] = (bf16)sum.y;
      } else {
        *(uint32_t*)(vtile + j * LD + 2 * pr) = *(const uint32_t*)((const bf16*)qkv_in + at);
      }
    }
  }
  if (tid < 64 && t0 + tid < n_tokens) {
    const int tok = t0 + tid, pos = tok_pos[tok];
    const int page = page_table[(size_t)tok_seq[tok] * table_stride + pos / SYN_PAGE];
    dst_base[tid] = ((size_t)page * nkv + kvh) * SYN_PAGE * hd;
    dst_slot[tid] = pos % SYN_PAGE;
  }
  __syncthreads();
  const int j = tid % 64;
  if (t0 + j < n_tokens)
    for (int d = tid / 64; d < V_DIMS && d0 + d < hd; d += 4)
      v_pages[dst_base[j] + v_page_offset(hd, d0 + d, dst_slot[j])] = vtile[j * LD + d];
}

// Both in one launch: the first qk_x * qk_y workgroups take the q and k heads, the others the v tiles
// (v_x * nkv * v_z of them, none where the layer writes no cache).
template <int LPH, bool PARTS>
__global__ void __launch_bounds__(256)
qkv_prompt_kernel(int qk_x, int qk_y, int v_x, const void* __restrict__ qkv, int n_parts, size_t part_stride,
                  bf16* __restrict__ q_out, bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                  const int* __restrict__ page_table, int table_stride, const int* __restrict__ tok_seq,
                  const int* __restrict__ tok_pos, const void* __restrict__ q_gain, const void* __restrict__ k_gain,
                  int gain_is_f32, float gain_offset, float eps, const float* __restrict__ cos_t,
                  const float* __restrict__ sin_t, int n_tokens, int nh, int nkv, int n_active) {
  const int b = blockIdx.x, n_qk = qk_x * qk_y;
  if (b < n_qk) {
    qk_heads_part<LPH, PARTS>(b % qk_x, b / qk_x, qkv, n_parts, part_stride, q_out, k_pages, page_table, table_stride,
                              tok_seq, tok_pos, q_gain, k_gain, gain_is_f32, gain_offset, eps, cos_t, sin_t, n_tokens,
                              nh, nkv, n_active);
  } else {
    const int c = b - n_qk;
    v_block_write_part<PARTS>(c % v_x, (c / v_x) % nkv, c / (v_x * nkv), qkv, n_parts, part_stride, v_pages, page_table,
                              table_stride, tok_seq, tok_pos, n_tokens, nh, nkv, LPH * 8);
  }
}

SYN_EXPORT int syn_qk_norm_rope_kv_write(const void* qkv, int n_parts, void* q_out, void* k_pages, void* v_pages,
                                         int is_f32, const int* page_table, int table_stride, const int* tok_seq,
                                         const int* tok_pos, const void* q_gain, const void* k_gain, int gain_is_f32,
                                         float gain_offset, float eps, const float* cos_t, const float* sin_t, int rot,
                                         int n_tokens, int nh, int nkv, int hd, int write_kv, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && nh > 0 && nkv > 0 && hd > 0, "qk_norm_rope_kv_write: empty input");
  SYN_CHECK(rot % 2 == 0 && rot >= 0 && rot <= hd, "qk_norm_rope_kv_write: rotary size %d does not fit head size %d",
            rot, hd);
  SYN_CHECK(hd % 2 == 0, "qk_norm_rope_kv_write: head size %d is odd", hd);
  SYN_CHECK((cos_t == nullptr) == (sin_t == nullptr), "qk_norm_rope_kv_write: cos and sin come together");
  SYN_CHECK(n_parts >= 0 && n_parts <= 64, "qk_norm_rope_kv_write: %d partial sums", n_parts);
  // prompts in bf16: the kernels that move 16 bytes a lane, where the head size and the rotation allow them
  const int lph = hd / 8;
  // (partial sums of up to 64 tokens stay with the kernel below, one wave a head: measured a little faster there)
  const bool fast = !is_f32 && (n_parts == 0 || n_tokens > 64) && hd % 8 == 0 && lph >= 2 && lph <= 32 && (lph & (lph - 1)) == 0 &&
                    (cos_t == nullptr || rot == hd) && (uintptr_t)qkv % 16 == 0 && (uintptr_t)q_out % 16 == 0 &&
                    (uintptr_t)k_pages % 16 == 0 && (uintptr_t)q_gain % 16 == 0 && (uintptr_t)k_gain % 16 == 0 &&
                    (uintptr_t)cos_t % 16 == 0 && (uintptr_t)sin_t % 16 == 0;
  if (fast) {
    const int n_active = write_kv ? nh + nkv : nh;
    const int hpb = 256 / lph;
    const int qk_x = (n_tokens + 3) / 4, qk_y = (n_active + hpb - 1) / hpb;
    const int v_x = (n_tokens + 63) / 64, v_blocks = write_kv ? v_x * nkv * ((hd + V_DIMS - 1) / V_DIMS) : 0;
    const size_t part_stride = (size_t)n_tokens * (nh + 2 * nkv) * hd;
    const long grid = (long)qk_x * qk_y + v_blocks;
    SYN_CHECK(grid <= 0x7fffffffL, "qk_norm_rope_kv_write: %d tokens are too many for one launch", n_tokens);
#define SYN_QKV(L)                                                                                                  \
  if (n_parts > 0)                                                                                                  \
    qkv_prompt_kernel<L, true><<<(unsigned)grid, 256, 0, stream>>>(                                                 \
        qk_x, qk_y, v_x, qkv, n_parts, part_stride, (bf16*)q_out, (bf16*)k_pages, (bf16*)v_pages, page_table,       \
        table_stride, tok_seq, tok_pos, q_gain, k_gain, gain_is_f32, gain_offset, eps, cos_t, sin_t, n_tokens, nh,  \
        nkv, n_active);                                                                                             \
  else                                                                                                              \
    qkv_prompt_kernel<L, false><<<(unsigned)grid, 256, 0, stream>>>(                                                \
        qk_x, qk_y, v_x, qkv, 0, 0, (bf16*)q_out, (bf16*)k_pages, (bf16*)v_pages, page_table, table_stride, tok_seq, \
        tok_pos, q_gain, k_gain, gain_is_f32, gain_offset, eps, cos_t, sin_t, n_tokens, nh, nkv, n_active)
    switch (lph) {
      case 2: SYN_QKV(2); break;
      case 4: SYN_QKV(4); break;
      case 8: SYN_QKV(8); break;
      case 16: SYN_QKV(16); break;
      default: SYN_QKV(32); break;
    }
#undef SYN_QKV
    SYN_LAUNCH_CHECK("qkv_prompt");
    return 0;
  }
  const int wpb = 4;
  const int heads = nh + 2 * nkv;
  dim3 grid(n_tokens, (heads + wpb - 1) / wpb);
  const size_t lds = (size_t)wpb * hd * sizeof(float);
  const size_t stride = (size_t)n_tokens * heads * hd;
#define SYN_QK(T, TIn)                                                                                             \
  qk_norm_rope_kv_write_kernel<T, TIn><<<grid, wpb * SYN_WAVE, lds, stream>>>(                                     \
      (const TIn*)qkv, n_parts > 0 ? n_parts : 1, stride, (T*)q_out, (T*)k_pages, (T*)v_pages, page_table,          \
      table_stride, tok_seq, tok_pos, q_gain, k_gain, gain_is_f32, gain_offset, eps, cos_t, sin_t, rot, nh, nkv, hd,   \
      write_kv)
  if (is_f32)
    SYN_QK(float, float);
  else if (n_parts > 0)
    SYN_QK(bf16, float);
  else
    SYN_QK(bf16, bf16);
#undef SYN_QK
  SYN_LAUNCH_CHECK("qk_norm_rope_kv_write");
  return 0;
}
