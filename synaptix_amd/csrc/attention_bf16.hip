// bf16 attention over the paged cache on MFMA, compiled once for each head size (-DSYN_HD=...).
//
// Cache pages hold 64 tokens: k_pages[page, kv_head, token, d] and, transposed so that both MFMA
// operands are contiguous along the contraction, v_pages[page, kv_head, d, token].
//
// The kernels compute S^T = K . Q^T for a block of 64 keys, so that a lane's accumulator values
// (4 keys, one query column) are exactly the B operand that O^T += V^T . P^T needs: the
// probabilities never leave registers.
//   v_mfma_f32_16x16x32_bf16 : A[i=lane%16][k=8*(lane/16)+e], B[k=8*(lane/16)+e][n=lane%16]
//   v_mfma_f32_16x16x16_bf16 : A[i=lane%16][k=4*(lane/16)+e], B[k=4*(lane/16)+e][n=lane%16]
//   both                     : D[i=4*(lane/16)+e][n=lane%16]
// Scores, maxima, exponentials and sums are 32-bit; P is rounded to bf16 for the second product
// (as crates/synaptix-kernels-cuda/src/cu/fused/attention/flash_splitq.cu:187-600 does); the output
// is rounded once.
//
//   prefill: a workgroup of 4 waves takes 128 query rows of one (sequence, head); a wave 32 of them.
//   decode : a wave takes (sequence, kv head, up to 16 heads of its group, one split of the keys);
//            the heads of a group share every K/V load.  A second kernel merges the splits.
// Reference counterparts: flash_splitq.cu (prefill), flash_decode.cu:92-205,340-387 (split + merge,
// one block a q-head there, scalar dot products).
#include "common.h"

#ifndef SYN_HD
#error "compile with -DSYN_HD=<head size>"
#endif
SYN_DEFINE_ERROR_CHANNEL

constexpr int HD = SYN_HD;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head sizes in steps of 16 up to 256");
constexpr int KS32 = HD / 32;
constexpr bool TAIL16 = (HD % 32) != 0;
constexpr int DT = HD / 16;

SYN_EXPORT int syn_attention_head_dim() { return HD; }

struct QFrag {
  bf16x8 k32[KS32 > 0 ? KS32 : 1];
  bf16x4 k16;
};

__device__ __forceinline__ f32x4 mfma16(bf16x4 a, bf16x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c,
                                                   0, 0, 0);
}

__device__ __forceinline__ void load_q(QFrag& f, const bf16* qptr, int lane) {
  const bf16x8 z8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bf16x4 z4 = {0, 0, 0, 0};
#pragma unroll
  for (int ks = 0; ks < KS32; ++ks) f.k32[ks] = qptr ? *(const bf16x8*)(qptr + ks * 32 + 8 * (lane / 16)) : z8;
  if (TAIL16) f.k16 = qptr ? *(const bf16x4*)(qptr + KS32 * 32 + 4 * (lane / 16)) : z4;
}

template <int QB>
struct AttnState {
  f32x4 o[DT][QB];
  float m[QB];
  float l[QB];  // this lane's share of the sum; lanes of a column are added at the end
};

template <int QB>
__device__ __forceinline__ void attn_init(AttnState<QB>& st) {
#pragma unroll
  for (int c = 0; c < QB; ++c) {
    st.m[c] = -INFINITY;
    st.l[c] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) st.o[dt][c] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
}

// One block of 64 keys starting at key0.  qpos[c] / lo[c]: visible keys of this lane's column in
// column block c are lo <= key <= qpos (qpos < 0: the column is padding).  kv_len: keys at and
// beyond it hold no data of this sequence.
template <int QB>
__device__ __forceinline__ void attn_block(AttnState<QB>& st, const QFrag (&qf)[QB], const bf16* __restrict__ kpage,
                                           const bf16* __restrict__ vpage, int key0, const int (&qpos)[QB],
                                           const int (&lo)[QB], int kv_len, float scale, int lane) {
  const int r16 = lane % 16, g4 = lane / 16;
  f32x4 s[4][QB];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
#pragma unroll
    for (int c = 0; c < QB; ++c) s[t][c] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const bf16* krow = kpage + (size_t)(t * 16 + r16) * HD;
#pragma unroll
    for (int ks = 0; ks < KS32; ++ks) {
      const bf16x8 a = *(const bf16x8*)(krow + ks * 32 + 8 * g4);
#pragma unroll
      for (int c = 0; c < QB; ++c) s[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[c].k32[ks], s[t][c], 0, 0, 0);
    }
    if (TAIL16) {
      const bf16x4 a = *(const bf16x4*)(krow + KS32 * 32 + 4 * g4);
#pragma unroll
      for (int c = 0; c < QB; ++c) s[t][c] = mfma16(a, qf[c].k16, s[t][c]);
    }
  }
#pragma unroll
  for (int c = 0; c < QB; ++c) {
    float mloc = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = key0 + t * 16 + 4 * g4 + e;
        float v = s[t][c][e] * scale;
        if (key > qpos[c] || key < lo[c]) v = -INFINITY;
        s[t][c][e] = v;
        mloc = fmaxf(mloc, v);
      }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, SYN_WAVE));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, SYN_WAVE));
    const float m_new = fmaxf(st.m[c], mloc);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a column that has seen no key yet
    const float alpha = __expf(st.m[c] - m_use);
    st.m[c] = m_new;
    float lsum = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float p = __expf(s[t][c][e] - m_use);
        s[t][c][e] = p;
        lsum += p;
      }
    st.l[c] = st.l[c] * alpha + lsum;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) st.o[dt][c] *= alpha;
  }
  const bool ragged = key0 + SYN_PAGE > kv_len;  // only the sequence's last page
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    bf16x4 pb[QB];
#pragma unroll
    for (int c = 0; c < QB; ++c)
#pragma unroll
      for (int e = 0; e < 4; ++e) pb[c][e] = (bf16)s[t][c][e];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      bf16x4 av = *(const bf16x4*)(vpage + (size_t)(dt * 16 + r16) * SYN_PAGE + t * 16 + 4 * g4);
      if (ragged) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (key0 + t * 16 + 4 * g4 + e >= kv_len) av[e] = (bf16)0.f;  // 0 * (whatever lies there) must be 0
      }
#pragma unroll
      for (int c = 0; c < QB; ++c) st.o[dt][c] = mfma16(av, pb[c], st.o[dt][c]);
    }
  }
}

// ------------------------------------------------------------------ prefill
constexpr int PF_QB = 2;                   // 16-column blocks a wave
constexpr int PF_WAVES = 4;
constexpr int PF_ROWS = PF_WAVES * PF_QB * 16;  // query rows a workgroup

__global__ void __launch_bounds__(PF_WAVES * SYN_WAVE)
attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                    const int* __restrict__ page_table, int table_stride, const int* __restrict__ seq_start,
                    const int* __restrict__ seq_past, int n_seqs, bf16* __restrict__ out, float scale, int window,
                    int nh, int nkv) {
  // which sequence and which rows: tiles are numbered sequence by sequence
  int seq = -1, q0 = 0, t = 0;
  for (int s = 0; s < n_seqs; ++s) {
    const int nt = (seq_start[s + 1] - seq_start[s] + PF_ROWS - 1) / PF_ROWS;
    if ((int)blockIdx.x < t + nt) {
      seq = s;
      q0 = ((int)blockIdx.x - t) * PF_ROWS;
      break;
    }
    t += nt;
  }
  if (seq < 0) return;
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int head = blockIdx.y, kvh = head / (nh / nkv);
  const int tok0 = seq_start[seq], n_new = seq_start[seq + 1] - tok0, past = seq_past[seq];
  const int r0 = q0 + wave * PF_QB * 16;
  if (r0 >= n_new) return;
  const int kv_len = past + n_new;

  QFrag qf[PF_QB];
  int qpos[PF_QB], lo[PF_QB];
#pragma unroll
  for (int c = 0; c < PF_QB; ++c) {
    const int row = r0 + c * 16 + lane % 16;
    const bool valid = row < n_new;
    qpos[c] = valid ? past + row : -1;
    lo[c] = (window > 0 && valid) ? max(0, qpos[c] - window + 1) : 0;
    load_q(qf[c], valid ? q + ((size_t)(tok0 + row) * nh + head) * HD : nullptr, lane);
  }
  AttnState<PF_QB> st;
  attn_init(st);
  const int kmax = past + min(r0 + PF_QB * 16 - 1, n_new - 1);
  const int kmin = window > 0 ? max(0, past + r0 - window + 1) : 0;
  for (int kb = kmin / SYN_PAGE; kb <= kmax / SYN_PAGE; ++kb) {
    const size_t base = ((size_t)page_table[(size_t)seq * table_stride + kb] * nkv + kvh) * SYN_PAGE * HD;
    attn_block<PF_QB>(st, qf, k_pages + base, v_pages + base, kb * SYN_PAGE, qpos, lo, kv_len, scale, lane);
  }
#pragma unroll
  for (int c = 0; c < PF_QB; ++c) {
    float l = st.l[c];
    l += __shfl_xor(l, 16, SYN_WAVE);
    l += __shfl_xor(l, 32, SYN_WAVE);
    if (qpos[c] < 0) continue;
    const float inv = 1.f / l;
    bf16* orow = out + ((size_t)(tok0 + r0 + c * 16 + lane % 16) * nh + head) * HD + 4 * (lane / 16);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (bf16)(st.o[dt][c][e] * inv);
      *(bf16x4*)(orow + dt * 16) = v;
    }
  }
}

SYN_EXPORT int syn_attention_prefill_bf16(const void* q, const void* k_pages, const void* v_pages,
                                          const int* page_table, int table_stride, const int* seq_start,
                                          const int* seq_past, int n_seqs, int n_tokens, void* out, float scale,
                                          int window, int nh, int nkv, int hd, hipStream_t stream) {
  SYN_CHECK(hd == HD, "attention_prefill: library built for head size %d, called with %d", HD, hd);
  SYN_CHECK(n_seqs > 0 && n_tokens >= n_seqs && nh > 0 && nkv > 0, "attention_prefill: empty input");
  SYN_CHECK(nh % nkv == 0, "attention_prefill: %d heads do not divide into %d kv heads", nh, nkv);
  SYN_CHECK(nh <= 65535, "attention_prefill: %d heads exceed the grid", nh);
  const int tiles = n_tokens / PF_ROWS + n_seqs;  // an upper bound; surplus workgroups leave at once
  attn_prefill_kernel<<<dim3(tiles, nh), PF_WAVES * SYN_WAVE, 0, stream>>>(
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_start, seq_past, n_seqs,
      (bf16*)out, scale, window, nh, nkv);
  SYN_LAUNCH_CHECK("attention_prefill");
  return 0;
}

// ------------------------------------------------------------------ decode: split over keys, then merge
// partial[(seq * nh + head) * n_splits + split] = { m, l, o[HD] } in float.
constexpr int PART = HD + 2;

__global__ void __launch_bounds__(SYN_WAVE)
attn_decode_split_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages,
                         const bf16* __restrict__ v_pages, const int* __restrict__ page_table, int table_stride,
                         const int* __restrict__ seq_len, float* __restrict__ partial, float scale, int window, int nh,
                         int nkv, int n_splits) {
  const int lane = threadIdx.x;
  const int seq = blockIdx.x, split = blockIdx.z;
  const int g = nh / nkv, chunks = (g + 15) / 16;
  const int kvh = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
  const int kv_len = seq_len[seq], pos = kv_len - 1;
  const int hg = chunk * 16 + lane % 16;  // head inside the group
  const bool valid = hg < g;
  const int head = kvh * g + hg;

  QFrag qf[1];
  int qpos[1], lo[1];
  qpos[0] = valid ? pos : -1;
  lo[0] = window > 0 ? max(0, pos - window + 1) : 0;
  load_q(qf[0], valid ? q + ((size_t)seq * nh + head) * HD : nullptr, lane);
  AttnState<1> st;
  attn_init(st);
  const int b_lo = lo[0] / SYN_PAGE, b_hi = pos / SYN_PAGE;
  const int per = (b_hi - b_lo + n_splits) / n_splits;  // ceil((b_hi - b_lo + 1) / n_splits)
  const int b0 = b_lo + split * per, b1 = min(b_hi + 1, b0 + per);
  for (int kb = b0; kb < b1; ++kb) {
    const size_t base = ((size_t)page_table[(size_t)seq * table_stride + kb] * nkv + kvh) * SYN_PAGE * HD;
    attn_block<1>(st, qf, k_pages + base, v_pages + base, kb * SYN_PAGE, qpos, lo, kv_len, scale, lane);
  }
  float l = st.l[0];
  l += __shfl_xor(l, 16, SYN_WAVE);
  l += __shfl_xor(l, 32, SYN_WAVE);
  if (!valid) return;
  float* p = partial + ((size_t)(seq * nh + head) * n_splits + split) * PART;
  if (lane / 16 == 0) {
    p[0] = st.m[0];
    p[1] = l;
  }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 4; ++e) p[2 + dt * 16 + 4 * (lane / 16) + e] = st.o[dt][0][e];
}

__global__ void __launch_bounds__(SYN_WAVE)
attn_decode_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out, int n_splits) {
  const int row = blockIdx.x, lane = threadIdx.x;  // row = seq * nh + head
  const float* p = partial + (size_t)row * n_splits * PART;
  float m = -INFINITY;
  for (int s = 0; s < n_splits; ++s) m = fmaxf(m, p[(size_t)s * PART]);
  float l = 0.f;
  float o[(HD + SYN_WAVE - 1) / SYN_WAVE] = {};
  for (int s = 0; s < n_splits; ++s) {
    const float ms = p[(size_t)s * PART];
    if (ms == -INFINITY) continue;  // a split that had no keys
    const float w = __expf(ms - m);
    l += w * p[(size_t)s * PART + 1];
#pragma unroll
    for (int i = 0; i < (HD + SYN_WAVE - 1) / SYN_WAVE; ++i) {
      const int d = lane + i * SYN_WAVE;
      if (d < HD) o[i] += w * p[(size_t)s * PART + 2 + d];
    }
  }
#pragma unroll
  for (int i = 0; i < (HD + SYN_WAVE - 1) / SYN_WAVE; ++i) {
    const int d = lane + i * SYN_WAVE;
    if (d < HD) out[(size_t)row * HD + d] = (bf16)(o[i] / l);
  }
}

// workspace: n_seqs * nh * n_splits * (HD + 2) floats
SYN_EXPORT int syn_attention_decode_bf16(const void* q, const void* k_pages, const void* v_pages,
                                         const int* page_table, int table_stride, const int* seq_len, int n_seqs,
                                         void* out, float* workspace, int n_splits, float scale, int window, int nh,
                                         int nkv, int hd, hipStream_t stream) {
  SYN_CHECK(hd == HD, "attention_decode: library built for head size %d, called with %d", HD, hd);
  SYN_CHECK(n_seqs > 0 && nh > 0 && nkv > 0 && n_splits > 0, "attention_decode: empty input");
  SYN_CHECK(nh % nkv == 0, "attention_decode: %d heads do not divide into %d kv heads", nh, nkv);
  const int chunks = (nh / nkv + 15) / 16;
  SYN_CHECK(nkv * chunks <= 65535 && n_splits <= 65535, "attention_decode: grid too large");
  attn_decode_split_kernel<<<dim3(n_seqs, nkv * chunks, n_splits), SYN_WAVE, 0, stream>>>(
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_len, workspace, scale,
      window, nh, nkv, n_splits);
  SYN_LAUNCH_CHECK("attention_decode_split");
  attn_decode_merge_kernel<<<n_seqs * nh, SYN_WAVE, 0, stream>>>(workspace, (bf16*)out, n_splits);
  SYN_LAUNCH_CHECK("attention_decode_merge");
  return 0;
}
