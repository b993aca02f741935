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
// Which key a row of a 16-row score tile stands for is free, as long as the masks and the V^T
// fragments follow: tile t = 2h + u of a block covers, for lane group g = lane / 16, the keys
// 32h + 8g + 4u .. + 3.  The two tiles of a half h then give a lane the probabilities of the 8
// consecutive keys 32h + 8g .. + 7: the B operand of one 16x16x32 step, whose V^T fragment is one
// 16-byte load.
// Scores, maxima, exponentials and sums are 32-bit; P is rounded to bf16 for the second product
// (as crates/synaptix-kernels-cuda/src/cu/fused/attention/flash_splitq.cu:187-600 does); the output
// is rounded once.
//
//   prefill: a workgroup of 8 waves takes 128 query rows of one (sequence, head); a wave 16 of them.
//   decode : a workgroup takes (sequence, kv head, up to 16 heads of its group, one split of the keys);
//            the heads of a group share every K/V load and the waves share the split's blocks.
//            A second kernel merges the splits when there is more than one.
// Reference counterparts: flash_splitq.cu (prefill), flash_decode.cu:92-205,340-387 (split + merge,
// one block a q-head there, scalar dot products).
#include "common.h"

#ifndef SYN_HD
#error "compile with -DSYN_HD=<head size>"
#endif
SYN_DEFINE_ERROR_CHANNEL

constexpr int HD = SYN_HD;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head sizes in steps of 16 up to 256");
constexpr bool TAIL16 = (HD % 32) != 0;
constexpr int DT = HD / 16;

SYN_EXPORT int syn_attention_head_dim() { return HD; }

// Fragments of Q (or of a K row block) along the head dimension.  Head sizes that are a multiple of
// 32 take k-steps of 32 (16x16x32); the others take k-steps of 16 throughout (16x16x16): one
// accumulation chain never mixes the two shapes.
constexpr int KSTEPS = TAIL16 ? HD / 16 : HD / 32;
constexpr int KW = TAIL16 ? 4 : 8;  // elements a lane holds for one k-step
typedef __attribute__((ext_vector_type(KW))) __bf16 kfrag_t;

struct QFrag {
  kfrag_t k[KSTEPS];
};

__device__ __forceinline__ f32x4 mfma16(bf16x4 a, bf16x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c,
                                                   0, 0, 0);
}

__device__ __forceinline__ f32x4 mfma_qk(bf16x4 a, bf16x4 b, f32x4 c) { return mfma16(a, b, c); }
__device__ __forceinline__ f32x4 mfma_qk(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// key (inside its block of 64) that row r of score tile t stands for, and that element e of lane
// group g's accumulator of tile t belongs to
__device__ __forceinline__ int tile_row_key(int t, int r) { return (t / 2) * 32 + 8 * (r / 4) + 4 * (t % 2) + r % 4; }
__device__ __forceinline__ int acc_key(int t, int g, int e) { return (t / 2) * 32 + 8 * g + 4 * (t % 2) + e; }

// where the row of key k lies when a block's K rows are stored tile after tile (the inverse of tile_row_key)
__device__ __forceinline__ int tile_slot(int k) { return 16 * (2 * (k / 32) + (k % 8) / 4) + 4 * ((k % 32) / 8) + k % 4; }

// the fragments of one row of HD elements: in k-step ks, lane group g = lane / 16 holds elements ks*4*KW + KW*g .. + KW
__device__ __forceinline__ void load_row(kfrag_t (&f)[KSTEPS], const bf16* row, int lane) {
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) f[ks] = *(const kfrag_t*)(row + ks * (4 * KW) + KW * (lane / 16));
}

__device__ __forceinline__ void load_q(QFrag& f, const bf16* qptr, int lane) {
  if (qptr) {
    load_row(f.k, qptr, lane);
  } else {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int e = 0; e < KW; ++e) f.k[ks][e] = (bf16)0.f;
  }
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

// ------------------------------------------------------------------ prefill
// A workgroup of 8 waves takes 128 query rows of one (sequence, head), a wave 16 of them; two waves
// share a SIMD, so that one multiplies while the other waits for LDS or memory.  Blocks of 64 keys go through LDS, double-buffered: while the waves work on one block the
// next one is on its way from memory into registers.  K lies in LDS as [64 keys, in tile order][HD + 8], V^T as
// [HD][64 + 8]; the paddings keep the 16-lane fragment reads free of bank conflicts.
// Softmax runs in the exp2 domain (scores times scale * log2 e); masking is applied only to blocks
// that reach beyond a row's causal limit, the window's start or the sequence's end.
// PV takes k-steps of 32 keys (see the key permutation above).
constexpr float RESCALE_AT = 8.f;
constexpr int PF_QB = 1;                        // 16-column blocks a wave
constexpr int PF_WAVES = 8;
constexpr int PF_THREADS = PF_WAVES * SYN_WAVE;
constexpr int PF_ROWS = PF_WAVES * PF_QB * 16;  // query rows a workgroup
constexpr int LDK = HD + 8;
constexpr int LDV = SYN_PAGE + 8;
constexpr int PF_TILE = SYN_PAGE * LDK + HD * LDV;          // bf16 elements of one buffer
constexpr int PF_CHUNKS = (8 * HD + PF_THREADS - 1) / PF_THREADS;  // 16-byte chunks a thread moves for K (and for V)

__global__ void __launch_bounds__(PF_THREADS)
attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                    const int* __restrict__ page_table, int table_stride, const int* __restrict__ seq_start,
                    const int* __restrict__ seq_past, int n_seqs, int n_tiles, bf16* __restrict__ out, float scale,
                    int window, int nh, int nkv) {
  extern __shared__ __attribute__((aligned(16))) bf16 lds[];  // [2][PF_TILE]
  // which sequence and which rows: tiles are numbered sequence by sequence; the grid runs through
  // them backwards so that the tiles with the most key blocks start first
  const int tile = n_tiles - 1 - (int)blockIdx.x;
  int seq = -1, q0 = 0, t_acc = 0;
  for (int s = 0; s < n_seqs; ++s) {
    const int nt = (seq_start[s + 1] - seq_start[s] + PF_ROWS - 1) / PF_ROWS;
    if (tile < t_acc + nt) {
      seq = s;
      q0 = (tile - t_acc) * PF_ROWS;
      break;
    }
    t_acc += nt;
  }
  if (seq < 0) return;  // the grid is an upper bound
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE;
  const int r16 = lane % 16, g4 = lane / 16;
  const int head = blockIdx.y, kvh = head / (nh / nkv);
  const int tok0 = seq_start[seq], n_new = seq_start[seq + 1] - tok0, past = seq_past[seq];
  const int kv_len = past + n_new;
  const int r0 = q0 + wave * PF_QB * 16;
  const bool wave_on = r0 < n_new;

  QFrag qf[PF_QB];
  int qpos[PF_QB], lo[PF_QB];
#pragma unroll
  for (int c = 0; c < PF_QB; ++c) {
    const int row = r0 + c * 16 + r16;
    const bool valid = row < n_new;
    qpos[c] = valid ? past + row : -1;
    lo[c] = (window > 0 && valid) ? max(0, qpos[c] - window + 1) : 0;
    load_q(qf[c], valid ? q + ((size_t)(tok0 + row) * nh + head) * HD : nullptr, lane);
  }
  // visible keys of this wave, and of the whole workgroup
  const int w_kmax = past + min(r0 + PF_QB * 16 - 1, n_new - 1);
  const int w_qmin = past + r0;                                        // smallest position of the wave
  const int w_kmin = window > 0 ? max(0, w_qmin - window + 1) : 0;
  const int g_kmax = past + min(q0 + PF_ROWS - 1, n_new - 1);
  const int g_kmin = window > 0 ? max(0, past + q0 - window + 1) : 0;
  const int kb_lo = g_kmin / SYN_PAGE, kb_hi = g_kmax / SYN_PAGE;
  const float scale2 = scale * 1.44269504088896340736f;

  AttnState<PF_QB> st;
  attn_init(st);

  bf16x8 rk[PF_CHUNKS], rv[PF_CHUNKS];
  auto fetch = [&](int kb) {
    const size_t base = ((size_t)page_table[(size_t)seq * table_stride + kb] * nkv + kvh) * SYN_PAGE * HD;
    const bf16* kp = k_pages + base;
    const bf16* vp = v_pages + base;
#pragma unroll
    for (int i = 0; i < PF_CHUNKS; ++i) {
      const int c = tid + i * PF_THREADS;
      if (c < 8 * HD) {
        rk[i] = *(const bf16x8*)(kp + (size_t)c * 8);   // K rows are contiguous: chunk c is elements 8c .. 8c+7
        rv[i] = *(const bf16x8*)(vp + (size_t)c * 8);   // and so are the rows of V^T
      }
    }
  };
  auto stash = [&](int buf, int kb) {
    bf16* ks = lds + buf * PF_TILE;
    bf16* vs = ks + SYN_PAGE * LDK;
    const bool ragged = (kb + 1) * SYN_PAGE > kv_len;
#pragma unroll
    for (int i = 0; i < PF_CHUNKS; ++i) {
      const int c = tid + i * PF_THREADS;
      if (c < 8 * HD) {
        const int key = c / (HD / 8), kcol = c % (HD / 8);
        *(bf16x8*)(ks + tile_slot(key) * LDK + kcol * 8) = rk[i];
        const int vrow = c / 8, vcol = c % 8;
        bf16x8 v = rv[i];
        if (ragged) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (kb * SYN_PAGE + vcol * 8 + e >= kv_len) v[e] = (bf16)0.f;  // 0 * (whatever lies there) must be 0
        }
        *(bf16x8*)(vs + vrow * LDV + vcol * 8) = v;
      }
    }
  };

  fetch(kb_lo);
  stash(0, kb_lo);
  __syncthreads();
  for (int kb = kb_lo; kb <= kb_hi; ++kb) {
    const int buf = (kb - kb_lo) & 1;
    if (kb < kb_hi) fetch(kb + 1);
    const int key0 = kb * SYN_PAGE;
    if (wave_on && key0 <= w_kmax && key0 + SYN_PAGE > w_kmin) {
      const bf16* ks = lds + buf * PF_TILE;
      const bf16* vs = ks + SYN_PAGE * LDK;
      f32x4 s[4][PF_QB];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int c = 0; c < PF_QB; ++c) s[t][c] = (f32x4){0.f, 0.f, 0.f, 0.f};
        kfrag_t ka[KSTEPS];
        load_row(ka, ks + (t * 16 + r16) * LDK, lane);  // rows lie in LDS in tile order
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk)
#pragma unroll
          for (int c = 0; c < PF_QB; ++c) s[t][c] = mfma_qk(ka[kk], qf[c].k[kk], s[t][c]);
      }
      // a block needs masking if some row of the wave does not see all of it
      const bool need_mask = key0 + SYN_PAGE - 1 > w_qmin ||                   // beyond some row's own position
                             (window > 0 && key0 < w_kmax - window + 1) ||    // before some row's window
                             r0 + PF_QB * 16 > n_new;                         // rows of padding
#pragma unroll
      for (int c = 0; c < PF_QB; ++c) {
        float mloc = -INFINITY;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v = s[t][c][e] * scale2;
            if (need_mask) {
              const int key = key0 + acc_key(t, g4, e);
              if (key > qpos[c] || key < lo[c]) v = -INFINITY;
            }
            s[t][c][e] = v;
            mloc = fmaxf(mloc, v);
          }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16, SYN_WAVE));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, SYN_WAVE));
        // st.m is the reference of the exponents, not the exact maximum: it is only raised when a
        // block exceeds it by more than RESCALE_AT (in log2 units), so that the accumulators are
        // rescaled in few blocks.  Probabilities then reach at most 2^RESCALE_AT, well inside
        // float and bf16 range; the final division by the sum removes the common factor.
        const bool raise = mloc > st.m[c] + RESCALE_AT || (st.m[c] == -INFINITY && mloc > -INFINITY);
        if (__any(raise)) {  // same decision for the whole wave: columns that stay get alpha = 1
          const float m_new = raise ? mloc : st.m[c];
          const float alpha = raise ? __builtin_amdgcn_exp2f(st.m[c] - m_new) : 1.f;  // from -inf: 0
          st.m[c] = m_new;
          st.l[c] *= alpha;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) st.o[dt][c] *= alpha;
        }
        const float m_use = st.m[c] == -INFINITY ? 0.f : st.m[c];  // a column that has seen no key yet
        float lsum = 0.f;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float p = __builtin_amdgcn_exp2f(s[t][c][e] - m_use);
            s[t][c][e] = p;
            lsum += p;
          }
        st.l[c] += lsum;
      }
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        bf16x8 pb[PF_QB];
#pragma unroll
        for (int c = 0; c < PF_QB; ++c)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            pb[c][e] = (bf16)s[2 * tt][c][e];
            pb[c][4 + e] = (bf16)s[2 * tt + 1][c][e];
          }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const bf16x8 av = *(const bf16x8*)(vs + (dt * 16 + r16) * LDV + tt * 32 + 8 * g4);
#pragma unroll
          for (int c = 0; c < PF_QB; ++c) st.o[dt][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pb[c], st.o[dt][c], 0, 0, 0);
        }
      }
    }
    if (kb < kb_hi) stash(buf ^ 1, kb + 1);  // the other buffer was last read before the previous barrier
    __syncthreads();
  }
  if (!wave_on) return;
#pragma unroll
  for (int c = 0; c < PF_QB; ++c) {
    float l = st.l[c];
    l += __shfl_xor(l, 16, SYN_WAVE);
    l += __shfl_xor(l, 32, SYN_WAVE);
    if (qpos[c] < 0) continue;
    const float inv = 1.f / l;
    bf16* orow = out + ((size_t)(tok0 + r0 + c * 16 + r16) * nh + head) * HD + 4 * g4;
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
  const size_t lds = (size_t)2 * PF_TILE * sizeof(bf16);
  static bool raised = false;
  if (lds > 65536 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds);
    SYN_CHECK(e == hipSuccess, "attention_prefill: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
    raised = true;
  }
  attn_prefill_kernel<<<dim3(tiles, nh), PF_THREADS, lds, stream>>>(
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_start, seq_past, n_seqs,
      tiles, (bf16*)out, scale, window, nh, nkv);
  SYN_LAUNCH_CHECK("attention_prefill");
  return 0;
}

// ------------------------------------------------------------------ decode: split over keys, then merge
// A workgroup of up to 8 waves takes (sequence, kv head, up to 16 heads of its group, one split of
// the key blocks); its waves take the split's blocks in turn and their states are combined in LDS.
// With one split the workgroup writes the output itself; else it writes a partial
//   partial[(seq * nh + head) * n_splits + split] = { m, l, o[HD] }   (float)
// and a second kernel merges the splits.
constexpr int PART = HD + 2;
constexpr int DEC_MAX_WAVES = HD > 128 ? 4 : 8;  // as many as keep their ~190 registers each without spilling

// Like attn_block for one column block, but every K and V fragment of the block is requested before
// the first product needs one: a block costs one trip to memory instead of two.
__device__ __forceinline__ void attn_block_decode(AttnState<1>& st, const QFrag& qf, const bf16* __restrict__ kpage,
                                                  const bf16* __restrict__ vpage, int key0, int qpos, int lo,
                                                  int kv_len, float scale, int lane) {
  const int r16 = lane % 16, g4 = lane / 16;
  kfrag_t ka[4][KSTEPS];
  bf16x8 va[2][DT];
#pragma unroll
  for (int t = 0; t < 4; ++t) load_row(ka[t], kpage + (size_t)tile_row_key(t, r16) * HD, lane);
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) va[h][dt] = *(const bf16x8*)(vpage + (size_t)(dt * 16 + r16) * SYN_PAGE + h * 32 + 8 * g4);

  f32x4 s[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    s[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) s[t] = mfma_qk(ka[t][ks], qf.k[ks], s[t]);
  }
  float mloc = -INFINITY;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int key = key0 + acc_key(t, g4, e);
      float v = s[t][e] * scale;
      if (key > qpos || key < lo) v = -INFINITY;
      s[t][e] = v;
      mloc = fmaxf(mloc, v);
    }
  mloc = fmaxf(mloc, __shfl_xor(mloc, 16, SYN_WAVE));
  mloc = fmaxf(mloc, __shfl_xor(mloc, 32, SYN_WAVE));
  const float m_new = fmaxf(st.m[0], mloc);
  const float m_use = m_new == -INFINITY ? 0.f : m_new;
  const float alpha = __expf(st.m[0] - m_use);
  st.m[0] = m_new;
  float lsum = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float p = __expf(s[t][e] - m_use);
      s[t][e] = p;
      lsum += p;
    }
  st.l[0] = st.l[0] * alpha + lsum;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) st.o[dt][0] *= alpha;
  const bool ragged = key0 + SYN_PAGE > kv_len;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    bf16x8 pb;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      pb[e] = (bf16)s[2 * h][e];
      pb[4 + e] = (bf16)s[2 * h + 1][e];
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      bf16x8 av = va[h][dt];
      if (ragged) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (key0 + h * 32 + 8 * g4 + e >= kv_len) av[e] = (bf16)0.f;  // 0 * (whatever lies there) must be 0
      }
      st.o[dt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pb, st.o[dt][0], 0, 0, 0);
    }
  }
}

__global__ void __launch_bounds__(DEC_MAX_WAVES * SYN_WAVE)
attn_decode_split_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages,
                         const bf16* __restrict__ v_pages, const int* __restrict__ page_table, int table_stride,
                         const int* __restrict__ seq_len, float* __restrict__ partial, bf16* __restrict__ out,
                         float scale, int window, int nh, int nkv, int n_splits, int cols_alloc) {
  // LDS: sm[waves][16] running maxima, sl[waves][16] sums, so[waves][cols_alloc][HD + 4] outputs
  extern __shared__ float dec_lds[];
  const int n_waves = blockDim.x / SYN_WAVE;
  float* sm = dec_lds;
  float* sl = sm + n_waves * 16;
  float* so = sl + n_waves * 16;
  constexpr int SO_LD = HD + 4;
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int seq = blockIdx.x, split = blockIdx.z;
  const int g = nh / nkv, chunks = (g + 15) / 16;
  const int kvh = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
  const int kv_len = seq_len[seq], pos = kv_len - 1;
  const int col = lane % 16;
  const int hg = chunk * 16 + col;  // head inside the group
  const bool valid = hg < g;
  const int n_cols = min(16, g - chunk * 16);

  QFrag qf;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  load_q(qf, valid ? q + ((size_t)seq * nh + kvh * g + hg) * HD : nullptr, lane);
  AttnState<1> st;
  attn_init(st);
  const int b_lo = lo / SYN_PAGE, b_hi = pos / SYN_PAGE;
  const int per = (b_hi - b_lo + n_splits) / n_splits;  // ceil((b_hi - b_lo + 1) / n_splits)
  const int b0 = b_lo + split * per, b1 = min(b_hi + 1, b0 + per);
  for (int kb = b0 + wave; kb < b1; kb += n_waves) {
    const size_t base = ((size_t)page_table[(size_t)seq * table_stride + kb] * nkv + kvh) * SYN_PAGE * HD;
    attn_block_decode(st, qf, k_pages + base, v_pages + base, kb * SYN_PAGE, valid ? pos : -1, lo, kv_len, scale, lane);
  }
  float l = st.l[0];
  l += __shfl_xor(l, 16, SYN_WAVE);
  l += __shfl_xor(l, 32, SYN_WAVE);
  if (lane < 16) {
    sm[wave * 16 + lane] = st.m[0];
    sl[wave * 16 + lane] = l;
  }
  if (valid) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int e = 0; e < 4; ++e) so[((size_t)wave * cols_alloc + col) * SO_LD + dt * 16 + 4 * (lane / 16) + e] = st.o[dt][0][e];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < n_cols * HD; idx += blockDim.x) {
    const int c = idx / HD, d = idx % HD;
    float m = -INFINITY;
    for (int w = 0; w < n_waves; ++w) m = fmaxf(m, sm[w * 16 + c]);
    float acc = 0.f, lsum = 0.f;
    for (int w = 0; w < n_waves; ++w) {
      const float mw = sm[w * 16 + c];
      if (mw == -INFINITY) continue;  // a wave that had no block
      const float f = __expf(mw - m);
      acc += f * so[((size_t)w * cols_alloc + c) * SO_LD + d];
      lsum += f * sl[w * 16 + c];
    }
    const int head = kvh * g + chunk * 16 + c;
    if (n_splits == 1) {
      out[((size_t)seq * nh + head) * HD + d] = (bf16)(acc / lsum);
    } else {
      float* p = partial + ((size_t)(seq * nh + head) * n_splits + split) * PART;
      p[2 + d] = acc;
      if (d == 0) {
        p[0] = m;
        p[1] = lsum;
      }
    }
  }
}

// one wave a (sequence, head): lanes first share the splits' maxima and sums, then each takes output dims
__global__ void __launch_bounds__(SYN_WAVE)
attn_decode_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out, int n_splits) {
  const int row = blockIdx.x, lane = threadIdx.x;  // row = seq * nh + head
  const float* p = partial + (size_t)row * n_splits * PART;
  float wsum[(HD + SYN_WAVE - 1) / SYN_WAVE] = {};
  float l = 0.f;
  float m = -INFINITY;
  for (int s0 = 0; s0 < n_splits; s0 += SYN_WAVE) {  // maximum over all splits
    const int s = s0 + lane;
    m = fmaxf(m, s < n_splits ? p[(size_t)s * PART] : -INFINITY);
  }
  m = wave_max(m);
  for (int s0 = 0; s0 < n_splits; s0 += SYN_WAVE) {
    const int s = s0 + lane;
    const float ms = s < n_splits ? p[(size_t)s * PART] : -INFINITY;
    const float w = ms == -INFINITY ? 0.f : __expf(ms - m);  // a split that had no keys weighs nothing
    l += s < n_splits ? w * p[(size_t)s * PART + 1] : 0.f;
    const int cnt = min(SYN_WAVE, n_splits - s0);
    for (int j = 0; j < cnt; ++j) {
      const float wj = __shfl(w, j, SYN_WAVE);
      if (wj == 0.f) continue;
#pragma unroll
      for (int i = 0; i < (HD + SYN_WAVE - 1) / SYN_WAVE; ++i) {
        const int d = lane + i * SYN_WAVE;
        if (d < HD) wsum[i] += wj * p[(size_t)(s0 + j) * PART + 2 + d];
      }
    }
  }
  l = wave_sum(l);
#pragma unroll
  for (int i = 0; i < (HD + SYN_WAVE - 1) / SYN_WAVE; ++i) {
    const int d = lane + i * SYN_WAVE;
    if (d < HD) out[(size_t)row * HD + d] = (bf16)(wsum[i] / l);
  }
}

// workspace: n_seqs * nh * n_splits * (HD + 2) floats (unused with one split)
SYN_EXPORT int syn_attention_decode_bf16(const void* q, const void* k_pages, const void* v_pages,
                                         const int* page_table, int table_stride, const int* seq_len, int n_seqs,
                                         void* out, float* workspace, int n_splits, float scale, int window, int nh,
                                         int nkv, int hd, hipStream_t stream) {
  SYN_CHECK(hd == HD, "attention_decode: library built for head size %d, called with %d", HD, hd);
  SYN_CHECK(n_seqs > 0 && nh > 0 && nkv > 0 && n_splits > 0, "attention_decode: empty input");
  SYN_CHECK(nh % nkv == 0, "attention_decode: %d heads do not divide into %d kv heads", nh, nkv);
  const int chunks = (nh / nkv + 15) / 16;
  SYN_CHECK(nkv * chunks <= 65535 && n_splits <= 65535, "attention_decode: grid too large");
  // waves a workgroup: as many as the LDS for their states allows (up to 8), but no more than make
  // about 2,048 waves in all: at large batches four waves a workgroup are plenty
  const int cols_alloc = nh / nkv < 16 ? nh / nkv : 16;
  int waves = DEC_MAX_WAVES;
  while (waves > 2 && ((size_t)waves * (32 + (size_t)cols_alloc * (HD + 4)) * sizeof(float) > 64 * 1024 ||
                       (long)n_seqs * nkv * chunks * n_splits * waves > 2048))
    waves /= 2;
  if (waves < 4 && (size_t)4 * (32 + (size_t)cols_alloc * (HD + 4)) * sizeof(float) <= 64 * 1024) waves = 4;
  const size_t lds = (size_t)waves * (32 + (size_t)cols_alloc * (HD + 4)) * sizeof(float);
  attn_decode_split_kernel<<<dim3(n_seqs, nkv * chunks, n_splits), waves * SYN_WAVE, lds, stream>>>(
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_len, workspace,
      (bf16*)out, scale, window, nh, nkv, n_splits, cols_alloc);
  SYN_LAUNCH_CHECK("attention_decode_split");
  if (n_splits > 1) {
    attn_decode_merge_kernel<<<n_seqs * nh, SYN_WAVE, 0, stream>>>(workspace, (bf16*)out, n_splits);
    SYN_LAUNCH_CHECK("attention_decode_merge");
  }
  return 0;
}
