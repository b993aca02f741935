// bf16 attention over the paged cache on MFMA, compiled once for each head size (-DSYN_HD=...).
//
// Cache pages hold 64 tokens: k_pages[page, kv_head, token, d]; the hd x 64 values of a V page of one
// kv head lie in the order of v_page_offset: transposed, so that both MFMA operands are contiguous
// along the contraction, and fragment after fragment, so that a decode wave loads each as one
// contiguous 1 KB.
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
//   prefill: a workgroup takes 128 query rows of one (sequence, head); a wave 32 of them (16 for heads beyond 128).
//   decode : a workgroup takes (sequence, kv head, up to 16 heads of its group, one split of the keys);
//            the heads of a group share every K/V load and the waves share the split's blocks.
//            A second kernel merges the splits when there is more than one.
// Reference counterparts: flash_splitq.cu (prefill), flash_decode.cu:92-205,340-387 (split + merge,
// one block a q-head there, scalar dot products).
#include "common.h"
#include "no_alloc.h"

#ifndef SYN_HD
#error "compile with -DSYN_HD=<head size>"
#endif
SYN_DEFINE_ERROR_CHANNEL

constexpr int HD = SYN_HD;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head sizes in steps of 16 up to 256");
constexpr bool TAIL16 = (HD % 32) != 0;
constexpr int DT = HD / 16;

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
// A workgroup takes 128 query rows of one (sequence, head); two or more waves share a SIMD, so that one
// multiplies while the other waits for LDS or memory.  Blocks of 64 keys go through LDS,
// double-buffered: while the waves work on one block the next one is on its way from memory into registers.  K lies in LDS as [64 keys, in tile order][HD + 8], V^T as
// [HD][64 + 8]; the paddings keep the 16-lane fragment reads free of bank conflicts.
// Softmax runs in the exp2 domain (scores times scale * log2 e); masking is applied only to blocks
// that reach beyond a row's causal limit, the window's start or the sequence's end.
// PV takes k-steps of 32 keys (see the key permutation above).
constexpr float RESCALE_AT = 8.f;
// A wave takes 16 query rows and eight waves make a workgroup: 126 registers at a head size of 128, so
// that two workgroups share a compute unit.  (32 rows a wave would share every K and V fragment read
// from LDS between two column blocks, but need 256 registers: measured slower, 89 against 74 us at 2,048 tokens.)
constexpr int PF_QB = 1;      // 16-column blocks a wave
constexpr int PF_WAVES = 8;
constexpr int PF_THREADS = PF_WAVES * SYN_WAVE;
constexpr int PF_ROWS = PF_WAVES * PF_QB * 16;  // query rows a workgroup
constexpr int LDK = HD + 8;
constexpr int LDV = SYN_PAGE + 8;
constexpr int PF_TILE = SYN_PAGE * LDK + HD * LDV;          // bf16 elements of one buffer
constexpr int PF_CHUNKS = (8 * HD + PF_THREADS - 1) / PF_THREADS;  // 16-byte chunks a thread moves for K (and for V)

// Which sequence and which 128 query rows workgroup blockIdx.y takes: tiles are numbered sequence by
// sequence.  Two workgroups share a compute unit, and a tile's work grows with its number: the first
// half of the grid takes the tiles from the last downwards, the second half from the first upwards,
// so that the pairs that meet on a unit have about equal work.  False: the grid is an upper bound.
// Sequences with fewer new tokens than skip_below have no tiles (their rows of `out` are left as they are).
__device__ __forceinline__ bool prefill_tile(const int* __restrict__ seq_start, int n_seqs, int skip_below, int& seq, int& q0) {
  auto tiles_of = [&](int s) {
    const int n = seq_start[s + 1] - seq_start[s];
    return n < skip_below ? 0 : (n + PF_ROWS - 1) / PF_ROWS;
  };
  int total = 0;
  for (int s = 0; s < n_seqs; ++s) total += tiles_of(s);
  const int y = blockIdx.y, half = (total + 1) / 2;
  if (y >= total) return false;
  const int tile = y < half ? total - 1 - y : y - half;
  int t_acc = 0;
  for (int s = 0; s < n_seqs; ++s) {
    const int nt = tiles_of(s);
    if (tile < t_acc + nt) {
      seq = s;
      q0 = (tile - t_acc) * PF_ROWS;
      return true;
    }
    t_acc += nt;
  }
  return false;
}

__global__ void __launch_bounds__(PF_THREADS)
attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                    const int* __restrict__ page_table, int table_stride, const int* __restrict__ seq_start,
                    const int* __restrict__ seq_past, int n_seqs, bf16* __restrict__ out, float scale,
                    int window, int nh, int nkv, ScoreTerms terms, int skip_below) {
  extern __shared__ __attribute__((aligned(16))) bf16 lds[];  // [2][PF_TILE]
  // Heads run fastest through the grid; workgroups go round the eight dies in turn, and the heads are
  // dealt so that each die gets neighbouring heads, which share their K and V.
  int seq, q0;
  if (!prefill_tile(seq_start, n_seqs, skip_below, seq, q0)) return;
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE;
  const int r16 = lane % 16, g4 = lane / 16;
  const int hx = blockIdx.x;
  const int head = nh % 8 == 0 ? (hx % 8) * (nh / 8) + hx / 8 : hx, kvh = head / (nh / nkv);
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
  const bool with_terms = score_terms_on(terms);
  const float slope = terms.slopes ? terms.slopes[head] : 0.f;

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
        rv[i] = *(const bf16x8*)(vp + (size_t)c * 8);   // a V page is read as it lies and put in place by stash
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
        // chunk c of a V page is the fragment c / 64 = h * DT + dt of lane c % 64: dims 16 dt + lane % 16, tokens 32 h + 8 (lane / 16) .. + 8
        const int vrow = ((c / 64) % DT) * 16 + c % 16, vcol = ((c / 64) / DT) * 4 + (c % 64) / 16;
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
            if (with_terms)   // in natural units, then into the exponent's base
              v = score_with_terms(s[t][c][e] * scale, slope, terms.softcap, qpos[c], key0 + acc_key(t, g4, e)) *
                  1.44269504088896340736f;
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

// ------------------------------------------------------------------ prefill, 32 query rows a wave
// The same tiles of 128 query rows with v_mfma_f32_32x32x16_bf16 for both products, for head sizes 64
// and 128: a workgroup of four waves, each with 32 query rows.  A fragment of K or V read from LDS (1 KB)
// then feeds a product of 32 x 32 x 16 instead of 16 x 16 x 32: half the LDS reads for the same work,
// which is what bounded the waves of 16 rows (one fragment read for every MFMA).
//   A[i = lane % 32][k = 8 (lane / 32) + e], B[k = 8 (lane / 32) + e][n = lane % 32],
//   D[i = 8 (e / 4) + 4 (lane / 32) + e % 4][n = lane % 32], e = 0 .. 15
// S^T = K . Q^T in two tiles of 32 keys; row m of a tile stands for key pf2_row_key(m), chosen so that a
// lane's accumulator values e = 8j .. 8j + 7 are the 8 consecutive keys 16 j + 8 (lane / 32) .. + 7: they
// are, rounded to bf16, the B operand of O^T += V^T . P^T for k-step j, and the matching V^T fragment is
// one 16-byte piece of the page as it lies in memory.  Both K and V blocks therefore go into LDS as they
// are, by loads that write LDS directly (no registers, no store instructions): V verbatim (a fragment
// read covers runs of 256 consecutive bytes), K with the 16-byte chunks of each row swizzled, since its
// fragment reads touch 32 rows at the same column.
constexpr bool PF2_OK = HD == 64 || HD == 128;
constexpr int PF2_WAVES = 4;
constexpr int PF2_THREADS = PF2_WAVES * SYN_WAVE;
constexpr int PF2_KBYTES = SYN_PAGE * HD * 2;   // a block of K; a block of V is as large
constexpr int PF2_BUF = 2 * PF2_KBYTES;         // one buffer: K, then V
constexpr int PF2_CPR = HD / 8;                 // 16-byte chunks in a row of K
constexpr int PF2_KS = HD / 16;                 // k-steps of the scores
constexpr int PF2_AHEAD = 6;                    // fragment reads on their way ahead of the MFMA that takes them
constexpr int PF2_DT = HD >= 32 ? HD / 32 : 1;  // tiles of 32 output dims (the kernel is compiled for every head size, launched for two)
static_assert(PF_ROWS == PF2_WAVES * 32, "both prefill kernels take tiles of the same number of rows");

__device__ __forceinline__ int pf2_swizzle(int row) { return PF2_CPR == 16 ? (row & 15) : ((row >> 1) & 7); }
__device__ __forceinline__ int pf2_row_key(int m) { return 16 * (m / 16) + 8 * ((m % 8) / 4) + 4 * ((m % 16) / 8) + m % 4; }

__global__ void __launch_bounds__(PF2_THREADS, 2)
attn_prefill32_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                      const int* __restrict__ page_table, int table_stride, const int* __restrict__ seq_start,
                      const int* __restrict__ seq_past, int n_seqs, bf16* __restrict__ out, float scale,
                      int window, int nh, int nkv, int skip_below) {
  extern __shared__ __attribute__((aligned(16))) char lds2[];  // [2][K block | V block]
  int seq, q0;
  if (!prefill_tile(seq_start, n_seqs, skip_below, seq, q0)) return;
  const int tid = threadIdx.x, lane = tid % SYN_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / SYN_WAVE);
  const int n32 = lane % 32, hh = lane / 32;
  const int hx = blockIdx.x;
  const int head = nh % 8 == 0 ? (hx % 8) * (nh / 8) + hx / 8 : hx, kvh = head / (nh / nkv);
  const int tok0 = seq_start[seq], n_new = seq_start[seq + 1] - tok0, past = seq_past[seq];
  const int kv_len = past + n_new;
  const int r0 = q0 + wave * 32;
  const bool wave_on = r0 < n_new;
  const int row = r0 + n32;
  const bool valid = row < n_new;
  const int qpos = valid ? past + row : -1;
  const int lo = (window > 0 && valid) ? max(0, qpos - window + 1) : 0;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 qf[PF2_KS];
#pragma unroll
  for (int ks = 0; ks < PF2_KS; ++ks)
    qf[ks] = valid ? *(const bf16x8*)(q + ((size_t)(tok0 + row) * nh + head) * HD + 16 * ks + 8 * hh) : zero8;
  // visible keys of this wave, and of the whole workgroup
  const int w_kmax = past + min(r0 + 31, n_new - 1);
  const int w_qmin = past + r0;
  const int w_kmin = window > 0 ? max(0, w_qmin - window + 1) : 0;
  const int g_kmax = past + min(q0 + PF_ROWS - 1, n_new - 1);
  const int g_kmin = window > 0 ? max(0, past + q0 - window + 1) : 0;
  const int kb_lo = g_kmin / SYN_PAGE, kb_hi = g_kmax / SYN_PAGE;
  const float scale2 = scale * 1.44269504088896340736f;   // > 0: the host sends other scales to the other kernel

  f32x16 o[PF2_DT];
#pragma unroll
  for (int d = 0; d < PF2_DT; ++d)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[d][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // Load j of a wave for a block: its share of K (even j) or of V (odd j), 1 KB straight into LDS.
  constexpr int NLOAD = 2 * (PF2_KBYTES / 1024 / PF2_WAVES);
  auto views_of = [&](int kb, BufferView& vk, BufferView& vv) {
    const size_t base =
        ((size_t)__builtin_amdgcn_readfirstlane(page_table[(size_t)seq * table_stride + kb]) * nkv + kvh) * SYN_PAGE * HD;
    vk = buffer_view(k_pages + base, PF2_KBYTES), vv = buffer_view(v_pages + base, PF2_KBYTES);
  };
  auto fetch_one = [&](const BufferView& vk, const BufferView& vv, int buf, int j) {
    char* dst = lds2 + buf * PF2_BUF;
    const int i = (j / 2) * PF2_WAVES + wave;              // which 1 KB of the block this load fills
    const int at = 64 * i + lane, krow = at / PF2_CPR, slot = at % PF2_CPR;
    if (j % 2 == 0) buffer_to_lds16(vk, dst + 1024 * i, (unsigned)((krow * PF2_CPR + (slot ^ pf2_swizzle(krow))) * 16), 0);
    else buffer_to_lds16(vv, dst + PF2_KBYTES + 1024 * i, (unsigned)(at * 16), 0);
  };
  auto landed = [&]() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's loads have written LDS; behind the barrier all have
    __syncthreads();
  };

  // One block of keys.  MORE: a next block exists, and its loads are issued here, one behind every second MFMA of
  // the scores: issued in a burst at the block's top, the loads of four waves queue at the texture addresser
  // (about 16 cycles for each KB) and every wave stands until its own are taken (measured: a sixth of a wave's time).
  auto block = [&](int kb, auto more) {
    constexpr bool MORE = decltype(more)::value;
    const int buf = (kb - kb_lo) & 1;                    // the other buffer was last read before the previous barrier
    BufferView nk, nv;
    if constexpr (MORE) views_of(kb + 1, nk, nv);
    const int key0 = kb * SYN_PAGE;
    char* ks_ = lds2 + buf * PF2_BUF;
    char* vs_ = ks_ + PF2_KBYTES;
    if (key0 + SYN_PAGE > kv_len) {
      // the sequence ends inside this block: whatever lies behind its end in the page is made zero, so
      // that 0 * (that) is 0.  Chunk c holds tokens 32 h + 8 g .. + 7 of one dim, c = (h * DT + dt) * 64 + 16 g + r.
      for (int c = tid; c < 8 * HD; c += PF2_THREADS) {
        const int tok = 32 * (c / (64 * DT)) + 8 * ((c % 64) / 16);
        if (key0 + tok + 8 > kv_len) {
          bf16x8 v = *(bf16x8*)(vs_ + c * 16);
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (key0 + tok + e >= kv_len) v[e] = (bf16)0.f;
          *(bf16x8*)(vs_ + c * 16) = v;
        }
      }
      __syncthreads();
    }
    if (wave_on && key0 <= w_kmax && key0 + SYN_PAGE > w_kmin) {
      // Fragment reads from LDS take longer than an MFMA: PF2_AHEAD of them are on their way before the
      // first product needs one, then one read follows each MFMA.  The first V fragments are requested
      // before the softmax, so that they arrive while its maxima are taken.
      constexpr int NQK = 2 * PF2_KS, NPV = 4 * PF2_DT;
      constexpr int AHEAD = NQK < PF2_AHEAD ? NQK : PF2_AHEAD, VAHEAD = NPV < PF2_AHEAD ? NPV : PF2_AHEAD;
      static_assert(!PF2_OK || NLOAD <= NQK / 2, "a load behind every second MFMA of the scores");
      f32x16 s[2];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) s[t][e] = 0.f;
      const int krow0 = pf2_row_key(n32), sw0 = pf2_swizzle(krow0), sw1 = pf2_swizzle(32 + krow0);
      auto k_frag = [&](int i) {   // read i: k-step i / 2 of score tile i % 2
        const int t = i % 2, ks = i / 2;
        return *(const bf16x8*)(ks_ + ((32 * t + krow0) * PF2_CPR + ((2 * ks + hh) ^ (t ? sw1 : sw0))) * 16);
      };
      auto v_frag = [&](int i) {   // read i: output tile i % PF2_DT of k-step i / PF2_DT = 2 t + j
        const int d = i % PF2_DT, tj = i / PF2_DT, t = tj / 2, j = tj % 2;
        return *(const bf16x8*)(vs_ + (((t * DT + 2 * d + n32 / 16) * 64 + (2 * j + hh) * 16 + n32 % 16)) * 16);
      };
      bf16x8 kf[NQK], vf[NPV];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < AHEAD; ++i) kf[i] = k_frag(i);
#pragma unroll
      for (int i = 0; i < NQK; ++i) {
        s[i % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i], qf[i / 2], s[i % 2], 0, 0, 0);
        if (i + AHEAD < NQK) kf[i + AHEAD] = k_frag(i + AHEAD);
        else if (i + AHEAD - NQK < VAHEAD) vf[i + AHEAD - NQK] = v_frag(i + AHEAD - NQK);
        if (MORE && i % 2 == 1 && i / 2 < NLOAD) fetch_one(nk, nv, buf ^ 1, i / 2);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
      for (int i = 0; i < NQK; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA,
        if (i + AHEAD < NQK || i + AHEAD - NQK < VAHEAD) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one read behind it,
        if (MORE && i % 2 == 1 && i / 2 < NLOAD) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);           // a load behind every second
      }
      __builtin_amdgcn_sched_barrier(0);
      // a block needs masking if some row of the wave does not see all of it
      const bool need_mask = key0 + SYN_PAGE - 1 > w_qmin || (window > 0 && key0 < w_kmax - window + 1) || r0 + 32 > n_new;
      if (need_mask) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int key = key0 + 32 * t + 16 * (e / 8) + 8 * hh + e % 8;
            if (key > qpos || key < lo) s[t][e] = -INFINITY;
          }
      }
      float mloc = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) mloc = fmaxf(mloc, s[t][e]);
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32, SYN_WAVE)) * scale2;
      // m_run is the reference of the exponents, not the exact maximum: it is only raised when a block
      // exceeds it by more than RESCALE_AT (in log2 units), so that the accumulators are rescaled in few blocks
      const bool raise = mloc > m_run + RESCALE_AT || (m_run == -INFINITY && mloc > -INFINITY);
      if (__any(raise)) {
        const float m_new = raise ? mloc : m_run;
        const float alpha = raise ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.f;  // from -inf: 0
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int d = 0; d < PF2_DT; ++d) o[d] *= alpha;
      }
      const float neg_m = m_run == -INFINITY ? 0.f : -m_run;  // a column that has seen no key yet
      float lsum = 0.f;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) {
        bf16x8 pb;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float p = __builtin_amdgcn_exp2f(fmaf(s[tj / 2][8 * (tj % 2) + e], scale2, neg_m));   // a masked score: 2^-inf = 0
          lsum += p;
          pb[e] = (bf16)p;
        }
#pragma unroll
        for (int d = 0; d < PF2_DT; ++d) {
          const int i = tj * PF2_DT + d;
          o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i], pb, o[d], 0, 0, 0);
          if (i + VAHEAD < NPV) vf[i + VAHEAD] = v_frag(i + VAHEAD);
        }
      }
      l_run += lsum;
    } else if constexpr (MORE) {
#pragma unroll
      for (int j = 0; j < NLOAD; ++j) fetch_one(nk, nv, buf ^ 1, j);
    }
    landed();
  };

  {
    BufferView vk, vv;
    views_of(kb_lo, vk, vv);
#pragma unroll
    for (int j = 0; j < NLOAD; ++j) fetch_one(vk, vv, 0, j);
  }
  landed();
  for (int kb = kb_lo; kb < kb_hi; ++kb) block(kb, std::true_type{});
  block(kb_hi, std::false_type{});
  if (!wave_on) return;
  float l = l_run + __shfl_xor(l_run, 32, SYN_WAVE);
  if (!valid) return;
  const float inv = 1.f / l;
  bf16* orow = out + ((size_t)(tok0 + row) * nh + head) * HD + 4 * hh;
#pragma unroll
  for (int d = 0; d < PF2_DT; ++d)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (bf16)(o[d][4 * b + e] * inv);
      *(bf16x4*)(orow + 32 * d + 8 * b) = v;
    }
}

SYN_EXPORT int syn_attention_prefill_bf16(const void* q, const void* k_pages, const void* v_pages,
                                          const int* page_table, int table_stride, const int* seq_start,
                                          const int* seq_past, int n_seqs, int n_tokens, void* out, float scale,
                                          int window, int nh, int nkv, int hd, int variant, const float* slopes,
                                          float softcap, int skip_below, hipStream_t stream) {
  // variant: 0 = whichever is faster for this head size, 1 = waves of 16 query rows (every head size),
  // 2 = waves of 32 query rows (head sizes 64 and 128, a positive scale, no terms on the scores)
  // slopes [nh] float or null, softcap (0: none): see ScoreTerms; the kernel with waves of 16 rows applies them
  // skip_below: sequences that bring fewer new tokens than this are left out (2: those with a single token, which
  // the caller hands to the decode kernel); 0 or 1: none
  SYN_CHECK(variant >= 0 && variant <= 2, "attention_prefill: unknown variant %d", variant);
  SYN_CHECK(softcap >= 0.f, "attention_prefill: a soft cap of %g", (double)softcap);
  const ScoreTerms terms = {slopes, softcap};
  const bool with_terms = slopes != nullptr || softcap > 0.f;
  SYN_CHECK(variant != 2 || (PF2_OK && scale > 0.f && !with_terms), "attention_prefill: waves of 32 rows take head sizes 64 "
            "and 128, a positive scale and no terms on the scores (head size %d, scale %g)", HD, (double)scale);
  SYN_CHECK(hd == HD, "attention_prefill: library built for head size %d, called with %d", HD, hd);
  SYN_CHECK(n_seqs > 0 && n_tokens >= n_seqs && nh > 0 && nkv > 0, "attention_prefill: empty input");
  SYN_CHECK(nh % nkv == 0, "attention_prefill: %d heads do not divide into %d kv heads", nh, nkv);
  const int tiles = n_tokens / PF_ROWS + n_seqs;  // an upper bound; surplus workgroups leave at once
  SYN_CHECK(tiles <= 65535, "attention_prefill: %d tiles of %d rows exceed the grid", tiles, PF_ROWS);
  const size_t lds = (size_t)2 * PF_TILE * sizeof(bf16);
  static OncePerDevice raised;
  if (lds > 65536) {
    const hipError_t e = once_per_device(raised, [&] {
      return hipFuncSetAttribute((const void*)attn_prefill_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    });
    SYN_CHECK(e == hipSuccess, "attention_prefill: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
  }
  if constexpr (PF2_OK) {
    if (variant == 2 || (variant == 0 && scale > 0.f && !with_terms)) {
      attn_prefill32_kernel<<<dim3(nh, tiles), PF2_THREADS, 2 * PF2_BUF, stream>>>(
          (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_start, seq_past,
          n_seqs, (bf16*)out, scale, window, nh, nkv, skip_below);
      SYN_LAUNCH_CHECK("attention_prefill32");
      return 0;
    }
  }
  attn_prefill_kernel<<<dim3(nh, tiles), PF_THREADS, lds, stream>>>(
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_start, seq_past, n_seqs,
      (bf16*)out, scale, window, nh, nkv, terms, skip_below);
  SYN_LAUNCH_CHECK("attention_prefill");
  return 0;
}

// ------------------------------------------------------------------ decode: split over keys, then merge
// A workgroup of up to 8 waves takes (sequence, kv head, up to 16 heads of its group, one split of
// the keys, in units of half a block); its waves take the split's units in turn and their states are
// combined in LDS.
// With one split the workgroup writes the output itself; else it writes a partial
//   partial[((first + split) * nh + head)] = { m, l, o[HD] }   (float; first: where the sequence's splits begin)
// and the splits are merged, in their order: by the workgroup of the sequence that finishes last
// (DecodeWork::counters given), or by a second kernel.
constexpr int PART = HD + 2;

// How the keys of a step's sequences are handed to workgroups.  Without `items` every sequence is cut
// into the same n_splits (grid.x sequences, grid.z splits).  With `items` the grid's x counts items
// {sequence, split | splits of the sequence << 16, first, the sequence's length} that the host has laid out,
// more splits for longer sequences, the longest pieces first; an item with sequence -1 is spare and its
// workgroups leave at once.
// counters: one int for each (sequence, grid.y), zero before the launch and zero again after it.
struct DecodeWork {
  float* partial;
  int* counters;
  const int4* items;
};

// A value that another workgroup, possibly on another XCD with a second-level cache of its own, reads
// within the same launch: stored through to memory, and read from there.
__device__ __forceinline__ void store_through(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_through(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr int DEC_MAX_WAVES = HD > 128 ? 4 : 8;  // as many as keep their registers (144 at a head size of 128, about twice that at 256) without spilling

// The unit of a wave's work is half a block: 32 keys, whose K rows and whose V fragments are each one
// contiguous piece of the page (64 * HD bytes).  Whole blocks leave the last round of a workgroup mostly
// idle where a split holds few of them (33 blocks over 4 splits and 8 waves: two rounds, the second for
// one wave).  These are the K and V fragments of one unit, all requested before the first product needs one.
constexpr int UNIT_KEYS = 32;
struct KvUnit {
  kfrag_t ka[2][KSTEPS];
  bf16x8 va[DT];
};

// kpage: the unit's first K row
__device__ __forceinline__ void load_k_decode(KvUnit& b, const bf16* __restrict__ kpage, int lane) {
  const int r16 = lane % 16;
#pragma unroll
  for (int t = 0; t < 2; ++t) load_row(b.ka[t], kpage + (size_t)tile_row_key(t, r16) * HD, lane);
}

// a fragment of V is 1 KB of the page, in lane order.  A decode step reads every key and value once: its
// loads are marked non-temporal (551 MB of cache for 64 sequences: 98.8 -> 88.5 us a layer; never slower
// from 1 to 64 sequences and 500 to 32,000 tokens).  vpage: the unit's first fragment
__device__ __forceinline__ void load_v_decode(KvUnit& b, const bf16* __restrict__ vpage, int lane) {
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    b.va[dt] = __builtin_nontemporal_load((const bf16x8*)(vpage + (size_t)(dt * 64 + lane) * 8));
}

// Head sizes that are a power of two from 32 on: a unit's K rows (32 x HD) are one contiguous piece of
// 64 * HD bytes, and a wave brings them into a piece of LDS of its own with loads of 1 KB that write
// LDS directly, then reads its fragments from there.  Loading K fragments straight from memory asks
// the first-level cache for 16 rows x 64 bytes with every instruction, which was measured to keep
// the texture addresser busy about 100 cycles an instruction and to bound the kernel at large
// batches.  (V needs no such detour: its pages are kept in fragment order.)
// In LDS the 16-byte chunk c of row r lies at slot c ^ f(r) of the row, with f chosen so that the 16
// rows a fragment read touches fall into different banks; the permutation is applied to the address
// that a lane fetches (the slot it fills is fixed by its number) and again by the reader.
constexpr bool STAGED = !TAIL16 && (HD & (HD - 1)) == 0;
constexpr int STAGE_BYTES = STAGED ? 64 * HD : 0;   // the K rows of one unit
constexpr int K_CPR = HD / 8;                       // 16-byte chunks in a K row
// the rows of a score tile differ in bits 0, 1, 3 and 4 of the key number: those four bits, less as
// many low ones as rows fit into the 256 bytes that the banks span
__device__ __forceinline__ int k_swizzle(int row) {
  constexpr int DROP = HD >= 128 ? 0 : (HD == 64 ? 1 : 2);
  return ((row & 3) | (((row >> 3) & 3) << 2)) >> DROP;
}

__device__ __forceinline__ void stage_k(const bf16* __restrict__ kpage, char* stage, int lane) {
  const BufferView view = buffer_view(kpage, STAGE_BYTES);
#pragma unroll
  for (int i = 0; i < HD / 16; ++i) {
    const int at = 64 * i + lane, row = at / K_CPR, slot = at % K_CPR;
    buffer_to_lds16<true>(view, stage + 1024 * i, (unsigned)((row * K_CPR + (slot ^ k_swizzle(row))) * 16), 0);
  }
}
// The staged K has landed: of this wave's loads at most the V fragments requested after it (DT loads)
// are still on their way.  Nothing that reads the piece may move above this.
__device__ __forceinline__ void staged_landed() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DT) : "memory"); }
// this wave's reads of the staged piece have returned: the piece may be filled again
__device__ __forceinline__ void staged_read() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

__device__ __forceinline__ void read_k_staged(KvUnit& b, const char* stage, int lane) {
  if constexpr (STAGED) {
    const int r16 = lane % 16, g4 = lane / 16;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int row = tile_row_key(t, r16), sw = k_swizzle(row);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) b.ka[t][ks] = *(const kfrag_t*)(stage + (row * K_CPR + ((ks * 4 + g4) ^ sw)) * 16);
    }
  }
}
// One unit of 32 keys in two parts, so that the loads of the next unit can follow each part at once:
// the scores and their softmax weights (reads the K fragments), then the weighted values (reads the V fragments).
__device__ __forceinline__ void decode_scores(const QFrag& qf, const KvUnit& unit, f32x4 (&s)[2]) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    s[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) s[t] = mfma_qk(unit.ka[t][ks], qf.k[ks], s[t]);
  }
}

// key0: the unit's first key
// qpos: the last key position that this column may see (-1: none); pos: the query's own position; slope, cap: the
// terms on the scores of this lane's head (with_terms false: none)
__device__ __forceinline__ void decode_weights(AttnState<1>& st, f32x4 (&s)[2], int key0, int qpos, int lo, float scale,
                                               int lane, bool with_terms, float slope, float cap, int pos) {
  const int g4 = lane / 16;
  float mloc = -INFINITY;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int key = key0 + acc_key(t, g4, e);
      float v = s[t][e] * scale;
      if (with_terms) v = score_with_terms(v, slope, cap, pos, key);
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
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float p = __expf(s[t][e] - m_use);
      s[t][e] = p;
      lsum += p;
    }
  st.l[0] = st.l[0] * alpha + lsum;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) st.o[dt][0] *= alpha;
}

__device__ __forceinline__ void decode_values(AttnState<1>& st, const KvUnit& unit, const f32x4 (&s)[2], int key0,
                                              int kv_len, int lane) {
  const int g4 = lane / 16;
  const bool ragged = key0 + UNIT_KEYS > kv_len;
  bf16x8 pb;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    pb[e] = (bf16)s[0][e];
    pb[4 + e] = (bf16)s[1][e];
  }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    bf16x8 av = unit.va[dt];
    if (ragged) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (key0 + 8 * g4 + e >= kv_len) av[e] = (bf16)0.f;  // 0 * (whatever lies there) must be 0
    }
    st.o[dt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pb, st.o[dt][0], 0, 0, 0);
  }
}

// What the kernel needs to take q, k and v of the new tokens from the fused projection itself
// instead of from a kernel before it: rows [q heads | k heads | v heads] of one token a sequence, as
// bf16 (n_parts == 0) or as n_parts float partial sums of a product cut along K.
struct QkvIntake {
  const void* qkv;
  int n_parts;
  size_t part_stride;
  const void* q_gain;  // RMSNorm gains of the q and k heads, or nullptr
  const void* k_gain;
  int gain_is_f32;
  float gain_offset;   // the gain is gain_offset + w[i]
  float eps;
  const float* cos_t;  // rotation tables [positions][rot / 2], or nullptr
  const float* sin_t;
  int rot;
  int own_kv;  // the layer writes its k and v into the cache (else it reads a cache that another layer wrote)
};

// FUSED: the workgroup first makes its q heads from the projection (sum of the partial sums,
// RMSNorm, rotation: all in 32-bit, rounded once to bf16 into LDS).  With own_kv the workgroup of
// split 0 makes the new k and v of its kv head likewise, writes them into the cache for later steps,
// and adds the new key to its result as one more partial state; the loop over the cache then covers
// the older keys only, so nothing is read that this launch writes.
template <bool FUSED>
__global__ void __launch_bounds__(DEC_MAX_WAVES * SYN_WAVE)
attn_decode_split_kernel(const bf16* __restrict__ q, bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                         const int* __restrict__ page_table, int table_stride, const int* __restrict__ seq_len,
                         DecodeWork work, bf16* __restrict__ out, float scale, int window, int nh, int nkv,
                         int n_splits_all, int cols_alloc, QkvIntake in, ScoreTerms terms) {
  // LDS: with STAGED first a piece of STAGE_BYTES for each wave; then
  //      sm[waves][16] running maxima, sl[waves][16] sums, so[waves][cols_alloc][HD + 4] outputs;
  // FUSED: then xs[waves][HD] floats, snew[16] scores of the new key, qs[cols_alloc][HD], knew[HD], vnew[HD] bf16
  extern __shared__ __attribute__((aligned(16))) float dec_lds[];
  const int n_waves = blockDim.x / SYN_WAVE;
  float* sm = dec_lds + (size_t)n_waves * (STAGE_BYTES / 4);   // the waves' staging pieces lie first
  float* sl = sm + n_waves * 16;
  float* so = sl + n_waves * 16;
  constexpr int SO_LD = HD + 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / SYN_WAVE), lane = threadIdx.x % SYN_WAVE;
  char* stage = (char*)dec_lds + (size_t)wave * STAGE_BYTES;
  // Without a work list the grid is (sequences, kv heads x chunks, splits); with one it is (kv heads x chunks, items),
  // the kv heads of an item next to each other (they lie side by side in a page).
  int seq = blockIdx.x, split = blockIdx.z, n_splits = n_splits_all, first = blockIdx.x * n_splits_all, item_len = -1;
  int group_of_heads = blockIdx.y, n_groups_of_heads = gridDim.y;
  if (work.items) {
    const int4 item = work.items[blockIdx.y];
    group_of_heads = blockIdx.x, n_groups_of_heads = gridDim.x;
    seq = __builtin_amdgcn_readfirstlane(item.x), first = __builtin_amdgcn_readfirstlane(item.z);
    split = __builtin_amdgcn_readfirstlane(item.y) & 0xFFFF, n_splits = __builtin_amdgcn_readfirstlane(item.y) >> 16;
    item_len = __builtin_amdgcn_readfirstlane(item.w);   // (with the item: one trip to memory less than through seq_len)
    // (a spare item, or one that does not fit the launch: nothing is read or written for it)
    const int n_seqs = gridDim.y / n_splits_all;
    if (seq < 0 || seq >= n_seqs || n_splits < 1 || split >= n_splits || first < 0 || first + n_splits > (int)gridDim.y ||
        item_len < 1)
      return;
  }
  float* const partial = work.partial;
  const int g = nh / nkv, chunks = (g + 15) / 16;
  const int kvh = group_of_heads / chunks, chunk = group_of_heads % chunks;
  const int kv_len = item_len > 0 ? item_len : seq_len[seq], pos = kv_len - 1;
  const int col = lane % 16;
  const int hg = chunk * 16 + col;  // head inside the group
  const bool valid = hg < g;
  const int n_cols = min(16, g - chunk * 16);
  const bool new_key = FUSED && in.own_kv;            // the newest key is not read from the cache
  const bool adds_new = new_key && split == 0;        // this workgroup makes it and adds it
  const bool with_terms = score_terms_on(terms);
  const float slope = (terms.slopes && valid) ? terms.slopes[kvh * g + hg] : 0.f;

  // keys read from the cache: all of them, or all but the newest; the units of this split; the first
  // unit of this wave is requested at once, before the workgroup prepares its q heads
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int n_old = new_key ? kv_len - 1 : kv_len;
  const int q_lim = new_key ? pos - 1 : pos;  // the last key position that the loop may see
  const int u_lo = lo / UNIT_KEYS, u_hi = n_old > 0 ? (n_old - 1) / UNIT_KEYS : u_lo - 1;
  const int per = (u_hi - u_lo + n_splits) / n_splits;  // ceil((u_hi - u_lo + 1) / n_splits)
  const int u0 = u_lo + split * per, u1 = min(u_hi + 1, u0 + per);
  constexpr int UNITS = SYN_PAGE / UNIT_KEYS;   // units in a page
  auto unit_at = [&](int u) {   // where the unit's K rows and V fragments begin in the page arrays; the same for all lanes
    const int page = __builtin_amdgcn_readfirstlane(page_table[(size_t)seq * table_stride + u / UNITS]);
    return ((size_t)page * nkv + kvh) * SYN_PAGE * HD + (size_t)(u % UNITS) * UNIT_KEYS * HD;
  };
  KvUnit unit;
  if (u0 + wave < u1) {
    const size_t base = unit_at(u0 + wave);
    if constexpr (STAGED) stage_k(k_pages + base, stage, lane);
    else load_k_decode(unit, k_pages + base, lane);
    load_v_decode(unit, v_pages + base, lane);
  }

  float* xs = so + (size_t)n_waves * cols_alloc * SO_LD;
  float* snew = xs + n_waves * HD;
  bf16* qs = (bf16*)(snew + 16);
  bf16* knew = qs + cols_alloc * HD;
  bf16* vnew = knew + HD;
  if constexpr (FUSED) {
    const int heads = nh + 2 * nkv, half = in.rot / 2;
    const int n_items = n_cols + (adds_new ? 2 : 0);  // q heads of this chunk, then k and v of the kv head
    for (int it0 = 0; it0 < n_items; it0 += n_waves) {  // the same number of rounds for every wave: barriers inside
      const int it = it0 + wave;
      const bool active = it < n_items;
      const int kind = it < n_cols ? 0 : (it == n_cols ? 1 : 2);
      const int head = kind == 0 ? kvh * g + chunk * 16 + it : (kind == 1 ? nh + kvh : nh + nkv + kvh);
      float* x = xs + wave * HD;
      // the angles of this lane's dims are requested now, together with the values, not after the barrier
      constexpr int PER = (HD + 2 * SYN_WAVE - 1) / (2 * SYN_WAVE);
      float cs[PER][2], sn[PER][2];
      const bool rotate = active && kind != 2 && in.cos_t != nullptr;
      if (rotate) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int d = 2 * lane + i * 2 * SYN_WAVE;
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            const bool in_rot = d + e < in.rot && d + e < HD;
            const int idx = d + e < half ? d + e : d + e - half;
            cs[i][e] = in_rot ? in.cos_t[(size_t)pos * half + idx] : 1.f;
            sn[i][e] = in_rot ? in.sin_t[(size_t)pos * half + idx] : 0.f;
          }
        }
      }
      if (active) {
        const size_t at = ((size_t)seq * heads + head) * HD;
        float ss = 0.f;
        for (int d = 2 * lane; d < HD; d += 2 * SYN_WAVE) {
          float v0, v1;
          if (in.n_parts > 0) {
            const float* src = (const float*)in.qkv + at + d;
            v0 = 0.f, v1 = 0.f;
            for (int p0 = 0; p0 < in.n_parts; p0 += 8) {  // eight partial sums in flight together, added in order
              float2 t[8];
#pragma unroll
              for (int u = 0; u < 8; ++u)
                t[u] = p0 + u < in.n_parts ? *(const float2*)(src + (size_t)(p0 + u) * in.part_stride) : make_float2(0.f, 0.f);
#pragma unroll
              for (int u = 0; u < 8; ++u) v0 += t[u].x, v1 += t[u].y;
            }
          } else {
            const bf16* src = (const bf16*)in.qkv + at;
            v0 = (float)src[d], v1 = (float)src[d + 1];
          }
          x[d] = v0, x[d + 1] = v1;
          ss += v0 * v0 + v1 * v1;
        }
        const void* gain = kind == 0 ? in.q_gain : (kind == 1 ? in.k_gain : nullptr);
        if (gain) {
          ss = wave_sum(ss);
          const float inv = rsqrtf(ss / (float)HD + in.eps);
          for (int d = 2 * lane; d < HD; d += 2 * SYN_WAVE) {
            x[d] = load_gain(gain, in.gain_is_f32, d, in.gain_offset) * x[d] * inv;
            x[d + 1] = load_gain(gain, in.gain_is_f32, d + 1, in.gain_offset) * x[d + 1] * inv;
          }
        }
      }
      __syncthreads();  // lanes read what other lanes of their wave wrote
      if (active) {
        auto rotated = [&](int d, float c, float sine) {
          float o = x[d];
          if (rotate && d < in.rot) o = d < half ? x[d] * c - x[d + half] * sine : x[d] * c + x[d - half] * sine;
          return (bf16)o;
        };
        bf16* dst = kind == 0 ? qs + it * HD : (kind == 1 ? knew : vnew);
        const size_t page_base = ((size_t)page_table[(size_t)seq * table_stride + pos / SYN_PAGE] * nkv + kvh) * SYN_PAGE * HD;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int d = 2 * lane + i * 2 * SYN_WAVE;
          if (d >= HD) break;
          const bf16 o0 = rotated(d, cs[i][0], sn[i][0]), o1 = rotated(d + 1, cs[i][1], sn[i][1]);
          dst[d] = o0, dst[d + 1] = o1;
          if (kind == 1) {
            bf16* row = k_pages + page_base + (size_t)(pos % SYN_PAGE) * HD;
            row[d] = o0, row[d + 1] = o1;
          } else if (kind == 2) {
            bf16* vpage = v_pages + page_base;
            vpage[v_page_offset(HD, d, pos % SYN_PAGE)] = o0, vpage[v_page_offset(HD, d + 1, pos % SYN_PAGE)] = o1;
          }
        }
      }
      __syncthreads();  // xs is written again in the next round; qs, knew, vnew are read below
    }
    if (adds_new) {
      // the new key's score for every head of the chunk, from the rounded q and k as the products see them
      for (int c = wave; c < n_cols; c += n_waves) {
        float dot = 0.f;
        for (int d = lane; d < HD; d += SYN_WAVE) dot += (float)qs[c * HD + d] * (float)knew[d];
        dot = wave_sum(dot);
        // (the new key lies at the query's own position: a soft cap applies, a penalty in the distance is zero)
        if (lane == 0) snew[c] = with_terms ? score_with_terms(dot * scale, 0.f, terms.softcap, pos, pos) : dot * scale;
      }
    }
  }

  QFrag qf;
  if constexpr (FUSED)
    load_q(qf, valid ? qs + col * HD : nullptr, lane);
  else
    load_q(qf, valid ? q + ((size_t)seq * nh + kvh * g + hg) * HD : nullptr, lane);
  AttnState<1> st;
  attn_init(st);
  // K of the next unit is requested as soon as the K fragments of this one are in registers (or have
  // been used), V of the next unit as soon as the V fragments have been used: K is on its way during
  // the products of this unit, V during the scores of the next, without a second set of registers
  for (int u = u0 + wave; u < u1; u += n_waves) {
    const int next = u + n_waves;
    const size_t next_base = next < u1 ? unit_at(next) : 0;
    const int key0 = u * UNIT_KEYS;
    f32x4 s[2];
    if constexpr (STAGED) {
      staged_landed();
      read_k_staged(unit, stage, lane);
      staged_read();
      if (next < u1) stage_k(k_pages + next_base, stage, lane);
      decode_scores(qf, unit, s);
    } else {
      decode_scores(qf, unit, s);
      if (next < u1) load_k_decode(unit, k_pages + next_base, lane);
    }
    decode_weights(st, s, key0, valid ? q_lim : -1, lo, scale, lane, with_terms, slope, terms.softcap, pos);
    decode_values(st, unit, s, key0, n_old, lane);
    if (next < u1) load_v_decode(unit, v_pages + next_base, lane);
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
    float m = adds_new ? snew[c] : -INFINITY;
    for (int w = 0; w < n_waves; ++w) m = fmaxf(m, sm[w * 16 + c]);
    float acc = 0.f, lsum = 0.f;
    for (int w = 0; w < n_waves; ++w) {
      const float mw = sm[w * 16 + c];
      if (mw == -INFINITY) continue;  // a wave that had no unit
      const float f = __expf(mw - m);
      acc += f * so[((size_t)w * cols_alloc + c) * SO_LD + d];
      lsum += f * sl[w * 16 + c];
    }
    if (adds_new) {  // the new key: weight exp(score - m), value vnew
      const float f = __expf(snew[c] - m);
      acc += f * (float)vnew[d];
      lsum += f;
    }
    const int head = kvh * g + chunk * 16 + c;
    if (n_splits == 1) {
      out[((size_t)seq * nh + head) * HD + d] = (bf16)(acc / lsum);
    } else {
      float* p = partial + (((size_t)first + split) * nh + head) * PART;
      store_through(p + 2 + d, acc);
      if (d == 0) {
        store_through(p, m);
        store_through(p + 1, lsum);
      }
    }
  }
  if (n_splits == 1 || work.counters == nullptr) return;

  // The workgroup of this (sequence, kv head, chunk) that finishes last merges the splits, in their
  // order whatever the order of arrival.  Every wave's stores have been acknowledged by memory before
  // its workgroup counts itself in; the one that counts last finds all of them there.
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  __syncthreads();
  int* const is_last = (int*)sm;        // (the loop above has finished reading sm)
  if (threadIdx.x == 0) {
    int* cnt = work.counters + (size_t)seq * n_groups_of_heads + group_of_heads;
    const int before = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = before == n_splits - 1;
    if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
    *is_last = last;
  }
  __syncthreads();
  if (!*is_last) return;
  for (int idx = threadIdx.x; idx < n_cols * HD; idx += blockDim.x) {
    const int c = idx / HD, d = idx % HD;
    const int head = kvh * g + chunk * 16 + c;
    const float* p = partial + ((size_t)first * nh + head) * PART;
    const size_t step = (size_t)nh * PART;   // from one split of the head to the next
    // all of up to 16 splits' values are asked for together (one trip to memory); further splits join a running
    // state, in their order
    constexpr int BATCH = 16;
    float m = -INFINITY, acc = 0.f, lsum = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += BATCH) {
      float ms[BATCH], ls[BATCH], vs[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const bool on = s0 + u < n_splits;
        const float* ps = p + (size_t)min(s0 + u, n_splits - 1) * step;
        ms[u] = load_through(ps);
        ls[u] = load_through(ps + 1);
        vs[u] = load_through(ps + 2 + d);
        if (!on) ms[u] = -INFINITY;
      }
      float m_new = m;
#pragma unroll
      for (int u = 0; u < BATCH; ++u) m_new = fmaxf(m_new, ms[u]);
      if (m_new == -INFINITY) continue;        // (no split of this batch had keys)
      const float keep = m == -INFINITY ? 0.f : __expf(m - m_new);
      acc *= keep, lsum *= keep;
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        if (ms[u] == -INFINITY) continue;       // a split that had no keys weighs nothing and may hold anything
        const float f = __expf(ms[u] - m_new);
        acc += f * vs[u];
        lsum += f * ls[u];
      }
      m = m_new;
    }
    out[((size_t)seq * nh + head) * HD + d] = (bf16)(acc / lsum);
  }
}

// one wave a (sequence, head): lanes first share the splits' maxima and sums, then each takes output dims
__global__ void __launch_bounds__(SYN_WAVE)
// of_seq: with a work list, {first, splits} of each sequence (the table behind the list's items); else every
// sequence has n_splits_all splits, the first at sequence * n_splits_all
attn_decode_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out, int n_splits_all, int nh,
                         const int2* __restrict__ of_seq) {
  const int row = blockIdx.x, lane = threadIdx.x;  // row = seq * nh + head
  const int seq = row / nh, head = row % nh;
  const size_t STEP = (size_t)nh * PART;           // from one split of the head to the next
  int first = seq * n_splits_all, n_splits = n_splits_all;
  if (of_seq) {
    first = __builtin_amdgcn_readfirstlane(of_seq[seq].x), n_splits = __builtin_amdgcn_readfirstlane(of_seq[seq].y);
    const int n_seqs = gridDim.x / nh;
    // (one split has written the output itself; a table that does not fit the launch is not followed)
    if (n_splits <= 1 || first < 0 || first + n_splits > n_seqs * n_splits_all) return;
  }
  const float* p = partial + ((size_t)first * nh + head) * PART;
  float wsum[(HD + SYN_WAVE - 1) / SYN_WAVE] = {};
  float l = 0.f;
  float m = -INFINITY;
  for (int s0 = 0; s0 < n_splits; s0 += SYN_WAVE) {  // maximum over all splits
    const int s = s0 + lane;
    m = fmaxf(m, s < n_splits ? p[(size_t)s * STEP] : -INFINITY);
  }
  m = wave_max(m);
  for (int s0 = 0; s0 < n_splits; s0 += SYN_WAVE) {
    const int s = s0 + lane;
    const float ms = s < n_splits ? p[(size_t)s * STEP] : -INFINITY;
    const float w = ms == -INFINITY ? 0.f : __expf(ms - m);  // a split that had no keys weighs nothing
    l += s < n_splits ? w * p[(size_t)s * STEP + 1] : 0.f;
    const int cnt = min(SYN_WAVE, n_splits - s0);
    for (int j0 = 0; j0 < cnt; j0 += 8) {  // eight splits' values in flight together, added in their order
      constexpr int NI = (HD + SYN_WAVE - 1) / SYN_WAVE;
      float vals[8][NI];
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int d = lane + i * SYN_WAVE;
          vals[u][i] = (j0 + u < cnt && d < HD) ? p[(size_t)(s0 + j0 + u) * STEP + 2 + d] : 0.f;
        }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float wj = __shfl(w, min(j0 + u, SYN_WAVE - 1), SYN_WAVE);
        if (j0 + u < cnt && wj != 0.f) {  // the same for the whole wave; a split without keys may hold anything
#pragma unroll
          for (int i = 0; i < NI; ++i) wsum[i] += wj * vals[u][i];
        }
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

// the decode kernels may use all of a compute unit's LDS: asked for once on each device
constexpr size_t DEC_LDS_MAX = 160 * 1024;
static hipError_t raise_decode_lds() {
  static OncePerDevice once;
  return once_per_device(once, [] {
    hipError_t e = hipFuncSetAttribute((const void*)attn_decode_split_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)DEC_LDS_MAX);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)attn_decode_split_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)DEC_LDS_MAX);
    return e;
  });
}

// workspace: n_seqs * nh * n_splits * (HD + 2) floats (unused with one split).
// counters (may be null): n_seqs * kv heads * ceil(group / 16) ints, zero.  With them the splits are merged inside the
// one launch where the grid is at most two workgroups a compute unit; where it is larger, and without them, a second
// kernel merges (a workgroup that waits for its stores and counts itself in holds its place that much longer, which a
// grid of several rounds pays in every round: 8 sequences of 32,000 tokens 9.3 ms a step against 9.1).
// items (may be null: every sequence in n_splits splits): n_items x {sequence, split | splits of the sequence << 16,
// first, length}, `first` + split < n_seqs * n_splits being the place of the split's partial results and length
// what seq_len holds for the sequence; behind them n_seqs x {first, splits}, the same by sequence.
static int launch_decode(const void* q, const QkvIntake* in, void* k_pages, void* v_pages, const int* page_table,
                         int table_stride, const int* seq_len, int n_seqs, void* out, float* workspace, int n_splits,
                         float scale, int window, int nh, int nkv, int hd, hipStream_t stream,
                         ScoreTerms terms = ScoreTerms{nullptr, 0.f}, int* counters = nullptr,
                         const int* items = nullptr, int n_items = 0) {
  SYN_CHECK(terms.softcap >= 0.f, "attention_decode: a soft cap of %g", (double)terms.softcap);
  SYN_CHECK(hd == HD, "attention_decode: library built for head size %d, called with %d", HD, hd);
  SYN_CHECK(n_seqs > 0 && nh > 0 && nkv > 0 && n_splits > 0, "attention_decode: empty input");
  SYN_CHECK(nh % nkv == 0, "attention_decode: %d heads do not divide into %d kv heads", nh, nkv);
  const int chunks = (nh / nkv + 15) / 16;
  SYN_CHECK(nkv * chunks <= 65535 && n_splits <= 65535 && n_items <= 65535, "attention_decode: grid too large");
  SYN_CHECK(items == nullptr || n_items == n_seqs * n_splits,
            "attention_decode: a list of %d items for %d sequences x %d splits", n_items, n_seqs, n_splits);
  // waves a workgroup: as many as the LDS for their states allows (up to 8), but no more than make
  // about 2,048 waves in all: at large batches four waves a workgroup are plenty
  const int cols_alloc = nh / nkv < 16 ? nh / nkv : 16;
  auto lds_for = [&](int waves) {
    size_t b = (size_t)waves * STAGE_BYTES + (size_t)waves * (32 + (size_t)cols_alloc * (HD + 4)) * sizeof(float);
    if (in) b += ((size_t)waves * HD + 16) * sizeof(float) + (size_t)(cols_alloc + 2) * HD * sizeof(bf16);
    return b;
  };
  constexpr size_t LDS_MAX = DEC_LDS_MAX;
  int waves = DEC_MAX_WAVES;
  while (waves > 2 && (lds_for(waves) > LDS_MAX || (long)n_seqs * nkv * chunks * n_splits * waves > 2048)) waves /= 2;
  if (waves < 4 && lds_for(4) <= LDS_MAX) waves = 4;
  const size_t lds = lds_for(waves);
  SYN_CHECK(lds <= LDS_MAX, "attention_decode: %zu bytes of LDS for %d heads a group", lds, nh / nkv);
  const hipError_t raised = raise_decode_lds();
  SYN_CHECK(raised == hipSuccess, "attention_decode: %zu bytes of LDS refused: %s", LDS_MAX, hipGetErrorString(raised));
  const dim3 grid = items ? dim3(nkv * chunks, n_items, 1) : dim3(n_seqs, nkv * chunks, n_splits);
  const bool merge_inside = counters != nullptr && (long)n_seqs * nkv * chunks * n_splits <= 2L * syn_compute_units();
  const DecodeWork work{workspace, merge_inside ? counters : nullptr, (const int4*)items};
  if (in)
    attn_decode_split_kernel<true><<<grid, waves * SYN_WAVE, lds, stream>>>(
        nullptr, (bf16*)k_pages, (bf16*)v_pages, page_table, table_stride, seq_len, work, (bf16*)out, scale,
        window, nh, nkv, n_splits, cols_alloc, *in, terms);
  else
    attn_decode_split_kernel<false><<<grid, waves * SYN_WAVE, lds, stream>>>(
        (const bf16*)q, (bf16*)k_pages, (bf16*)v_pages, page_table, table_stride, seq_len, work, (bf16*)out,
        scale, window, nh, nkv, n_splits, cols_alloc, QkvIntake{}, terms);
  SYN_LAUNCH_CHECK("attention_decode_split");
  if (n_splits > 1 && !merge_inside) {
    attn_decode_merge_kernel<<<n_seqs * nh, SYN_WAVE, 0, stream>>>(workspace, (bf16*)out, n_splits, nh,
                                                                   items ? (const int2*)(items + 4L * n_items) : nullptr);
    SYN_LAUNCH_CHECK("attention_decode_merge");
  }
  return 0;
}

SYN_EXPORT int syn_attention_decode_bf16(const void* q, const void* k_pages, const void* v_pages,
                                         const int* page_table, int table_stride, const int* seq_len, int n_seqs,
                                         void* out, float* workspace, int n_splits, float scale, int window, int nh,
                                         int nkv, int hd, hipStream_t stream) {
  return launch_decode(q, nullptr, (void*)k_pages, (void*)v_pages, page_table, table_stride, seq_len, n_seqs, out,
                       workspace, n_splits, scale, window, nh, nkv, hd, stream);
}

// the same with terms on the scores (slopes [nh] float or null, softcap (0: none), see ScoreTerms) and with
// the merge of the splits inside the one launch (counters, items: see launch_decode; both may be null)
SYN_EXPORT int syn_attention_decode_terms_bf16(const void* q, const void* k_pages, const void* v_pages,
                                               const int* page_table, int table_stride, const int* seq_len, int n_seqs,
                                               void* out, float* workspace, int n_splits, float scale, int window,
                                               int nh, int nkv, int hd, const float* slopes, float softcap,
                                               int* counters, const int* items, int n_items, hipStream_t stream) {
  return launch_decode(q, nullptr, (void*)k_pages, (void*)v_pages, page_table, table_stride, seq_len, n_seqs, out,
                       workspace, n_splits, scale, window, nh, nkv, hd, stream, ScoreTerms{slopes, softcap}, counters,
                       items, n_items);
}

// ---- the same without a workspace argument: see no_alloc.h ----
// `scratch` is a device array; in host code its name is only a handle for hipGetSymbolAddress, never
// an address to hand to a kernel.  Each GPU holds its own copy at its own address: the address is
// looked up once per device, with that device current, and kept.
static __device__ __align__(256) unsigned char scratch[SYN_NOALLOC_SCRATCH_BYTES];
static float* scratch_of_device[SYN_MAX_DEVICES];

// What a first call on a device does besides launching: the address of this device's copy of the array, and
// the decode kernels' LDS limit.  Neither is stream work, so neither may happen while a stream is captured:
// callers that capture call this (or the entry point once) beforehand, with the device current.
SYN_EXPORT int syn_attention_decode_noalloc_init() {
  static OncePerDevice once;
  hipError_t e = once_per_device(once, [] {
    int dev = -1;
    hipError_t r = hipGetDevice(&dev);
    if (r != hipSuccess) return r;
    void* p = nullptr;
    r = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (r != hipSuccess) return r;
    if (p == nullptr) return hipErrorInvalidSymbol;
    scratch_of_device[dev] = (float*)p;   // once_per_device has checked dev and holds its lock
    return hipSuccess;
  });
  SYN_CHECK(e == hipSuccess, "attention_decode_noalloc: the scratch array has no address on the current device: %s",
            hipGetErrorString(e));
  e = raise_decode_lds();
  SYN_CHECK(e == hipSuccess, "attention_decode_noalloc: %zu bytes of LDS refused: %s", DEC_LDS_MAX, hipGetErrorString(e));
  return 0;
}

SYN_EXPORT int syn_attention_decode_bf16_noalloc(const void* q, const void* k_pages, const void* v_pages,
                                                 const int* page_table, int table_stride, const int* seq_len,
                                                 int n_seqs, void* out, int n_splits, float scale, int window, int nh,
                                                 int nkv, int hd, hipStream_t stream) {
  SYN_CHECK(n_seqs > 0 && nh > 0 && n_splits > 0 && hd > 0, "attention_decode_noalloc: empty input");
  const unsigned long long need = (unsigned long long)n_seqs * nh * n_splits * (hd + 2) * sizeof(float);
  SYN_CHECK(need <= SYN_NOALLOC_SCRATCH_BYTES,
            "attention_decode_noalloc: %d sequences x %d heads x %d splits need %llu bytes of partial results, the "
            "library keeps %u; use fewer splits or the entry point with a workspace argument",
            n_seqs, nh, n_splits, need, (unsigned)SYN_NOALLOC_SCRATCH_BYTES);
  if (const int rc = syn_attention_decode_noalloc_init()) return rc;   // after the first call on a device: two flag reads
  int dev = -1;
  const hipError_t e = hipGetDevice(&dev);
  SYN_CHECK(e == hipSuccess && dev >= 0 && dev < SYN_MAX_DEVICES, "attention_decode_noalloc: no current device (%s)",
            hipGetErrorString(e));
  float* ws = scratch_of_device[dev];   // written once, before the flag that the init call has just read under its lock
  return launch_decode(q, nullptr, (void*)k_pages, (void*)v_pages, page_table, table_stride, seq_len, n_seqs, out, ws,
                       n_splits, scale, window, nh, nkv, hd, stream);
}

// The same for one new token a sequence whose q, k and v come straight from the fused projection:
// qkv [n_seqs, (nh + 2 nkv) * hd] in bf16 (n_parts == 0), or n_parts float partial sums of that
// shape one after another.  q/k RMSNorm (gains may be null), rotation at position seq_len - 1 (tables
// may be null; `rot` dims rotate), and with own_kv the write of the new k and v into the cache happen
// inside the attention kernel.
SYN_EXPORT int syn_attention_decode_fused_bf16(const void* qkv, int n_parts, void* k_pages, void* v_pages,
                                               const int* page_table, int table_stride, const int* seq_len,
                                               int n_seqs, void* out, float* workspace, int n_splits, float scale,
                                               int window, int nh, int nkv, int hd, const void* q_gain,
                                               const void* k_gain, int gain_is_f32, float gain_offset, float eps,
                                               const float* cos_t,
                                               const float* sin_t, int rot, int own_kv, const float* slopes,
                                               float softcap, int* counters, const int* items, int n_items,
                                               hipStream_t stream) {
  SYN_CHECK(rot % 2 == 0 && rot >= 0 && rot <= hd, "attention_decode_fused: rotary size %d does not fit head size %d",
            rot, hd);
  SYN_CHECK((cos_t == nullptr) == (sin_t == nullptr), "attention_decode_fused: cos and sin come together");
  SYN_CHECK(n_parts >= 0 && n_parts <= 64, "attention_decode_fused: %d partial sums", n_parts);
  QkvIntake in;
  in.qkv = qkv;
  in.n_parts = n_parts;
  in.part_stride = (size_t)n_seqs * (nh + 2 * nkv) * hd;
  in.q_gain = q_gain, in.k_gain = k_gain, in.gain_is_f32 = gain_is_f32, in.gain_offset = gain_offset, in.eps = eps;
  in.cos_t = cos_t, in.sin_t = sin_t, in.rot = rot, in.own_kv = own_kv;
  return launch_decode(nullptr, &in, k_pages, v_pages, page_table, table_stride, seq_len, n_seqs, out, workspace,
                       n_splits, scale, window, nh, nkv, hd, stream, ScoreTerms{slopes, softcap}, counters, items,
                       n_items);
}
