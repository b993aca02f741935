// Attention over the paged cache in true 32-bit: one wave for each (token, head), plain FMA,
// online softmax over blocks of 64 keys.  Any head size up to 256, prefill and decode alike.
//
//   query of token t sits at position p = tok_pos[t] of sequence tok_seq[t];
//   key j is visible iff j <= p and (window <= 0 or j > p - window);
//   head h reads kv head h / (nh / nkv).
// Definition as in crates/synaptix-kernels-cuda/tests/cuda_flash_decode.rs:32-90 and the mask of
// crates/synaptix-models/llm/common/src/model.rs:2581-2596.
//
// Cache pages hold 64 tokens: k_pages[page, kv_head, token, d], v_pages[page, kv_head, d, token].
#include "common.h"

#define ATTN32_MAX_HD 256

__global__ void __launch_bounds__(SYN_WAVE)
attn_f32_kernel(const float* __restrict__ q, const float* __restrict__ k_pages, const float* __restrict__ v_pages,
                const int* __restrict__ page_table, int table_stride, const int* __restrict__ tok_seq,
                const int* __restrict__ tok_pos, float* __restrict__ out, float scale, int window, int nh, int nkv,
                int hd, ScoreTerms terms) {
  __shared__ float qs[ATTN32_MAX_HD];
  __shared__ float ps[SYN_PAGE];
  const int tok = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int seq = tok_seq[tok], pos = tok_pos[tok];
  const int kvh = head / (nh / nkv);
  const float* qr = q + ((size_t)tok * nh + head) * hd;
  for (int d = lane; d < hd; d += SYN_WAVE) qs[d] = qr[d];
  __syncthreads();

  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const bool with_terms = score_terms_on(terms);
  const float slope = terms.slopes ? terms.slopes[head] : 0.f;
  float m = -INFINITY, l = 0.f;
  float o[ATTN32_MAX_HD / SYN_WAVE] = {0.f, 0.f, 0.f, 0.f};
  for (int kb = lo / SYN_PAGE; kb <= pos / SYN_PAGE; ++kb) {
    const int page = page_table[(size_t)seq * table_stride + kb];
    const size_t base = ((size_t)page * nkv + kvh) * SYN_PAGE * hd;
    const int key = kb * SYN_PAGE + lane;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const float* kr = k_pages + base + (size_t)lane * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], kr[d], dot);
      s = dot * scale;
      if (with_terms) s = score_with_terms(s, slope, terms.softcap, pos, key);
    }
    const float m_new = fmaxf(m, wave_max(s));  // every block of the range holds a visible key
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
    ps[lane] = p;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ATTN32_MAX_HD / SYN_WAVE; ++i) {
      const int d = lane + i * SYN_WAVE;
      if (d < hd) {
        const float* vr = v_pages + base + (size_t)d * SYN_PAGE;
        float acc = o[i] * alpha;
        for (int j = 0; j < SYN_PAGE; ++j) {
          const float pj = ps[j];
          if (pj != 0.f) acc = fmaf(pj, vr[j], acc);  // slots past the sequence's end may hold anything
        }
        o[i] = acc;
      }
    }
    __syncthreads();
  }
  float* orow = out + ((size_t)tok * nh + head) * hd;
#pragma unroll
  for (int i = 0; i < ATTN32_MAX_HD / SYN_WAVE; ++i) {
    const int d = lane + i * SYN_WAVE;
    if (d < hd) orow[d] = o[i] / l;
  }
}

// slopes [nh] float or null, softcap (0: none): see ScoreTerms
SYN_EXPORT int syn_attention_f32(const float* q, const float* k_pages, const float* v_pages, const int* page_table,
                                 int table_stride, const int* tok_seq, const int* tok_pos, float* out, float scale,
                                 int window, int n_tokens, int nh, int nkv, int hd, const float* slopes, float softcap,
                                 hipStream_t stream) {
  SYN_CHECK(softcap >= 0.f, "attention_f32: a soft cap of %g", (double)softcap);
  SYN_CHECK(n_tokens > 0 && nh > 0 && nkv > 0, "attention_f32: empty input");
  SYN_CHECK(nh % nkv == 0, "attention_f32: %d heads do not divide into %d kv heads", nh, nkv);
  SYN_CHECK(hd > 0 && hd <= ATTN32_MAX_HD, "attention_f32: head size %d is outside 1..%d", hd, ATTN32_MAX_HD);
  attn_f32_kernel<<<dim3(n_tokens, nh), SYN_WAVE, 0, stream>>>(q, k_pages, v_pages, page_table, table_stride, tok_seq,
                                                               tok_pos, out, scale, window, nh, nkv, hd,
                                                               ScoreTerms{slopes, softcap});
  SYN_LAUNCH_CHECK("attention_f32");
  return 0;
}
