// Plain C++ twins of the HIP kernels: the same operations on float arrays in host memory, written for
// reading, one loop nest each, no tiling and no vector code.  They are the oracle that stands beside
// every kernel, in the role of the reference's CPU kernels
// (crates/synaptix-kernels-cpu/src/rmsnorm.rs:1-27, attention.rs:3-51).
//
// Layouts are the kernels' own, in their plain (float) form: rows [n, width]; cache pages
// k[page, kv_head, 64, hd] and v[page, kv_head, hd, 64]; a page table [sequences, table_stride].
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <vector>

#define REF_API extern "C" __attribute__((visibility("default")))
static const int PAGE = 64;

// x[n, :] = table[ids[n], :]
REF_API void ref_embed(const float* table, const int* ids, float* out, int n, int width) {
  for (int i = 0; i < n; ++i)
    for (int d = 0; d < width; ++d) out[(size_t)i * width + d] = table[(size_t)ids[i] * width + d];
}

// resid += delta (if given); out = resid * rsqrt(mean(resid^2) + eps) * (gain_offset + gain)
REF_API void ref_add_rmsnorm(float* resid, const float* delta, const float* gain, float gain_offset, float eps,
                             float* out, int n, int width) {
  for (int i = 0; i < n; ++i) {
    float* x = resid + (size_t)i * width;
    double ss = 0.0;
    for (int d = 0; d < width; ++d) {
      if (delta) x[d] += delta[(size_t)i * width + d];
      ss += (double)x[d] * x[d];
    }
    const float inv = 1.0f / std::sqrt((float)(ss / width) + eps);
    for (int d = 0; d < width; ++d) out[(size_t)i * width + d] = (gain_offset + gain[d]) * x[d] * inv;
  }
}

// out[n, i] = silu(gu[n, i]) * gu[n, I + i], silu(z) = z / (1 + e^-z)
REF_API void ref_swiglu(const float* gu, float* out, int n, int inter) {
  for (int r = 0; r < n; ++r)
    for (int i = 0; i < inter; ++i) {
      const float g = gu[(size_t)r * 2 * inter + i], u = gu[(size_t)r * 2 * inter + inter + i];
      out[(size_t)r * inter + i] = g / (1.0f + std::exp(-g)) * u;
    }
}

// out[M, N] = x[M, K] . w[N, K]^T
REF_API void ref_gemm(const float* x, const float* w, float* out, int M, int N, int K) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) acc += (double)x[(size_t)m * K + k] * w[(size_t)n * K + k];
      out[(size_t)m * N + n] = (float)acc;
    }
}

// One head: optional RMSNorm over the head, then the half-split rotation of the first `rot` dims at
// position pos (cos, sin [positions, rot / 2]; null: no rotation).
static void norm_and_rotate(const float* x, float* o, int hd, const float* gain, float gain_offset, float eps,
                            const float* cos_t, const float* sin_t, int rot, int pos) {
  std::vector<float> t(x, x + hd);
  if (gain) {
    double ss = 0.0;
    for (int d = 0; d < hd; ++d) ss += (double)x[d] * x[d];
    const float inv = 1.0f / std::sqrt((float)(ss / hd) + eps);
    for (int d = 0; d < hd; ++d) t[d] = (gain_offset + gain[d]) * x[d] * inv;
  }
  const int half = rot / 2;
  for (int d = 0; d < hd; ++d) {
    if (!cos_t || d >= rot) {
      o[d] = t[d];
    } else if (d < half) {
      o[d] = t[d] * cos_t[(size_t)pos * half + d] - t[d + half] * sin_t[(size_t)pos * half + d];
    } else {
      o[d] = t[d] * cos_t[(size_t)pos * half + d - half] + t[d - half] * sin_t[(size_t)pos * half + d - half];
    }
  }
}

// A fused projection row [q heads | k heads | v heads] of each token: q and k normed and rotated, q to
// q_out, k and v into the pages of the token's sequence at its position.
REF_API void ref_qk_norm_rope_kv_write(const float* qkv, float* q_out, float* k_pages, float* v_pages,
                                       const int* page_table, int table_stride, const int* tok_seq, const int* tok_pos,
                                       const float* q_gain, const float* k_gain, float gain_offset, float eps,
                                       const float* cos_t, const float* sin_t, int rot, int n_tokens, int nh, int nkv,
                                       int hd, int write_kv) {
  const int heads = nh + 2 * nkv;
  std::vector<float> tmp(hd);
  for (int n = 0; n < n_tokens; ++n) {
    const int pos = tok_pos[n];
    const float* row = qkv + (size_t)n * heads * hd;
    for (int h = 0; h < nh; ++h)
      norm_and_rotate(row + (size_t)h * hd, q_out + ((size_t)n * nh + h) * hd, hd, q_gain, gain_offset, eps, cos_t, sin_t,
                      rot, pos);
    if (!write_kv) continue;
    const int page = page_table[(size_t)tok_seq[n] * table_stride + pos / PAGE];
    for (int h = 0; h < nkv; ++h) {
      norm_and_rotate(row + (size_t)(nh + h) * hd, tmp.data(), hd, k_gain, gain_offset, eps, cos_t, sin_t, rot, pos);
      for (int d = 0; d < hd; ++d) {
        k_pages[(((size_t)page * nkv + h) * PAGE + pos % PAGE) * hd + d] = tmp[d];
        v_pages[(((size_t)page * nkv + h) * hd + d) * PAGE + pos % PAGE] = row[(size_t)(nh + nkv + h) * hd + d];
      }
    }
  }
}

// Causal attention of each token over the pages of its sequence: key j is visible from position p iff
// j <= p and (window == 0 or p < j + window); head h reads kv head h / (nh / nkv); exact two-pass softmax.
REF_API void ref_attention(const float* q, const float* k_pages, const float* v_pages, const int* page_table,
                           int table_stride, const int* tok_seq, const int* tok_pos, float* out, float scale, int window,
                           int n_tokens, int nh, int nkv, int hd) {
  const int g = nh / nkv;
  std::vector<double> score;
  for (int n = 0; n < n_tokens; ++n) {
    const int pos = tok_pos[n], first = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
    const int* pages = page_table + (size_t)tok_seq[n] * table_stride;
    for (int h = 0; h < nh; ++h) {
      const int kvh = h / g;
      const float* qh = q + ((size_t)n * nh + h) * hd;
      score.assign(pos + 1, 0.0);
      double top = -INFINITY;
      for (int j = first; j <= pos; ++j) {
        const float* kr = k_pages + (((size_t)pages[j / PAGE] * nkv + kvh) * PAGE + j % PAGE) * hd;
        double s = 0.0;
        for (int d = 0; d < hd; ++d) s += (double)qh[d] * kr[d];
        score[j] = s * scale;
        if (score[j] > top) top = score[j];
      }
      double sum = 0.0;
      for (int j = first; j <= pos; ++j) sum += (score[j] = std::exp(score[j] - top));
      for (int d = 0; d < hd; ++d) {
        double acc = 0.0;
        for (int j = first; j <= pos; ++j)
          acc += score[j] * v_pages[(((size_t)pages[j / PAGE] * nkv + kvh) * hd + d) * PAGE + j % PAGE];
        out[((size_t)n * nh + h) * hd + d] = (float)(acc / sum);
      }
    }
  }
}

// out[r] = the last of the largest logits where temperature is null or <= 0, else the first index whose
// cumulated softmax(logits / temperature) exceeds uniform[r] (the last index if none does).
REF_API void ref_sample_rows(const float* logits, const float* temperature, const float* uniform, int* out, int rows,
                             int vocab) {
  for (int r = 0; r < rows; ++r) {
    const float* x = logits + (size_t)r * vocab;
    int best = 0;
    for (int i = 0; i < vocab; ++i)
      if (x[i] >= x[best]) best = i;
    if (!temperature || temperature[r] <= 0.0f) {
      out[r] = best;
      continue;
    }
    const float t = temperature[r], top = x[best] / t;
    double sum = 0.0;
    for (int i = 0; i < vocab; ++i) sum += std::exp((double)(x[i] / t - top));
    double cum = 0.0;
    int pick = vocab - 1;
    for (int i = 0; i < vocab; ++i) {
      cum += std::exp((double)(x[i] / t - top)) / sum;
      if ((double)uniform[r] < cum) {
        pick = i;
        break;
      }
    }
    out[r] = pick;
  }
}
