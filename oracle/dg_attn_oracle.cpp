// CPU oracle for the denoise-step attention.  TEST INFRASTRUCTURE ONLY: see dg_attn_oracle.h
// for the reference file:line each function follows and for what pins it.
#include "dg_attn_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

inline uint32_t f32_bits(float v) {
  uint32_t u;
  std::memcpy(&u, &v, 4);
  return u;
}
inline float bits_f32(uint32_t u) {
  float v;
  std::memcpy(&v, &u, 4);
  return v;
}

inline int threads_or_all(int n) {
#ifdef _OPENMP
  return n > 0 ? n : omp_get_max_threads();
#else
  (void)n;
  return 1;
#endif
}

// Key bounds for one query row.  attention.metal:49-63, attention_mma2.metal:199-206.
struct RowRange {
  uint32_t lo, hi;          // visible iff lo <= t < hi ...
  uint32_t extra_lo;        // ... or t >= extra_lo (only when causal_sees_masked), always t < t_all
};

inline RowRange row_range(const dgo_desc& d, uint32_t tok) {
  const uint32_t t_all = d.kv_len + d.canvas;
  const bool causal = tok < d.causal_rows;
  const uint32_t qpos = d.kv_len + tok;
  RowRange r;
  r.hi = causal ? std::min(t_all, qpos + 1u) : t_all;
  r.lo = 0;
  if (d.window != 0) {
    const uint32_t wm1 = d.window - 1u;
    const uint32_t anchor = causal ? qpos : d.kv_len;
    r.lo = anchor > wm1 ? anchor - wm1 : 0u;
  }
  if (!causal && d.t_lo_override >= 0) r.lo = (uint32_t)d.t_lo_override;
  r.extra_lo = (causal && d.causal_sees_masked) ? d.kv_len + d.causal_rows : t_all;
  return r;
}

inline bool vis(const RowRange& r, uint32_t t, uint32_t t_all) {
  return t < t_all && ((t >= r.lo && t < r.hi) || t >= r.extra_lo);
}

inline uint32_t slot_of(const dgo_desc& d, uint32_t t) {
  return d.kv_ring_mask ? (t & d.kv_ring_mask) : t;  // attention_device.metal:27-33
}

inline float dot_seq(const float* a, const float* b, uint32_t n) {
  float s = 0.0f;
  for (uint32_t i = 0; i < n; ++i) s += a[i] * b[i];
  return s;
}

inline float dot_fast(const float* __restrict a, const float* __restrict b, uint32_t n) {
  float s = 0.0f;
#pragma omp simd reduction(+ : s)
  for (uint32_t i = 0; i < n; ++i) s += a[i] * b[i];
  return s;
}

// One key folded into one row's (m, l, acc): cpu.rs:175-188.
inline void fold_key(float s, const float* __restrict v, uint32_t hd, float& m, float& l,
                     float* __restrict acc) {
  const float mn = std::max(m, s);
  const float corr = std::exp(m - mn);
  const float p = std::exp(s - mn);
  for (uint32_t i = 0; i < hd; ++i) acc[i] *= corr;
  l = l * corr + p;
  m = mn;
  for (uint32_t i = 0; i < hd; ++i) acc[i] += p * v[i];
}

}  // namespace

extern "C" {

int dgo_max_threads(void) { return threads_or_all(0); }

void dgo_desc_reference_layout(dgo_desc* d) {
  const int64_t row = (int64_t)d->n_kv_heads * d->head_dim;
  d->k_off = 0;
  d->k_tok_stride = 2 * row;
  d->k_head_stride = d->head_dim;
  d->v_off = row;
  d->v_tok_stride = 2 * row;
  d->v_head_stride = d->head_dim;
}

void dgo_desc_head_major_layout(dgo_desc* d, int64_t t_cap) {
  d->k_off = 0;
  d->k_tok_stride = d->head_dim;
  d->k_head_stride = t_cap * d->head_dim;
  d->v_off = (int64_t)d->n_kv_heads * t_cap * d->head_dim;
  d->v_tok_stride = d->head_dim;
  d->v_head_stride = t_cap * d->head_dim;
}

int dgo_visible(const dgo_desc* d, uint32_t tok, uint32_t t) {
  return vis(row_range(*d, tok), t, d->kv_len + d->canvas) ? 1 : 0;
}

uint64_t dgo_visible_pairs(const dgo_desc* d) {
  const uint32_t t_all = d->kv_len + d->canvas;
  uint64_t n = 0;
  for (uint32_t tok = 0; tok < d->canvas; ++tok) {
    const RowRange r = row_range(*d, tok);
    const uint32_t hi = std::min(r.hi, t_all);
    if (hi > r.lo) n += hi - r.lo;
    const uint32_t e = std::max(r.extra_lo, hi);
    if (t_all > e) n += t_all - e;
  }
  return n;
}

void dgo_attention_f32(const dgo_desc* dp, const float* q, const float* kv, float* out, float* lse,
                       const uint32_t* tok_list, uint32_t n_tok, int n_threads) {
  const dgo_desc d = *dp;
  const uint32_t hd = d.head_dim, nq = d.n_q_heads, nkv = d.n_kv_heads;
  const uint32_t group = nq / nkv;
  const uint32_t t_all = d.kv_len + d.canvas;
  const float scale = d.scale == 0.0f ? 1.0f : d.scale;
  const uint32_t rows = tok_list ? n_tok : d.canvas;
  const bool strict = d.strict_order != 0;
  const long units = (long)rows * nkv;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads_or_all(n_threads))
  for (long u = 0; u < units; ++u) {
    const uint32_t tok = tok_list ? tok_list[u / nkv] : (uint32_t)(u / nkv);
    const uint32_t kvh = (uint32_t)(u % nkv);
    const RowRange r = row_range(d, tok);
    std::vector<float> acc((size_t)group * hd, 0.0f);
    std::vector<float> m(group, -std::numeric_limits<float>::infinity()), l(group, 0.0f);
    const uint32_t t_first = r.lo;
    for (uint32_t t = t_first; t < t_all; ++t) {
      if (!vis(r, t, t_all)) {
        if (t >= r.hi && r.extra_lo >= t_all) break;
        continue;
      }
      const uint32_t slot = slot_of(d, t);
      const float* kk = kv + d.k_off + (int64_t)slot * d.k_tok_stride + (int64_t)kvh * d.k_head_stride;
      const float* vv = kv + d.v_off + (int64_t)slot * d.v_tok_stride + (int64_t)kvh * d.v_head_stride;
      for (uint32_t g = 0; g < group; ++g) {
        const uint32_t qh = kvh * group + g;  // kvh = qh / (Hq/Hkv): cpu.rs:165
        const float* qv = q + ((size_t)tok * nq + qh) * hd;
        float s = strict ? dot_seq(qv, kk, hd) : dot_fast(qv, kk, hd);
        s *= scale;
        fold_key(s, vv, hd, m[g], l[g], &acc[(size_t)g * hd]);
      }
    }
    for (uint32_t g = 0; g < group; ++g) {
      const uint32_t qh = kvh * group + g;
      float* o = out + ((size_t)tok * nq + qh) * hd;
      const float* a = &acc[(size_t)g * hd];
      // attention_mma2.metal:297 guard: a row with no visible key stores 0.
      for (uint32_t i = 0; i < hd; ++i) o[i] = l[g] > 0.0f ? a[i] / l[g] : 0.0f;
      if (lse) lse[(size_t)tok * nq + qh] = m[g] + std::log(l[g]);
    }
  }
}

// Top-k sparse attention: attention_topk/cpu.rs:41-120 (selection, tie-break, renormalised softmax,
// summation in selection order) with the per-row k of attention_topk.metal:160-182.
uint32_t dgo_topk_row_k(const uint32_t k_cfg[4], uint32_t n_valid, int causal_row) {
  uint32_t k_req;
  if (k_cfg[1] != 0u) {
    const uint32_t gran = std::max(k_cfg[0], 1u);
    const uint32_t t_equiv = causal_row ? ((n_valid + gran - 1u) / gran) * gran : n_valid;
    k_req = std::min(std::max(t_equiv / k_cfg[1], k_cfg[2]), k_cfg[3]);
  } else {
    k_req = std::max(k_cfg[0], 1u);   // cpu.rs:59 (k.max(1))
  }
  return std::min(k_req, n_valid);
}

void dgo_attention_topk_f32(const dgo_desc* dp, const uint32_t k_cfg[4], const float* q, const float* kv, float* out,
                            uint32_t* sel_idx, uint32_t sel_cap, uint32_t* sel_count, const uint32_t* tok_list,
                            uint32_t n_tok, int n_threads) {
  const dgo_desc d = *dp;
  const uint32_t hd = d.head_dim, nq = d.n_q_heads, nkv = d.n_kv_heads;
  const uint32_t group = nq / nkv;
  const uint32_t t_all = d.kv_len + d.canvas;
  const float scale = d.scale == 0.0f ? 1.0f : d.scale;
  const uint32_t rows = tok_list ? n_tok : d.canvas;
  const long units = (long)rows * nq;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads_or_all(n_threads))
  for (long u = 0; u < units; ++u) {
    const uint32_t tok = tok_list ? tok_list[u / nq] : (uint32_t)(u / nq);
    const uint32_t qh = (uint32_t)(u % nq);
    const uint32_t kvh = qh / group;
    const RowRange r = row_range(d, tok);
    const float* qv = q + ((size_t)tok * nq + qh) * hd;
    float* o = out + ((size_t)tok * nq + qh) * hd;
    // step 1: every valid score, a sequential fp32 dot product (cpu.rs:70-80)
    std::vector<std::pair<float, uint32_t>> sc;
    sc.reserve(t_all);
    for (uint32_t t = 0; t < t_all; ++t) {
      if (!vis(r, t, t_all)) continue;
      const float* kk = kv + d.k_off + (int64_t)slot_of(d, t) * d.k_tok_stride + (int64_t)kvh * d.k_head_stride;
      sc.emplace_back(dot_seq(qv, kk, hd) * scale, t);
    }
    const uint32_t n_valid = (uint32_t)sc.size();
    const uint32_t kk_ = dgo_topk_row_k(k_cfg, n_valid, tok < d.causal_rows ? 1 : 0);
    for (uint32_t i = 0; i < hd; ++i) o[i] = 0.0f;
    if (sel_count) sel_count[(size_t)tok * nq + qh] = kk_;
    if (kk_ == 0) continue;
    // step 2: top-k by (score descending, index ascending) (cpu.rs:88-93)
    std::partial_sort(sc.begin(), sc.begin() + kk_, sc.end(), [](const auto& a, const auto& b) {
      return a.first > b.first || (a.first == b.first && a.second < b.second);
    });
    // step 3: softmax over the selected scores only (cpu.rs:95-104)
    const float mmax = sc[0].first;
    std::vector<float> probs(kk_);
    float l = 0.0f;
    for (uint32_t j = 0; j < kk_; ++j) {
      probs[j] = std::exp(sc[j].first - mmax);
      l += probs[j];
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    // step 4: weighted sum of the selected V rows, in selection order (cpu.rs:106-114)
    for (uint32_t j = 0; j < kk_; ++j) {
      const float pj = probs[j] * inv;
      const float* vv = kv + d.v_off + (int64_t)slot_of(d, sc[j].second) * d.v_tok_stride + (int64_t)kvh * d.v_head_stride;
      for (uint32_t i = 0; i < hd; ++i) o[i] += pj * vv[i];
      if (sel_idx && j < sel_cap) sel_idx[((size_t)tok * nq + qh) * sel_cap + j] = sc[j].second;
    }
  }
}

// FNV-1a, continuing seed_hash: src/metal/step_kernel/runtime.rs:127-133.
uint64_t dgo_fnv1a64(const uint8_t* bytes, size_t n, uint64_t seed_hash) {
  uint64_t h = seed_hash;
  for (size_t i = 0; i < n; ++i) {
    h ^= (uint64_t)bytes[i];
    h *= 0x00000100000001b3ull;
  }
  return h;
}

void dgo_attention_f64(const dgo_desc* dp, const float* q, const float* kv, double* out, double* lse,
                       const uint32_t* tok_list, uint32_t n_tok, int n_threads) {
  const dgo_desc d = *dp;
  const uint32_t hd = d.head_dim, nq = d.n_q_heads, nkv = d.n_kv_heads;
  const uint32_t group = nq / nkv;
  const uint32_t t_all = d.kv_len + d.canvas;
  const double scale = d.scale == 0.0f ? 1.0 : (double)d.scale;
  const uint32_t rows = tok_list ? n_tok : d.canvas;
  const long units = (long)rows * nq;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads_or_all(n_threads))
  for (long u = 0; u < units; ++u) {
    const uint32_t tok = tok_list ? tok_list[u / nq] : (uint32_t)(u / nq);
    const uint32_t qh = (uint32_t)(u % nq);
    const uint32_t kvh = qh / group;
    const RowRange r = row_range(d, tok);
    const float* qv = q + ((size_t)tok * nq + qh) * hd;
    std::vector<double> s(t_all, 0.0);
    std::vector<uint8_t> ok(t_all, 0);
    double mx = -std::numeric_limits<double>::infinity();
    for (uint32_t t = 0; t < t_all; ++t) {
      if (!vis(r, t, t_all)) continue;
      ok[t] = 1;
      const float* kk = kv + d.k_off + (int64_t)slot_of(d, t) * d.k_tok_stride + (int64_t)kvh * d.k_head_stride;
      double acc = 0.0;
      for (uint32_t i = 0; i < hd; ++i) acc += (double)qv[i] * (double)kk[i];
      s[t] = acc * scale;
      mx = std::max(mx, s[t]);
    }
    std::vector<double> o(hd, 0.0);
    double den = 0.0;
    for (uint32_t t = 0; t < t_all; ++t) {
      if (!ok[t]) continue;
      const double p = std::exp(s[t] - mx);
      den += p;
      const float* vv = kv + d.v_off + (int64_t)slot_of(d, t) * d.v_tok_stride + (int64_t)kvh * d.v_head_stride;
      for (uint32_t i = 0; i < hd; ++i) o[i] += p * (double)vv[i];
    }
    double* op = out + ((size_t)tok * nq + qh) * hd;
    for (uint32_t i = 0; i < hd; ++i) op[i] = den > 0.0 ? o[i] / den : 0.0;
    if (lse) lse[(size_t)tok * nq + qh] = mx + std::log(den);
  }
}

void dgo_attention_blocked_f32(const dgo_desc* dp, const float* q, const float* kv, float* out, float* lse,
                               uint32_t bk, int n_threads) {
  const dgo_desc d = *dp;
  const uint32_t hd = d.head_dim, nq = d.n_q_heads, nkv = d.n_kv_heads;
  const uint32_t group = nq / nkv;
  const uint32_t t_all = d.kv_len + d.canvas;
  const float scale = d.scale == 0.0f ? 1.0f : d.scale;
  const float ninf = -std::numeric_limits<float>::infinity();
  if (bk == 0) bk = 1;
  const long units = (long)d.canvas * nq;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads_or_all(n_threads))
  for (long u = 0; u < units; ++u) {
    const uint32_t tok = (uint32_t)(u / nq), qh = (uint32_t)(u % nq), kvh = qh / group;
    const RowRange r = row_range(d, tok);
    const float* qv = q + ((size_t)tok * nq + qh) * hd;
    float m = ninf, l = 0.0f;
    std::vector<float> acc(hd, 0.0f), sblock(bk);
    std::vector<uint32_t> tblock(bk);
    for (uint32_t t0 = 0; t0 < t_all; t0 += bk) {
      const uint32_t t1 = std::min(t0 + bk, t_all);
      // block scores and block max over the visible columns (attention_flash/mod.rs:57-69)
      float m_block = ninf;
      uint32_t n = 0;
      for (uint32_t t = t0; t < t1; ++t) {
        if (!vis(r, t, t_all)) continue;
        const float* kk = kv + d.k_off + (int64_t)slot_of(d, t) * d.k_tok_stride + (int64_t)kvh * d.k_head_stride;
        const float s = dot_seq(qv, kk, hd) * scale;
        m_block = std::max(m_block, s);
        sblock[n] = s;
        tblock[n] = t;
        ++n;
      }
      if (n == 0) continue;
      // online combine (attention_flash/mod.rs:70-86)
      const float m_new = std::max(m, m_block);
      const float corr = std::exp(m - m_new);
      for (uint32_t i = 0; i < hd; ++i) acc[i] *= corr;
      l *= corr;
      for (uint32_t j = 0; j < n; ++j) {
        const float p = std::exp(sblock[j] - m_new);
        const float* vv = kv + d.v_off + (int64_t)slot_of(d, tblock[j]) * d.v_tok_stride + (int64_t)kvh * d.v_head_stride;
        for (uint32_t i = 0; i < hd; ++i) acc[i] += p * vv[i];
        l += p;
      }
      m = m_new;
    }
    float* o = out + ((size_t)tok * nq + qh) * hd;
    for (uint32_t i = 0; i < hd; ++i) o[i] = l > 0.0f ? acc[i] / l : 0.0f;
    if (lse) lse[(size_t)tok * nq + qh] = m + std::log(l);
  }
}

void dgo_attention_partial_f32(const dgo_desc* dp, const float* q, const float* kv, uint32_t t_begin,
                               uint32_t t_end, float* acc_out, float* m_out, float* l_out, int n_threads) {
  const dgo_desc d = *dp;
  const uint32_t hd = d.head_dim, nq = d.n_q_heads, nkv = d.n_kv_heads;
  const uint32_t group = nq / nkv;
  const uint32_t t_all = d.kv_len + d.canvas;
  const float scale = d.scale == 0.0f ? 1.0f : d.scale;
  const long units = (long)d.canvas * nq;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads_or_all(n_threads))
  for (long u = 0; u < units; ++u) {
    const uint32_t tok = (uint32_t)(u / nq), qh = (uint32_t)(u % nq), kvh = qh / group;
    const RowRange r = row_range(d, tok);
    const float* qv = q + ((size_t)tok * nq + qh) * hd;
    float m = -std::numeric_limits<float>::infinity(), l = 0.0f;
    float* acc = acc_out + (size_t)u * hd;
    for (uint32_t i = 0; i < hd; ++i) acc[i] = 0.0f;
    for (uint32_t t = t_begin; t < std::min(t_end, t_all); ++t) {
      if (!vis(r, t, t_all)) continue;
      const uint32_t slot = slot_of(d, t);
      const float* kk = kv + d.k_off + (int64_t)slot * d.k_tok_stride + (int64_t)kvh * d.k_head_stride;
      const float* vv = kv + d.v_off + (int64_t)slot * d.v_tok_stride + (int64_t)kvh * d.v_head_stride;
      fold_key(dot_seq(qv, kk, hd) * scale, vv, hd, m, l, acc);
    }
    m_out[u] = m;
    l_out[u] = l;
  }
}

void dgo_merge_partials_f32(uint32_t rows, uint32_t head_dim, uint32_t n_parts, const float* const* acc,
                            const float* const* m, const float* const* l, float* out, float* lse) {
  for (uint32_t r = 0; r < rows; ++r) {
    float mx = -std::numeric_limits<float>::infinity();
    for (uint32_t p = 0; p < n_parts; ++p) mx = std::max(mx, m[p][r]);
    double den = 0.0;
    std::vector<double> o(head_dim, 0.0);
    for (uint32_t p = 0; p < n_parts; ++p) {
      if (!(l[p][r] > 0.0f)) continue;
      const double w = std::exp((double)m[p][r] - (double)mx);
      den += w * (double)l[p][r];
      const float* a = acc[p] + (size_t)r * head_dim;
      for (uint32_t i = 0; i < head_dim; ++i) o[i] += w * (double)a[i];
    }
    for (uint32_t i = 0; i < head_dim; ++i) out[(size_t)r * head_dim + i] = den > 0.0 ? (float)(o[i] / den) : 0.0f;
    if (lse) lse[r] = (float)((double)mx + std::log(den));
  }
}

void dgo_attention_bitmap_f32(uint32_t seq_len, uint32_t total_kv, uint32_t n_heads, uint32_t n_kv_heads,
                              uint32_t hd, const float* q, const float* k, const float* v,
                              const uint8_t* mask, float* out) {
  const float MASK_NEG = -1e9f;  // src/model/attention.rs:11
  const uint32_t n_groups = n_heads / n_kv_heads;
  const size_t kv_dim = (size_t)n_kv_heads * hd;
  std::vector<float> scores((size_t)seq_len * n_heads * total_kv);
  // attention_scores_gqa_ext (attention.rs:861-887)
  for (uint32_t qi = 0; qi < seq_len; ++qi)
    for (uint32_t h = 0; h < n_heads; ++h) {
      const uint32_t kv_h = h / n_groups;
      const float* qv = q + ((size_t)qi * n_heads + h) * hd;
      float* row = &scores[((size_t)qi * n_heads + h) * total_kv];
      for (uint32_t ki = 0; ki < total_kv; ++ki) row[ki] = dot_seq(qv, k + (size_t)ki * kv_dim + (size_t)kv_h * hd, hd);
    }
  // apply_decoder_mask (attention.rs:889-907)
  for (uint32_t qi = 0; qi < seq_len; ++qi)
    for (uint32_t h = 0; h < n_heads; ++h) {
      float* row = &scores[((size_t)qi * n_heads + h) * total_kv];
      for (uint32_t ki = 0; ki < total_kv; ++ki)
        if (!mask[(size_t)qi * total_kv + ki]) row[ki] = MASK_NEG;
    }
  // softmax_rows (shaders/cpu/mod.rs:175-190)
  for (size_t r = 0; r < (size_t)seq_len * n_heads; ++r) {
    float* row = &scores[r * total_kv];
    float mx = -std::numeric_limits<float>::infinity();
    for (uint32_t c = 0; c < total_kv; ++c) mx = std::max(mx, row[c]);
    float sum = 0.0f;
    for (uint32_t c = 0; c < total_kv; ++c) {
      row[c] = std::exp(row[c] - mx);
      sum += row[c];
    }
    const float inv = 1.0f / sum;
    for (uint32_t c = 0; c < total_kv; ++c) row[c] *= inv;
  }
  // attention_output_gqa_ext (attention.rs:909-934)
  std::fill(out, out + (size_t)seq_len * n_heads * hd, 0.0f);
  for (uint32_t qi = 0; qi < seq_len; ++qi)
    for (uint32_t h = 0; h < n_heads; ++h) {
      const uint32_t kv_h = h / n_groups;
      const float* row = &scores[((size_t)qi * n_heads + h) * total_kv];
      float* o = out + ((size_t)qi * n_heads + h) * hd;
      for (uint32_t ki = 0; ki < total_kv; ++ki) {
        const float w = row[ki];
        const float* vv = v + (size_t)ki * kv_dim + (size_t)kv_h * hd;
        for (uint32_t i = 0; i < hd; ++i) o[i] += w * vv[i];
      }
    }
}

// ---- rounding: bf16.rs:5-41, f16.rs:3-47 ----
uint16_t dgo_f32_to_bf16_trunc(float v) { return (uint16_t)(f32_bits(v) >> 16); }

uint16_t dgo_f32_to_bf16_rne(float v) {
  uint32_t u = f32_bits(v);
  if ((u & 0x7f800000u) == 0x7f800000u) {  // inf / nan
    if (u & 0x007fffffu) return (uint16_t)((u >> 16) | 0x0040u);
    return (uint16_t)(u >> 16);
  }
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

float dgo_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

uint16_t dgo_f32_to_f16_trunc(float v) {
  // v.clamp(-65504, 65504) propagates NaN like Rust's f32::clamp
  float c = v;
  if (c < -65504.0f) c = -65504.0f;
  if (c > 65504.0f) c = 65504.0f;
  const uint32_t bits = f32_bits(c);
  const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
  const int exp = (int)((bits >> 23) & 0xffu);
  const uint32_t mant = bits & 0x7fffffu;
  if (exp == 0xff) return (uint16_t)(sign | (mant == 0 ? 0 : 0x7e00));
  if (exp == 0) return sign;
  const int new_exp = exp - 127 + 15;
  if (new_exp >= 0x1f) return (uint16_t)(sign | 0x7c00);
  if (new_exp <= 0) return sign;
  return (uint16_t)(sign | ((uint16_t)new_exp << 10) | (uint16_t)(mant >> 13));
}

uint16_t dgo_f32_to_f16_rne(float v) {
  const uint32_t x = f32_bits(v);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return (uint16_t)(sign | (ax > 0x7f800000u ? 0x7e00u : 0x7c00u));
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds to >= 65520 -> inf
  if (ax < 0x33000001u) return (uint16_t)sign;                // below half the smallest subnormal
  int exp = (int)(ax >> 23) - 127;
  uint32_t mant = (ax & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t base;
  if (exp < -14) {  // subnormal result
    shift = 13 + (-14 - exp);
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(exp + 15) << 10;
    mant &= 0x7fffffu;
  }
  uint32_t half = mant >> shift;
  const uint32_t rem = mant & ((1u << shift) - 1u);
  const uint32_t mid = 1u << (shift - 1);
  if (rem > mid || (rem == mid && (half & 1u))) ++half;
  return (uint16_t)(sign | (base + half));
}

float dgo_f16_to_f32(uint16_t bits) {
  const uint32_t sign = (bits >> 15) & 1u, exp = (bits >> 10) & 0x1fu, mant = bits & 0x3ffu;
  if (exp == 0) {
    if (mant == 0) return sign ? -0.0f : 0.0f;
    const float val = (float)mant * 5.9604644775390625e-08f;  // 2^-24
    return sign ? -val : val;
  }
  if (exp == 0x1f) {
    if (mant == 0) return sign ? -std::numeric_limits<float>::infinity() : std::numeric_limits<float>::infinity();
    return std::numeric_limits<float>::quiet_NaN();
  }
  return bits_f32((sign << 31) | ((exp + 112u) << 23) | (mant << 13));
}

void dgo_to_bits(const float* x, uint16_t* bits, size_t n, int mode) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < (long)n; ++i) {
    switch (mode) {
      case 0: bits[i] = dgo_f32_to_bf16_trunc(x[i]); break;
      case 1: bits[i] = dgo_f32_to_bf16_rne(x[i]); break;
      case 2: bits[i] = dgo_f32_to_f16_trunc(x[i]); break;
      default: bits[i] = dgo_f32_to_f16_rne(x[i]); break;
    }
  }
}

void dgo_from_bits(const uint16_t* bits, float* x, size_t n, int is_f16) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < (long)n; ++i) x[i] = is_f16 ? dgo_f16_to_f32(bits[i]) : dgo_bf16_to_f32(bits[i]);
}

void dgo_round_array(float* x, size_t n, int mode) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < (long)n; ++i) {
    switch (mode) {
      case 0: x[i] = dgo_bf16_to_f32(dgo_f32_to_bf16_trunc(x[i])); break;
      case 1: x[i] = dgo_bf16_to_f32(dgo_f32_to_bf16_rne(x[i])); break;
      case 2: x[i] = dgo_f16_to_f32(dgo_f32_to_f16_trunc(x[i])); break;
      default: x[i] = dgo_f16_to_f32(dgo_f32_to_f16_rne(x[i])); break;
    }
  }
}

void dgo_rms_norm_no_scale(float* out, const float* x, size_t n, float eps) {
  float sum_sq = 0.0f;
  for (size_t i = 0; i < n; ++i) sum_sq += x[i] * x[i];
  const float rms_inv = 1.0f / std::sqrt(sum_sq / (float)n + eps);
  for (size_t i = 0; i < n; ++i) out[i] = x[i] * rms_inv;
}

void dgo_rms_norm_head(float* x, const float* weight, size_t n, float eps) {
  float ss = 0.0f;
  for (size_t i = 0; i < n; ++i) ss += x[i] * x[i];
  const float inv = 1.0f / std::sqrt(ss / (float)n + eps);
  for (size_t i = 0; i < n; ++i) x[i] *= inv * (weight ? weight[i] : 1.0f);
}

// ---- producer: per-head RMSNorm + RoPE + KV-cache write ----
void dgo_rope_split_half(float* x, uint32_t rot, uint32_t head_dim, float theta, uint32_t pos) {  // cpu.rs:31-45
  const uint32_t half_rot = rot / 2;
  for (uint32_t dd = 0; dd < half_rot; ++dd) {
    const float inv_freq = std::pow(theta, -2.0f * (float)dd / (float)head_dim);
    const float a = (float)pos * inv_freq;
    const float c = std::cos(a), s = std::sin(a);
    const float x0 = x[dd], x1 = x[dd + half_rot];
    x[dd] = x0 * c - x1 * s;
    x[dd + half_rot] = x0 * s + x1 * c;
  }
}

void dgo_rope_proportional(float* x, uint32_t rotary_dim, uint32_t head_dim, float theta, uint32_t pos) {  // cpu.rs:48-65
  const uint32_t half_head = head_dim / 2, half_rot = rotary_dim / 2;
  for (uint32_t dd = 0; dd < half_rot; ++dd) {
    const float inv_freq = std::pow(theta, -2.0f * (float)dd / (float)head_dim);
    const float a = (float)pos * inv_freq;
    const float c = std::cos(a), s = std::sin(a);
    const float x0 = x[dd], x1 = x[half_head + dd];
    x[dd] = x0 * c - x1 * s;
    x[half_head + dd] = x0 * s + x1 * c;
  }
}

void dgo_qk_rope_kv_f32(const dgo_rope_desc* d, float* q, float* k, const float* v, float* kvcache,
                        const float* q_norm_w, const float* k_norm_w) {  // cpu.rs:78-145
  const uint32_t hd = d->head_dim, nkv = d->n_kv_heads, nq = d->n_q_heads;
  const uint32_t rot = d->is_full ? hd / 4 : hd;            // cpu.rs:17-23
  const float theta = d->is_full ? 1.0e6f : 1.0e4f;         // cpu.rs:25-27
  std::vector<float> tmp(hd);
  for (uint32_t tok = 0; tok < d->canvas; ++tok) {
    const uint32_t pos = d->kv_len + tok;
    const bool kv_write = pos < d->kv_write_end;            // qk_rope_kv.metal:56-60
    const int64_t slot = d->kv_ring_mask ? (int64_t)(pos & d->kv_ring_mask) : (int64_t)pos;  // attention_device.metal:28-30
    for (uint32_t h = 0; h < nq + 2 * nkv; ++h) {
      const bool is_q = h < nq, is_k = !is_q && h < nq + nkv;
      const uint32_t hh = is_q ? h : (h - nq) % nkv;
      if (!is_q && !is_k) {                                 // V head: cpu.rs:110-122
        const float* src = (d->v_from_k ? k : v) + ((size_t)tok * nkv + hh) * hd;
        std::copy(src, src + hd, tmp.begin());
        dgo_rms_norm_head(tmp.data(), nullptr, hd, 1e-6f);
        if (kv_write) std::copy(tmp.begin(), tmp.end(), kvcache + d->v_off + slot * d->v_tok_stride + (int64_t)hh * d->v_head_stride);
        continue;
      }
      float* head = is_q ? q + ((size_t)tok * nq + hh) * hd : k + ((size_t)tok * nkv + hh) * hd;
      std::copy(head, head + hd, tmp.begin());
      dgo_rms_norm_head(tmp.data(), is_q ? q_norm_w : k_norm_w, hd, 1e-6f);
      if (d->is_full) dgo_rope_proportional(tmp.data(), rot, hd, theta, pos);
      else dgo_rope_split_half(tmp.data(), rot, hd, theta, pos);
      if (is_k) {
        if (kv_write) std::copy(tmp.begin(), tmp.end(), kvcache + d->k_off + slot * d->k_tok_stride + (int64_t)hh * d->k_head_stride);
        // V aliases the raw k projection on such layers: leave k untouched for the V pass (cpu.rs:137-140)
        if (!d->v_from_k) std::copy(tmp.begin(), tmp.end(), head);
      } else {
        std::copy(tmp.begin(), tmp.end(), head);
      }
    }
  }
}

void dgo_fixture_rope(int which, float* q, float* k, float* v, float* qw, float* kw) {  // qk_rope_kv/mod.rs:80-189
  if (which == 0) {          // tiny_fixture: canvas 2, Hq 4, Hkv 2, hd 32
    const size_t nq = 2 * 4 * 32, nk = 2 * 2 * 32;
    for (size_t i = 0; i < nq; ++i) q[i] = std::sin((float)i * 0.13f) * 0.5f;
    for (size_t i = 0; i < nk; ++i) k[i] = std::cos((float)i * 0.17f) * 0.4f;
    for (size_t i = 0; i < nk; ++i) v[i] = std::sin((float)i * 0.11f) * 0.3f;
    for (size_t i = 0; i < 32; ++i) qw[i] = kw[i] = 1.0f;
  } else if (which == 1) {   // full_layer_fixture: canvas 2, Hq 4, Hkv 2, hd 64
    const size_t nq = 2 * 4 * 64, nk = 2 * 2 * 64;
    for (size_t i = 0; i < nq; ++i) q[i] = std::sin((float)i * 0.07f) * 0.6f;
    for (size_t i = 0; i < nk; ++i) k[i] = std::cos((float)i * 0.09f) * 0.5f;
    for (size_t i = 0; i < nk; ++i) v[i] = std::sin((float)i * 0.08f) * 0.45f;
    for (size_t i = 0; i < 64; ++i) qw[i] = kw[i] = 1.0f;
  } else {                   // full_hd512_v_alias_fixture: canvas 1, Hq 16, Hkv 2, hd 512
    const size_t nq = 1 * 16 * 512, nk = 1 * 2 * 512;
    for (size_t i = 0; i < nq; ++i) q[i] = std::sin((float)i * 0.031f) * 0.55f;
    for (size_t i = 0; i < nk; ++i) k[i] = std::cos((float)i * 0.029f) * 0.48f;
    for (size_t i = 0; i < nk; ++i) v[i] = 0.0f;
    for (size_t i = 0; i < 512; ++i) {
      qw[i] = 1.0f + (float)i * 0.0001f;
      kw[i] = 1.0f - (float)i * 0.00005f;
    }
  }
}

// ---- fixture generators ----
void dgo_fixture_tiny(float* q, float* kv) {  // attention/mod.rs:59-95
  const uint32_t canvas = 2, nq = 4, nkv = 2, hd = 32, kv_len = 2, t_total = kv_len + canvas;
  for (uint32_t t = 0; t < t_total; ++t)
    for (uint32_t h = 0; h < nkv; ++h)
      for (uint32_t dd = 0; dd < hd; ++dd) {
        const size_t k_i = (size_t)t * nkv * hd * 2 + h * hd + dd;
        const size_t v_i = (size_t)t * nkv * hd * 2 + nkv * hd + h * hd + dd;
        kv[k_i] = std::sin((float)(t * 17 + h * 3 + dd) * 0.05f);
        kv[v_i] = std::cos((float)(t * 13 + h * 5 + dd) * 0.04f);
      }
  for (uint32_t i = 0; i < canvas * nq * hd; ++i) q[i] = std::sin((float)i * 0.11f) * 0.6f;
}

void dgo_fixture_wide(float* q, float* kv) {  // attention/mod.rs:97-126
  const uint32_t canvas = 4, nq = 8, nkv = 2, hd = 64, kv_len = 4, t_total = kv_len + canvas;
  for (uint32_t i = 0; i < t_total * nkv * hd * 2; ++i) kv[i] = std::sin((float)i * 0.031f) * 0.3f;
  for (uint32_t i = 0; i < canvas * nq * hd; ++i) q[i] = std::cos((float)i * 0.02f) * 0.5f;
}

void dgo_fixture_model_attn(uint32_t canvas, uint32_t nq, uint32_t nkv, uint32_t hd, uint32_t kv_len,
                            float* q, float* kv) {  // attention/mod.rs:128-167
  const size_t t_total = (size_t)kv_len + canvas;
  for (size_t t = 0; t < t_total; ++t)
    for (size_t h = 0; h < nkv; ++h)
      for (size_t dd = 0; dd < hd; ++dd) {
        const size_t k_i = t * nkv * hd * 2 + h * hd + dd;
        const size_t v_i = k_i + (size_t)nkv * hd;
        kv[k_i] = std::sin((float)(t * 19 + h * 7 + dd) * 0.0031f) * 0.4f;
        kv[v_i] = std::cos((float)(t * 23 + h * 11 + dd) * 0.0027f) * 0.35f;
      }
  const size_t nqe = (size_t)canvas * nq * hd;
  for (size_t i = 0; i < nqe; ++i) q[i] = std::sin((float)i * 0.017f) * 0.5f + 0.02f * (float)(i % hd);
}

void dgo_fixture_model_full(uint32_t canvas, uint32_t nq, uint32_t nkv, uint32_t hd, uint32_t kv_len,
                            float* q, float* kv) {  // attention_gemm/mod.rs:410-432
  const size_t t_total = (size_t)kv_len + canvas;
  const size_t nkve = t_total * nkv * hd * 2;
  for (size_t i = 0; i < nkve; ++i) kv[i] = std::sin((float)(i % 4096) * 0.0007f) * 0.35f;
  const size_t nqe = (size_t)canvas * nq * hd;
  for (size_t i = 0; i < nqe; ++i) q[i] = std::sin((float)i * 0.013f) * 0.4f;
}

void dgo_synthetic_fill_kv(uint16_t* bits, size_t n, uint64_t seed) {  // step_kernel/runtime.rs:190-206
  uint64_t s = seed | 1u;
  for (size_t i = 0; i < n; ++i) {
    s ^= s >> 12;
    s ^= s << 25;
    s ^= s >> 27;
    const uint16_t r = (uint16_t)((s * 0x2545F4914F6CDD1DULL) >> 32);
    bits[i] = (uint16_t)((r & 0x03FF) | 0x3000 | ((r & 0x0400) << 5));
  }
}

}  // extern "C"
