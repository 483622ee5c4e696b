// Top-k sparse attention for gfx950 (MI355X): per (query row, head) only the k highest-scoring
// visible keys are kept, softmax is renormalised over them and their V rows are gathered
// (reference: src/shaders/attn/attention_topk/attention_topk.metal, CPU twin cpu.rs:41-120).
//
// Two kernels per pass over a block of canvas rows:
//   topk_scores_kernel  S = Q.K^T on MFMA, fp32, written to a score plane [Hq][rows][t_pad].  Same
//                       decomposition as the dense kernel (stacked GQA rows, K tiles by
//                       direct-to-LDS loads, Q resident in registers) without softmax or P.V,
//                       so key-range splits need no merge: every split writes its own columns.
//   topk_select_kernel  one workgroup per (row, head): exact top-k by fp32 score with a radix
//                       select on the order-preserving integer image of the scores (11 + 11 + 10
//                       bits).  Histogram levels run over the score row in memory only until the
//                       class that holds the k-th score fits an LDS candidate list (at most one
//                       level for model-sized rows, none for short ones); the remaining levels,
//                       the tie-break (equal scores: lower key position first, as the CPU twin)
//                       and the softmax run in LDS.  The kept keys are sorted by position, so the
//                       order of the P.V sum and with it every output bit is reproducible, then the
//                       V rows are gathered with one 16-byte load per lane and row (hd 512).
// The host walks the canvas in row blocks sized so that the score plane stays within the
// memory-side cache.
#include "attn_params.h"
#include "mfma_tile.h"

namespace dg {
namespace {

constexpr int kCandCap = 4096;     // LDS candidate list of the select kernel
// radix digits of the 32-bit key, most significant first: 11 + 11 + 10 bits
__device__ __forceinline__ uint32_t digit_shift(int level) { return level == 0 ? 21u : level == 1 ? 10u : 0u; }
__device__ __forceinline__ uint32_t digit_bits(int level) { return level == 2 ? 10u : 11u; }
constexpr int kMaxBins = 2048;

// ---------------------------------------------------------------------------------------------
// scores
// ---------------------------------------------------------------------------------------------

// wait until at most N vector-memory operations of this wave are outstanding, then the workgroup
// barrier, as one statement the compiler cannot move memory accesses across.  (A __syncthreads()
// would also wait for the score stores, and with them for every prefetched tile.)
template <int N>
__device__ __forceinline__ void wait_loads_then_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt immediate");
  constexpr int enc = 0x0F70 | (N & 15) | ((N >> 4) << 14);
  asm volatile("s_waitcnt %0\n\ts_barrier" ::"n"(enc) : "memory");
}

template <int D, bool F16>
__global__ void __launch_bounds__(256) topk_scores_kernel(const TopkParams tp) {
  const AttnParams& p = tp.a;
  using L = Lay<D>;
  constexpr int NSTEP = D / 16;
  constexpr int NLD = L::NLD;
  constexpr int PF = 3, NB = PF + 1;   // K tiles in flight ahead of the one being multiplied
  static_assert((PF - 1) * NLD < 64, "wait count");
  __shared__ __attribute__((aligned(1024))) char smem[NB * L::K_BYTES];

  // (KV head, split, row tile) units in 8 equal runs, one per XCD (ids go round-robin over them)
  const uint32_t n_units = p.hkv * tp.n_splits * tp.n_mtiles;
  const uint32_t per_xcd = (n_units + 7u) >> 3;
  const uint32_t wg = blockIdx.x;
  const uint32_t unit = (wg & 7u) * per_xcd + (wg >> 3);
  if (unit >= n_units) return;
  const uint32_t stream = __builtin_amdgcn_readfirstlane(unit / tp.n_mtiles);
  const uint32_t mt = __builtin_amdgcn_readfirstlane(unit % tp.n_mtiles);
  const uint32_t kvh = __builtin_amdgcn_readfirstlane(stream / tp.n_splits);
  const uint32_t split = __builtin_amdgcn_readfirstlane(stream % tp.n_splits);

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t g2 = lane >> 5, l32 = lane & 31u;

  const uint32_t rows_total = tp.ntok * p.group;
  const uint32_t row0 = mt * kBlockM;
  const uint32_t r = row0 + wave * 32u + l32;
  const bool row_ok = r < rows_total;
  const uint32_t tok_l = row_ok ? r / p.group : 0u;           // row within this pass
  const uint32_t tok = tp.tok0 + tok_l;
  const uint32_t qh = kvh * p.group + (row_ok ? r % p.group : 0u);

  // key tiles some row of this row tile can see
  uint32_t lo_min, hi_max;
  {
    const uint32_t last_row = min(row0 + kBlockM, rows_total) - 1u;
    const uint32_t tok_a = tp.tok0 + row0 / p.group, tok_b = tp.tok0 + last_row / p.group;
    const RowBounds ba = row_bounds(p, tok_a), bb = row_bounds(p, tok_b);
    lo_min = min(ba.lo, bb.lo);
    hi_max = max(ba.hi, bb.hi);
    if (tok_a < p.causal_rows && tok_b >= p.causal_rows) {
      const RowBounds bc = row_bounds(p, p.causal_rows - 1u), bd = row_bounds(p, p.causal_rows);
      lo_min = min(lo_min, min(bc.lo, bd.lo));
      hi_max = max(hi_max, max(bc.hi, bd.hi));
    }
    if (tok_a < p.causal_rows && p.extra_lo < p.t_all) hi_max = p.t_all;
    lo_min = __builtin_amdgcn_readfirstlane(lo_min);
    hi_max = __builtin_amdgcn_readfirstlane(hi_max);
  }
  const uint32_t mt_begin = max(lo_min / kBlockN, tp.tile_first);
  const uint32_t mt_end = max(min((hi_max + kBlockN - 1) / kBlockN, tp.tile_end), mt_begin);
  const uint32_t per_split = (mt_end - mt_begin + tp.n_splits - 1u) / tp.n_splits;
  const uint32_t tb = __builtin_amdgcn_readfirstlane(min(mt_begin + split * per_split, mt_end));
  const uint32_t te = __builtin_amdgcn_readfirstlane(min(tb + per_split, mt_end));
  if (te <= tb) return;

  // Q fragments: B operand of S^T = K.Q^T, lane = row, 8 consecutive d per step
  u32x4 qf[NSTEP];
  {
    const size_t qoff = ((size_t)tok * p.hq + qh) * D + 8u * g2;
    const uint16_t* qp = (const uint16_t*)p.q + qoff;
    if (F16 && p.q_is_bf16) {
#pragma unroll
      for (int s = 0; s < NSTEP; ++s) {
        u32x4 raw = row_ok ? *(const u32x4*)(qp + 16 * s) : u32x4{0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 4; ++e)
          qf[s][e] = pack2<true>(__uint_as_float(raw[e] << 16), __uint_as_float(raw[e] & 0xffff0000u));
      }
    } else {
#pragma unroll
      for (int s = 0; s < NSTEP; ++s) qf[s] = row_ok ? *(const u32x4*)(qp + 16 * s) : u32x4{0, 0, 0, 0};
    }
  }

  const char* kbase = (const char*)p.k + (int64_t)kvh * p.k_head_stride * 2;
  const int64_t kstride_b = p.k_tok_stride * 2;
  const uint32_t k_lane_off = l32 * L::K_STRIDE + (L::PAD ? g2 * 16u : 0u);
  const uint32_t k_swz = L::swz_k(l32);
  const uint32_t t_last = (te - 1u) * kBlockN;
  // loads for a tile past the last one fetch the last tile again into a buffer nobody reads, so
  // that every iteration issues the same number of loads and the wait counts stay fixed
  auto issue_k = [&](uint32_t j) {
    lds_char* buf = (lds_char*)(smem + ((j - tb) % NB) * L::K_BYTES);
    const TileLoad tl = make_tile_load<D, false, false>(kbase, kstride_b, min(j * kBlockN, t_last), 0u, p.t_all,
                                                        p.ring_mask, buf, wave, lane);
    issue_tile<D, false>(tl, wave, lane);
  };
  float* const srow = tp.s_plane + ((size_t)qh * tp.ntok + tok_l) * tp.t_pad;

#pragma unroll
  for (int i = 0; i < PF; ++i) issue_k(tb + i);
  for (uint32_t j = tb; j < te; ++j) {
    // this wave's loads of K(j) have landed (the PF-1 tiles behind it may still be in flight);
    // after the barrier everybody's have, and everybody is done reading K(j-1), whose buffer
    // takes K(j+PF)
    wait_loads_then_barrier<(PF - 1) * NLD>();
    issue_k(j + PF);
    lds_char* const kb = (lds_char*)(smem + ((j - tb) % NB) * L::K_BYTES);
    f32x16 s;
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
    for (int st = 0; st < NSTEP; ++st) {
      u32x4 a;
      if constexpr (L::PAD) {
        a = *(lds_u32x4*)(kb + k_lane_off + 32 * st);
      } else {
        const uint32_t c = (uint32_t)(2 * st) + g2;
        a = *(lds_u32x4*)(kb + k_lane_off + ((c ^ k_swz) << 4));
      }
      s = mfma16<F16>(a, qf[st], s);
    }
    // register e of the block is key t0 + 8 (e >> 2) + 4 g2 + (e & 3) of row l32
    if (row_ok) {
      float* dst = srow + j * kBlockN + 4u * g2;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *(f32x4*)(dst + 8 * q4) = f32x4{s[4 * q4] * tp.scale, s[4 * q4 + 1] * tp.scale, s[4 * q4 + 2] * tp.scale,
                                         s[4 * q4 + 3] * tp.scale};
    }
  }
  wait_vmem_all();   // no direct-to-LDS load may outlive the workgroup's LDS
}

// ---------------------------------------------------------------------------------------------
// select + softmax + gathered P.V
// ---------------------------------------------------------------------------------------------

// order-preserving integer image of a score (larger float <-> larger key); NaN sorts lowest
__device__ __forceinline__ uint32_t score_key(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0u;
  return (u & 0x80000000u) ? ~u : (u ^ 0x80000000u);
}

// number of keys row bounds b let through
__device__ __forceinline__ uint32_t visible_count(const RowBounds& b, uint32_t t_all) {
  const uint32_t hi = min(b.hi, t_all);
  const uint32_t len_a = hi > b.lo ? hi - b.lo : 0u;
  if (b.extra >= t_all) return len_a;
  if (len_a == 0u) return t_all - b.extra;
  if (b.extra <= b.lo) return t_all - b.extra;
  if (b.extra < hi) return t_all - b.lo;
  return len_a + (t_all - b.extra);
}

struct SelectShared {
  uint32_t hist[kMaxBins];
  uint32_t tot[256];
  uint32_t res[4];              // chosen bin, entries above it, entries in it
  uint32_t n_sel, n_cand, pad0, pad1;
  uint32_t cand_key[kCandCap];
  uint32_t cand_t[kCandCap];
  float sel_s[kTopkMaxK];
  uint32_t sel_t[kTopkMaxK];
};

// From hist[0 .. nbins): the bin that holds the `remaining`-th largest entry, counting from the
// top bin down.  Leaves {bin, entries in higher bins, entries in the bin} in sh.res.  All 256
// threads call it; it contains barriers.
__device__ __forceinline__ void pick_bin(SelectShared& sh, uint32_t nbins, uint32_t remaining, uint32_t tid) {
  const uint32_t per = nbins >> 8;          // bins per thread: 8 or 4
  uint32_t c[8];
  uint32_t sum = 0;
#pragma unroll
  for (uint32_t i = 0; i < 8; ++i) {
    c[i] = i < per ? sh.hist[tid * per + i] : 0u;
    sum += c[i];
  }
  sh.tot[tid] = sum;
  __syncthreads();
  uint32_t above = 0;                        // entries in the bins of higher threads
  for (uint32_t t = tid + 1; t < 256u; ++t) above += sh.tot[t];
  if (above < remaining && remaining <= above + sum) {
    uint32_t run = above;
#pragma unroll
    for (int i = 7; i >= 0; --i) {
      if ((uint32_t)i < per) {
        if (run < remaining && remaining <= run + c[i]) {
          sh.res[0] = tid * per + (uint32_t)i;
          sh.res[1] = run;
          sh.res[2] = c[i];
        }
        run += c[i];
      }
    }
  }
  __syncthreads();
}

template <int D, bool F16>
__global__ void __launch_bounds__(256) topk_select_kernel(const TopkParams tp) {
  const AttnParams& p = tp.a;
  __shared__ SelectShared sh;
  static_assert(4 * D * sizeof(float) <= sizeof(sh.cand_key), "the P.V partial sums reuse the candidate list");
  float (*const red)[D] = (float (*)[D])sh.cand_key;
  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, wave = tid >> 6;
  const uint32_t tok_l = blockIdx.x, qh = blockIdx.y;
  const uint32_t tok = tp.tok0 + tok_l;
  const uint32_t kvh = qh / p.group;
  const RowBounds rb = row_bounds(p, tok);
  const uint32_t n_valid = visible_count(rb, p.t_all);

  // keys kept for this row (attention_topk.metal:160-182)
  uint32_t k_req;
  if (tp.k_cfg[1] != 0u) {
    const uint32_t gran = max(tp.k_cfg[0], 1u);
    const uint32_t t_equiv = tok < p.causal_rows ? ((n_valid + gran - 1u) / gran) * gran : n_valid;
    k_req = min(max(t_equiv / tp.k_cfg[1], tp.k_cfg[2]), tp.k_cfg[3]);
  } else {
    k_req = max(tp.k_cfg[0], 1u);
  }
  const uint32_t k = min(min(k_req, n_valid), (uint32_t)kTopkMaxK);

  const size_t out_off = ((size_t)tok * p.hq + qh) * D;
  if (k == 0u) {   // a row that sees no key stores zeros, like the dense path
    for (uint32_t d = tid; d < (uint32_t)D; d += 256u) {
      if (p.out_dtype == 2u) ((float*)p.out)[out_off + d] = 0.f;
      else ((uint16_t*)p.out)[out_off + d] = 0;
    }
    return;
  }

  const float* srow = tp.s_plane + ((size_t)qh * tp.ntok + tok_l) * tp.t_pad;
  // positions to scan: the hull of the visible set, widened to whole float4s
  const uint32_t hull_lo = (rb.extra < p.t_all ? min(rb.lo, rb.extra) : rb.lo) & ~3u;
  const uint32_t hull_hi = rb.extra < p.t_all ? p.t_all : min(rb.hi, p.t_all);

  if (tid == 0) {
    sh.n_sel = 0;
    sh.n_cand = 0;
    sh.res[0] = sh.res[1] = sh.res[2] = 0;
  }

  // ---- levels over the score row in memory, until the class of the k-th score fits the list ----
  uint32_t prefix = 0, pbits = 0, remaining = k, class_count = n_valid;
  int level = 0;
  for (; level < 3 && class_count > (uint32_t)kCandCap; ++level) {
    const uint32_t nbins = 1u << digit_bits(level);
    for (uint32_t b = tid; b < nbins; b += 256u) sh.hist[b] = 0;
    __syncthreads();
    for (uint32_t t4 = hull_lo + 4u * tid; t4 < hull_hi; t4 += 1024u) {
      const f32x4 v = *(const f32x4*)(srow + t4);
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t t = t4 + i;
        if (key_visible(rb, t, p.t_all)) {
          const uint32_t key = score_key(v[i]);
          if (pbits == 0u || (key >> (32u - pbits)) == prefix)
            atomicAdd(&sh.hist[(key >> digit_shift(level)) & (nbins - 1u)], 1u);
        }
      }
    }
    __syncthreads();
    pick_bin(sh, nbins, remaining, tid);
    remaining -= sh.res[1];
    prefix = (prefix << digit_bits(level)) | sh.res[0];
    pbits += digit_bits(level);
    class_count = sh.res[2];
    __syncthreads();
  }

  if (class_count > (uint32_t)kCandCap) {
    // More than a list's worth of bit-identical scores at the threshold (a degenerate row, e.g.
    // an all-zero query).  Keys above go in as they come; of the ties the first `remaining` by
    // position are taken by one wave walking the row in order.
    for (uint32_t t4 = hull_lo + 4u * tid; t4 < hull_hi; t4 += 1024u) {
      const f32x4 v = *(const f32x4*)(srow + t4);
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t t = t4 + i;
        if (key_visible(rb, t, p.t_all) && score_key(v[i]) > prefix) {
          const uint32_t slot = atomicAdd(&sh.n_sel, 1u);
          if (slot < (uint32_t)kTopkMaxK) {
            sh.sel_s[slot] = v[i];
            sh.sel_t[slot] = t;
          }
        }
      }
    }
    __syncthreads();
    if (wave == 0) {
      const uint32_t first = k - remaining;
      uint32_t taken = 0;
      for (uint32_t t0 = hull_lo; t0 < hull_hi && taken < remaining; t0 += 64u) {
        const uint32_t t = t0 + lane;
        float sv = 0.f;
        bool tie = false;
        if (t < hull_hi && key_visible(rb, t, p.t_all)) {
          sv = srow[t];
          tie = score_key(sv) == prefix;
        }
        const unsigned long long m = __builtin_amdgcn_ballot_w64(tie);
        const uint32_t rank = taken + __builtin_popcountll(m & ((1ull << lane) - 1ull));
        if (tie && rank < remaining && first + rank < (uint32_t)kTopkMaxK) {
          sh.sel_s[first + rank] = sv;
          sh.sel_t[first + rank] = t;
        }
        taken += __builtin_popcountll(m);
      }
    }
    __syncthreads();
  } else {
    // ---- one pass: keys above the class go straight to the kept list, the class to the candidates ----
    for (uint32_t t4 = hull_lo + 4u * tid; t4 < hull_hi; t4 += 1024u) {
      const f32x4 v = *(const f32x4*)(srow + t4);
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t t = t4 + i;
        if (key_visible(rb, t, p.t_all)) {
          const uint32_t key = score_key(v[i]);
          const uint32_t hi = pbits ? key >> (32u - pbits) : 0u;
          if (hi > prefix) {
            const uint32_t slot = atomicAdd(&sh.n_sel, 1u);
            if (slot < (uint32_t)kTopkMaxK) {
              sh.sel_s[slot] = v[i];
              sh.sel_t[slot] = t;
            }
          } else if (hi == prefix) {
            const uint32_t slot = atomicAdd(&sh.n_cand, 1u);
            if (slot < (uint32_t)kCandCap) {
              sh.cand_key[slot] = key;
              sh.cand_t[slot] = t;
            }
          }
        }
      }
    }
    __syncthreads();
    const uint32_t n_cand = min(sh.n_cand, (uint32_t)kCandCap);

    // ---- remaining levels over the candidate list ----
    for (; level < 3; ++level) {
      const uint32_t nbins = 1u << digit_bits(level);
      for (uint32_t b = tid; b < nbins; b += 256u) sh.hist[b] = 0;
      __syncthreads();
      for (uint32_t i = tid; i < n_cand; i += 256u) {
        const uint32_t key = sh.cand_key[i];
        if (pbits == 0u || (key >> (32u - pbits)) == prefix)
          atomicAdd(&sh.hist[(key >> digit_shift(level)) & (nbins - 1u)], 1u);
      }
      __syncthreads();
      pick_bin(sh, nbins, remaining, tid);
      remaining -= sh.res[1];
      prefix = (prefix << digit_bits(level)) | sh.res[0];
      pbits += digit_bits(level);
      class_count = sh.res[2];
      __syncthreads();
    }
    // prefix is now the k-th largest key; `remaining` of the class_count keys equal to it are kept

    // ---- equal scores: the lower positions win.  Threshold on position by the same select ----
    uint32_t t_key_min = 0u;   // ties with ~t >= t_key_min are kept
    if (class_count > remaining) {
      uint32_t tp_prefix = 0, tp_bits = 0, tp_rem = remaining;
      for (int lv = 0; lv < 3; ++lv) {
        const uint32_t nbins = 1u << digit_bits(lv);
        for (uint32_t b = tid; b < nbins; b += 256u) sh.hist[b] = 0;
        __syncthreads();
        for (uint32_t i = tid; i < n_cand; i += 256u) {
          if (sh.cand_key[i] == prefix) {
            const uint32_t key2 = ~sh.cand_t[i];
            if (tp_bits == 0u || (key2 >> (32u - tp_bits)) == tp_prefix)
              atomicAdd(&sh.hist[(key2 >> digit_shift(lv)) & (nbins - 1u)], 1u);
          }
        }
        __syncthreads();
        pick_bin(sh, nbins, tp_rem, tid);
        tp_rem -= sh.res[1];
        tp_prefix = (tp_prefix << digit_bits(lv)) | sh.res[0];
        tp_bits += digit_bits(lv);
        __syncthreads();
      }
      t_key_min = tp_prefix;
    }
    for (uint32_t i = tid; i < n_cand; i += 256u) {
      const uint32_t key = sh.cand_key[i];
      const uint32_t t = sh.cand_t[i];
      if (key > prefix || (key == prefix && ~t >= t_key_min)) {
        const uint32_t slot = atomicAdd(&sh.n_sel, 1u);
        if (slot < (uint32_t)kTopkMaxK) {
          sh.sel_s[slot] = srow[t];
          sh.sel_t[slot] = t;
        }
      }
    }
    __syncthreads();
  }

  // ---- sort the kept keys by position (bitonic, padded with +inf positions) ----
  uint32_t npow = 1;
  while (npow < k) npow <<= 1;
  for (uint32_t i = k + tid; i < npow; i += 256u) {
    sh.sel_t[i] = 0xffffffffu;
    sh.sel_s[i] = -INFINITY;
  }
  __syncthreads();
  for (uint32_t size = 2; size <= npow; size <<= 1) {
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      for (uint32_t i = tid; i < (npow >> 1); i += 256u) {
        const uint32_t lo = 2u * i - (i & (stride - 1u));
        const uint32_t hi = lo + stride;
        const bool up = (lo & size) == 0u;
        const uint32_t a = sh.sel_t[lo], b = sh.sel_t[hi];
        if ((a > b) == up) {
          sh.sel_t[lo] = b;
          sh.sel_t[hi] = a;
          const float fa = sh.sel_s[lo];
          sh.sel_s[lo] = sh.sel_s[hi];
          sh.sel_s[hi] = fa;
        }
      }
      __syncthreads();
    }
  }

  // ---- softmax over the kept scores (cpu.rs:95-104) ----
  float* const fred = (float*)sh.hist;   // histogram storage is free now
  float m = -INFINITY;
  for (uint32_t j = tid; j < k; j += 256u) m = fmaxf(m, sh.sel_s[j]);
  fred[tid] = m;
  __syncthreads();
  for (uint32_t w = 128; w > 0; w >>= 1) {
    if (tid < w) fred[tid] = fmaxf(fred[tid], fred[tid + w]);
    __syncthreads();
  }
  const float mmax = fred[0];
  __syncthreads();
  float l = 0.f;
  for (uint32_t j = tid; j < k; j += 256u) {
    const float e = expf(sh.sel_s[j] - mmax);
    sh.sel_s[j] = e;
    l += e;
  }
  fred[tid] = l;
  __syncthreads();
  for (uint32_t w = 128; w > 0; w >>= 1) {
    if (tid < w) fred[tid] += fred[tid + w];
    __syncthreads();
  }
  const float lsum = fred[0];
  const float inv = lsum > 0.f ? 1.f / lsum : 0.f;

  // ---- gathered P.V: wave w takes kept keys w, w+4, ...; a lane owns PER consecutive d ----
  constexpr int PER = D >= 64 ? D / 64 : 1;
  const bool lane_on = lane * PER < (uint32_t)D;
  float acc[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) acc[i] = 0.f;
  const char* vbase = (const char*)p.v + (int64_t)kvh * p.v_head_stride * 2 + (size_t)lane * PER * 2;
  const int64_t vstride_b = p.v_tok_stride * 2;
  for (uint32_t j = wave; j < k; j += 4u) {
    const float pj = sh.sel_s[j] * inv;
    const uint32_t tj = min(sh.sel_t[j], p.t_all - 1u);   // (kept positions are < t_all by construction)
    const uint16_t* vp = (const uint16_t*)(vbase + (int64_t)kv_slot(p.ring_mask, tj) * vstride_b);
    if (lane_on) {
      uint16_t raw[PER];
      if constexpr (PER == 8) {
        const u32x4 x = *(const u32x4*)vp;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          raw[2 * i] = (uint16_t)(x[i] & 0xffffu);
          raw[2 * i + 1] = (uint16_t)(x[i] >> 16);
        }
      } else if constexpr (PER == 4) {
        const u32x2 x = *(const u32x2*)vp;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          raw[2 * i] = (uint16_t)(x[i] & 0xffffu);
          raw[2 * i + 1] = (uint16_t)(x[i] >> 16);
        }
      } else if constexpr (PER == 2) {
        const uint32_t x = *(const uint32_t*)vp;
        raw[0] = (uint16_t)(x & 0xffffu);
        raw[1] = (uint16_t)(x >> 16);
      } else {
        raw[0] = *vp;
      }
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const float v = F16 ? (float)__builtin_bit_cast(_Float16, raw[i]) : bf16_bits_to_f32(raw[i]);
        acc[i] = __builtin_fmaf(pj, v, acc[i]);
      }
    }
  }
  if (lane_on) {
#pragma unroll
    for (int i = 0; i < PER; ++i) red[wave][lane * PER + i] = acc[i];
  }
  __syncthreads();
  for (uint32_t d = tid; d < (uint32_t)D; d += 256u) {
    const float o = ((red[0][d] + red[1][d]) + red[2][d]) + red[3][d];
    if (p.out_dtype == 2u) ((float*)p.out)[out_off + d] = o;
    else ((uint16_t*)p.out)[out_off + d] = f32_to_bf16_bits(o, p.out_trunc != 0u);
  }
}

template <int D, bool F16>
hipError_t launch_pair(const TopkParams& tp, hipStream_t s) {
  const uint32_t n_units = tp.a.hkv * tp.n_splits * tp.n_mtiles;
  const uint32_t grid = ((n_units + 7u) / 8u) * 8u;
  hipLaunchKernelGGL((topk_scores_kernel<D, F16>), dim3(grid), dim3(256), 0, s, tp);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((topk_select_kernel<D, F16>), dim3(tp.ntok, tp.a.hq), dim3(256), 0, s, tp);
  return hipGetLastError();
}

template <bool F16>
hipError_t launch_by_dim(const TopkParams& tp, uint32_t head_dim, hipStream_t s) {
  switch (head_dim) {
    case 32: return launch_pair<32, F16>(tp, s);
    case 64: return launch_pair<64, F16>(tp, s);
    case 128: return launch_pair<128, F16>(tp, s);
    case 256: return launch_pair<256, F16>(tp, s);
    case 512: return launch_pair<512, F16>(tp, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

hipError_t launch_attn_topk(const TopkParams& tp, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s) {
  return kv_dtype == 1u ? launch_by_dim<true>(tp, head_dim, s) : launch_by_dim<false>(tp, head_dim, s);
}

}  // namespace dg
