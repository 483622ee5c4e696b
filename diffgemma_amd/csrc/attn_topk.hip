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

constexpr int kCandCap = 2048;     // LDS candidate list of the select kernel (sized for 4 workgroups per CU)

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

  // Q fragments: lane = row, 8 consecutive d per step
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
  auto k_desc = [&](uint32_t j) {
    lds_char* buf = (lds_char*)(smem + ((j - tb) % NB) * L::K_BYTES);
    return make_tile_load<D, false, false>(kbase, kstride_b, min(j * kBlockN, t_last), 0u, p.t_all, p.ring_mask, buf,
                                           wave, lane);
  };
  auto issue_k = [&](uint32_t j) { issue_tile<D, false>(k_desc(j), wave, lane); };
  // The product is taken as S = Q.K^T (A = Q, B = K): the output lane is then the key and
  // register e of the block is query row 8 (e >> 2) + 4 g2 + (e & 3) of this wave's 32, so one
  // store instruction writes 32 consecutive keys of two rows: whole 128-byte lines.  (With the
  // operands the other way round every store scatters 32-byte pieces over 32 rows and the
  // kernel is bound by the write path.)  Where each of the 16 rows lives, and whether it exists:
  uint32_t row_off[16];      // byte offset of this lane's key column in the row, in the first key tile
  uint32_t row_mask = 0;
  const bool full_tile = row0 + kBlockM <= rows_total;      // (the same in every lane)
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const uint32_t rr = row0 + wave * 32u + 8u * (e >> 2) + 4u * g2 + (e & 3);
    const bool ok = rr < rows_total;
    const uint32_t tl = ok ? rr / p.group : 0u;
    const uint32_t hh = kvh * p.group + (ok ? rr % p.group : 0u);
    row_off[e] = ((hh * tp.ntok + tl) * tp.t_pad + l32) * 4u;
    row_mask |= ok ? 1u << e : 0u;
  }
#pragma unroll
  for (int i = 0; i < PF; ++i) issue_k(tb + i);
  // lane l32 holds key t0 + l32 of sixteen rows; element e of a tile's scores goes to
  // (uniform tile base) + (per-lane 32-bit offset)
  auto store_elem = [&](auto e_c, const f32x16& sc, uint32_t tile) {
    constexpr int e = decltype(e_c)::value;
    char* const base = (char*)tp.s_plane + (size_t)tile * (kBlockN * sizeof(float));
    if (full_tile || (row_mask & (1u << e))) *(float*)(base + row_off[e]) = sc[e] * tp.scale;
  };
  auto store_tile = [&](const f32x16& sc, uint32_t tile) {
    static_for<0, 16>([&](auto e_c) { store_elem(e_c, sc, tile); });
  };
  f32x16 s_prev;
#pragma unroll
  for (int e = 0; e < 16; ++e) s_prev[e] = 0.f;
  for (uint32_t j = tb; j < te; ++j) {
    // this wave's loads of K(j) have landed (the PF-1 tiles behind it may still be in flight);
    // after the barrier everybody's have, and everybody is done reading K(j-1), whose buffer
    // takes K(j+PF).  The scores of tile j-1 are stored only now, a tile late, between the
    // first half of this tile's MFMAs: stores count in the same counter as the loads, and issued
    // right before the wait they would have to drain first; issued here they are at least half
    // a tile old at the next wait, and their address arithmetic hides behind the matrix pipe.
    wait_loads_then_barrier<(PF - 1) * NLD>();
    const bool have_prev = j > tb;
    // (the loads of K(j+PF) are issued between the MFMAs below: back to back each of them holds
    // the wave's issue slot for about two MFMAs' worth of cycles)
    const TileLoad tl_next = k_desc(j + PF);
    lds_char* const kb = (lds_char*)(smem + ((j - tb) % NB) * L::K_BYTES);
    f32x16 s;
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.f;
    // K fragments in chunks of CH: the reads of chunk c+1 are issued before the MFMAs of chunk c
    // (left to itself the compiler reads two fragments, waits, multiplies, and the LDS latency
    // is paid sixteen times per tile)
    constexpr int CH = NSTEP < 8 ? NSTEP : 8;
    constexpr int NCHUNK = NSTEP / CH;
    constexpr int LPC = (NLD + NCHUNK - 1) / NCHUNK;      // tile loads issued per chunk
    constexpr int LGAP = CH / LPC;                         // MFMAs between two of them
    static_assert(LPC * NCHUNK >= NLD && LPC <= CH, "tile loads must fit between the MFMAs");
    constexpr int SHALF = NSTEP / 2 > 0 ? NSTEP / 2 : 1;   // MFMAs that carry stores of the previous tile
    constexpr int SPM = (16 + SHALF - 1) / SHALF;          // stores behind each of them
    u32x4 fr[2][CH];
    auto read_chunk = [&](int c, u32x4 (&dst)[CH]) {
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const int st = c * CH + i;
        if constexpr (L::PAD) {
          dst[i] = *(lds_u32x4*)(kb + k_lane_off + 32 * st);
        } else {
          const uint32_t cc = (uint32_t)(2 * st) + g2;
          dst[i] = *(lds_u32x4*)(kb + k_lane_off + ((cc ^ k_swz) << 4));
        }
      }
    };
    read_chunk(0, fr[0]);
    static_for<0, NCHUNK>([&](auto c_c) {
      constexpr int c = decltype(c_c)::value;
      if constexpr (c + 1 < NCHUNK) read_chunk(c + 1, fr[(c + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      static_for<0, CH>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        s = mfma16<F16>(qf[c * CH + i], fr[c & 1][i], s);
        if constexpr (i % LGAP == LGAP / 2 && c * LPC + i / LGAP < NLD) {
          issue_tile_part<D, false, c * LPC + i / LGAP>(tl_next, wave, lane);
          __builtin_amdgcn_sched_barrier(0);
        }
        constexpr int m = c * CH + i;                 // MFMA index within the tile
        if constexpr (m < SHALF) {
          if (have_prev) static_for<m * SPM, (m + 1) * SPM < 16 ? (m + 1) * SPM : 16>([&](auto e_c) { store_elem(e_c, s_prev, j - 1u); });
          __builtin_amdgcn_sched_barrier(0);
        }
      });
      __builtin_amdgcn_sched_barrier(0);
    });
    s_prev = s;
  }
  store_tile(s_prev, te - 1u);
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

// the score a key stands for (inverse of score_key for every non-NaN score)
__device__ __forceinline__ float key_score(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? key ^ 0x80000000u : ~key);
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
  const uint32_t lane = tid & 63u, wave = tid >> 6;
  uint32_t c[8];
  uint32_t sum = 0;
#pragma unroll
  for (uint32_t i = 0; i < 8; ++i) {
    c[i] = i < per ? sh.hist[tid * per + i] : 0u;
    sum += c[i];
  }
  // entries in the bins of higher threads: suffix sum over the lanes of the wave, then the
  // totals of the higher waves
  uint32_t incl = sum;
#pragma unroll
  for (uint32_t off = 1; off < 64u; off <<= 1) {
    const uint32_t v = __shfl_down(incl, off, 64);
    if (lane + off < 64u) incl += v;
  }
  if (lane == 0) sh.tot[wave] = incl;
  __syncthreads();
  uint32_t above = incl - sum;
  for (uint32_t w = wave + 1; w < 4u; ++w) above += sh.tot[w];
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

// The `need`-th largest of the keys key_of(i) yields for i in [0, n) (key_of returns false for
// entries that do not take part), by three histogram levels over LDS.  Returns the key; *n_equal
// = entries equal to it, *take_equal = how many of those belong to the `need` largest.  All 256
// threads call it with the same arguments; needs 1 <= need <= number of participating entries.
template <typename KeyOf>
__device__ __forceinline__ uint32_t lds_kth_largest(SelectShared& sh, uint32_t n, uint32_t need, uint32_t tid,
                                                    KeyOf&& key_of, uint32_t* take_equal, uint32_t* n_equal) {
  uint32_t prefix = 0, pbits = 0, remaining = need, cls = 0;
  for (int lv = 0; lv < 3; ++lv) {
    const uint32_t nbins = 1u << digit_bits(lv);
    for (uint32_t b = tid; b < nbins; b += 256u) sh.hist[b] = 0;
    __syncthreads();
    for (uint32_t i = tid; i < n; i += 256u) {
      uint32_t key;
      if (key_of(i, key) && (pbits == 0u || (key >> (32u - pbits)) == prefix))
        atomicAdd(&sh.hist[(key >> digit_shift(lv)) & (nbins - 1u)], 1u);
    }
    __syncthreads();
    pick_bin(sh, nbins, remaining, tid);
    remaining -= sh.res[1];
    prefix = (prefix << digit_bits(lv)) | sh.res[0];
    pbits += digit_bits(lv);
    cls = sh.res[2];
    __syncthreads();
  }
  *take_equal = remaining;
  *n_equal = cls;
  return prefix;
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

  // f(position, score) for every visible key of the row; each thread takes one float4 out of
  // every 256 and has four of them in flight.  The plane is read once: non-temporal loads (here and
  // for the sample above), so that 135 MB of scores per block do not push the V rows, which every
  // row of a KV group gathers from, out of the L2s (whole call 0.715 -> 0.664 ms)
  auto scan_row = [&](auto&& f) {
    for (uint32_t t4 = hull_lo + 4u * tid; t4 < hull_hi; t4 += 4096u) {
      f32x4 v[4];
#pragma unroll
      for (uint32_t u = 0; u < 4; ++u) {
        const uint32_t a = t4 + 1024u * u;
        v[u] = a < hull_hi ? __builtin_nontemporal_load((const f32x4*)(srow + a)) : f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (uint32_t u = 0; u < 4; ++u) {
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
          const uint32_t t = t4 + 1024u * u + i;
          if (t < hull_hi && key_visible(rb, t, p.t_all)) f(t, v[u][i]);
        }
      }
    }
  };
  if (tid == 0) {
    sh.n_sel = 0;
    sh.n_cand = 0;
    sh.res[0] = sh.res[1] = sh.res[2] = 0;
  }

  uint32_t prefix = 0, pbits = 0, remaining = k, class_count = n_valid;
  int level = 0;
  bool have_cand = false;   // the candidate list already holds every key at or above a sampled threshold

  // ---- long rows: cut at a threshold taken from a sample, so that the row is read once ----
  // About 2048 keys at an even stride give the key tau below which ~2.5 k keys are expected;
  // one pass collects everything >= tau.  If that is at least k and fits the list, the exact
  // k-th key is found in LDS; otherwise (an unlucky or clustered sample) the exact histogram
  // levels below run instead.
  if (n_valid > (uint32_t)kCandCap) {
    const uint32_t stride = max(1u, (hull_hi - hull_lo + 2047u) / 2048u);
    const uint32_t m = (hull_hi - hull_lo + stride - 1u) / stride;     // sample slots, at most 2048
    {
      float sv[8];
#pragma unroll
      for (uint32_t u = 0; u < 8; ++u) {      // m <= 2048: eight samples per thread, all in flight
        const uint32_t i = tid + 256u * u;
        sv[u] = i < m ? __builtin_nontemporal_load(srow + hull_lo + i * stride) : 0.f;
      }
#pragma unroll
      for (uint32_t u = 0; u < 8; ++u) {
        const uint32_t i = tid + 256u * u;
        // (an invisible position takes part as the lowest key, which cannot reach the top ranks asked for)
        if (i < m) sh.cand_key[i] = key_visible(rb, hull_lo + i * stride, p.t_all) ? score_key(sv[u]) : 0u;
      }
    }
    __syncthreads();
    if (m > 0u) {
      // aim at ~2.5 k keys at or above tau, but never beyond 3/4 of the list
      const uint64_t want = min<uint64_t>(5ull * k / 2ull, 3ull * kCandCap / 4ull);
      const uint32_t r = min(m, (uint32_t)((want * m + n_valid - 1ull) / n_valid) + 8u);
      uint32_t te, ne;
      const uint32_t tau = lds_kth_largest(
          sh, m, r, tid, [&](uint32_t i, uint32_t& key) { key = sh.cand_key[i]; return true; }, &te, &ne);
      scan_row([&](uint32_t t, float sv) {
        const uint32_t key = score_key(sv);
        if (key >= tau) {
          const uint32_t slot = atomicAdd(&sh.n_cand, 1u);
          if (slot < (uint32_t)kCandCap) {
            sh.cand_key[slot] = key;
            sh.cand_t[slot] = t;
          }
        }
      });
      __syncthreads();
      const uint32_t got = sh.n_cand;
      have_cand = got >= k && got <= (uint32_t)kCandCap;
      if (have_cand) class_count = got;
      __syncthreads();
      if (!have_cand && tid == 0) sh.n_cand = 0;
    }
    __syncthreads();
  }

  // ---- exact levels over the score row in memory, until the class of the k-th score fits the list ----
  for (; !have_cand && level < 3 && class_count > (uint32_t)kCandCap; ++level) {
    const uint32_t nbins = 1u << digit_bits(level);
    for (uint32_t b = tid; b < nbins; b += 256u) sh.hist[b] = 0;
    __syncthreads();
    scan_row([&](uint32_t, float sv) {
      const uint32_t key = score_key(sv);
      if (pbits == 0u || (key >> (32u - pbits)) == prefix)
        atomicAdd(&sh.hist[(key >> digit_shift(level)) & (nbins - 1u)], 1u);
    });
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
    scan_row([&](uint32_t t, float sv) {
      if (score_key(sv) > prefix) {
        const uint32_t slot = atomicAdd(&sh.n_sel, 1u);
        if (slot < (uint32_t)kTopkMaxK) {
          sh.sel_s[slot] = sv;
          sh.sel_t[slot] = t;
        }
      }
    });
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
    if (!have_cand) {
      // ---- one pass: keys above the class go straight to the kept list, the class to the candidates ----
      scan_row([&](uint32_t t, float sv) {
        const uint32_t key = score_key(sv);
        const uint32_t hi = pbits ? key >> (32u - pbits) : 0u;
        if (hi > prefix) {
          const uint32_t slot = atomicAdd(&sh.n_sel, 1u);
          if (slot < (uint32_t)kTopkMaxK) {
            sh.sel_s[slot] = sv;
            sh.sel_t[slot] = t;
          }
        } else if (hi == prefix) {
          const uint32_t slot = atomicAdd(&sh.n_cand, 1u);
          if (slot < (uint32_t)kCandCap) {
            sh.cand_key[slot] = key;
            sh.cand_t[slot] = t;
          }
        }
      });
      __syncthreads();
    }
    const uint32_t n_cand = min(sh.n_cand, (uint32_t)kCandCap);

    // ---- the k-th key among the candidates: the levels not yet done, over the list ----
    uint32_t thr = prefix, take_eq = remaining, n_eq = class_count;
    if (level < 3) {
      // (the list holds exactly the keys whose leading pbits bits equal prefix: rebuild the full
      // key of the threshold from the remaining levels)
      uint32_t lp = prefix, lb = pbits, rem = remaining, cls = class_count;
      for (int lv = level; lv < 3; ++lv) {
        const uint32_t nbins = 1u << digit_bits(lv);
        for (uint32_t b = tid; b < nbins; b += 256u) sh.hist[b] = 0;
        __syncthreads();
        for (uint32_t i = tid; i < n_cand; i += 256u) {
          const uint32_t key = sh.cand_key[i];
          if (lb == 0u || (key >> (32u - lb)) == lp) atomicAdd(&sh.hist[(key >> digit_shift(lv)) & (nbins - 1u)], 1u);
        }
        __syncthreads();
        pick_bin(sh, nbins, rem, tid);
        rem -= sh.res[1];
        lp = (lp << digit_bits(lv)) | sh.res[0];
        lb += digit_bits(lv);
        cls = sh.res[2];
        __syncthreads();
      }
      thr = lp;
      take_eq = rem;
      n_eq = cls;
    }
    // thr is the k-th largest key; take_eq of the n_eq keys equal to it are kept

    // ---- equal scores: the lower positions win.  Threshold on position by the same select ----
    uint32_t t_key_min = 0u;   // ties with ~t >= t_key_min are kept
    if (n_eq > take_eq) {
      uint32_t te, ne;
      t_key_min = lds_kth_largest(
          sh, n_cand, take_eq, tid,
          [&](uint32_t i, uint32_t& key) {
            key = ~sh.cand_t[i];
            return sh.cand_key[i] == thr;
          },
          &te, &ne);
    }
    for (uint32_t i = tid; i < n_cand; i += 256u) {
      const uint32_t key = sh.cand_key[i];
      const uint32_t t = sh.cand_t[i];
      if (key > thr || (key == thr && ~t >= t_key_min)) {
        const uint32_t slot = atomicAdd(&sh.n_sel, 1u);
        if (slot < (uint32_t)kTopkMaxK) {
          sh.sel_s[slot] = key_score(key);
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
  // kept keys in groups of GU per wave (wave w takes groups w, w+4, ...): the GU row loads of a
  // group are issued before any of them is used, so a row's latency is paid once per group
  constexpr int GU = 8;
  auto load_row = [&](const uint16_t* vp, uint16_t (&raw)[PER]) {
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
  };
  for (uint32_t j0 = wave * GU; j0 < k; j0 += 4u * GU) {
    float pj[GU];
    uint16_t raw[GU][PER];
#pragma unroll
    for (int u = 0; u < GU; ++u) {
      const uint32_t j = min(j0 + (uint32_t)u, k - 1u);          // past the end: the last key again, weight 0
      pj[u] = j0 + (uint32_t)u < k ? sh.sel_s[j] * inv : 0.f;
      const uint32_t tj = min(sh.sel_t[j], p.t_all - 1u);       // (kept positions are < t_all by construction)
      const uint16_t* vp = (const uint16_t*)(vbase + (int64_t)kv_slot(p.ring_mask, tj) * vstride_b);
      if (lane_on) load_row(vp, raw[u]);
    }
    if (lane_on) {
#pragma unroll
      for (int u = 0; u < GU; ++u) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const float v = F16 ? (float)__builtin_bit_cast(_Float16, raw[u][i]) : bf16_bits_to_f32(raw[u][i]);
          acc[i] = __builtin_fmaf(pj[u], v, acc[i]);
        }
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
hipError_t launch_stage(const TopkParams& tp, int stage, hipStream_t s) {
  if (stage == 0) {
    const uint32_t n_units = tp.a.hkv * tp.n_splits * tp.n_mtiles;
    const uint32_t grid = ((n_units + 7u) / 8u) * 8u;
    hipLaunchKernelGGL((topk_scores_kernel<D, F16>), dim3(grid), dim3(256), 0, s, tp);
  } else {
    hipLaunchKernelGGL((topk_select_kernel<D, F16>), dim3(tp.ntok, tp.a.hq), dim3(256), 0, s, tp);
  }
  return hipGetLastError();
}

template <bool F16>
hipError_t launch_by_dim(const TopkParams& tp, int stage, uint32_t head_dim, hipStream_t s) {
  switch (head_dim) {
    case 32: return launch_stage<32, F16>(tp, stage, s);
    case 64: return launch_stage<64, F16>(tp, stage, s);
    case 128: return launch_stage<128, F16>(tp, stage, s);
    case 256: return launch_stage<256, F16>(tp, stage, s);
    case 512: return launch_stage<512, F16>(tp, stage, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

hipError_t launch_topk_scores(const TopkParams& tp, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s) {
  return kv_dtype == 1u ? launch_by_dim<true>(tp, 0, head_dim, s) : launch_by_dim<false>(tp, 0, head_dim, s);
}
hipError_t launch_topk_select(const TopkParams& tp, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s) {
  return kv_dtype == 1u ? launch_by_dim<true>(tp, 1, head_dim, s) : launch_by_dim<false>(tp, 1, head_dim, s);
}

}  // namespace dg
