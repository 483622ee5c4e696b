// Denoise-step attention for short key ranges (a sliding-window layer: ~1300 visible keys) in ONE launch.
//
// A sliding layer is a 5 GFLOP problem: split over workgroups along the keys (attn_mfma.hip), most of its
// time is what the split costs (partial rows written to memory, a second kernel that reads them back, two
// launches), not its tile loop.  Here the keys are split over the four WAVES of a workgroup instead and the
// partial results meet in LDS:
//
//   workgroup = 32 stacked query rows of one KV head (stacked row = canvas_row * group + head_in_group),
//   wave w    = a quarter of the key tiles those rows can see, all 32 rows, the whole head_dim.
//
// A wave holds Q (B operand of S^T = K.Q^T) for the 32 rows and the 32 x head_dim accumulators O in
// registers, streams its own 32-key K and V tiles into its own piece of LDS with direct-to-LDS loads, and
// waits only for its own loads (vmcnt): the tile loop has no workgroup barrier.  The score accumulator
// holds, per lane, 16 keys of the lane's row in exactly the order the B operand of O^T += V^T.P^T wants
// them, so P never leaves the registers.  K and V have one buffer each per wave (two would not fit the
// LDS): per tile a wave runs softmax(j), with the loads of K(j+1) issued as soon as the tile's maximum has
// read the scores (the K buffer is free once the scores of tile j exist), then P.V(j), then the scores of tile
// j+1 with the loads of V(j+1) between its middle MFMAs (the V buffer is free after P.V).  A tile's loads go out
// in groups under one setting of M0 (the instruction's immediate offset moves the LDS address as well).
// At the end the four (m, l, O) of a row are combined through LDS with the closed form
//   m = max m_i,  l = sum l_i 2^(m_i - m),  O = sum O_i 2^(m_i - m) / l,
// always in the order of the waves (run-to-run bit-identical), and each output row is stored once, whole.
//
// The cost of this shape: a tile is read by one wave only, so every workgroup streams all keys of its KV
// head through its compute unit's load path (64 B/clk: 32 KiB per wave and tile is 2048 cycles for four
// waves, twice the tile's MFMA time) and reads every byte back from LDS once, V through the transposing
// read at half rate; and the launch has only n_kv_heads * rows / 32 workgroups (128 on a sliding layer).
// Measured at head_dim 256: 7 us fixed + 1.1 us per tile and wave.  It beats the split kernel up to about
// 64 visible key tiles (a sliding layer's 40: 18.1 us against 23.4 us for kernel + merge); the host picks
// it there (dg_attn_api.hip) and the split kernel elsewhere.
// Softmax arithmetic (lazy reference max, exponent offset under which negligible weights become exact zeros,
// row sum over the rounded probabilities) is that of attn_mfma.hip, without its explicit zeroing of weights
// far below the running max (a power device of the long kernel; here it would only cost instructions).
#include "attn_params.h"
#include "mfma_tile.h"
#include "wt_store.h"

namespace dg {
namespace {

constexpr int kWsRows = 32;   // stacked rows per workgroup

template <bool F16>
constexpr float kWsTau = F16 ? 15.9f : 120.0f;   // as attn_mfma.hip: how far a tile max may exceed the reference
template <bool F16>
constexpr float kWsPOff = F16 ? 0.0f : 86.0f;    // probabilities are stored as 2^(score - reference - offset)
// With f16 probabilities a raise puts the reference this many binades ABOVE the running max, so that the next
// raise needs a score 2^(15.9 + 4) over it: a wave of a sliding layer rescales O 3.3 times in its 10 tiles instead
// of 5.6 (a rescale is 128 accumulation registers read, multiplied and written: as long as a tile).  The price is
// f16's tail: a weight more than 2^(24 - 4) below the row's largest is stored with an absolute error of up to
// 2^-25 of the reference or dropped, i.e. up to 2^-21 of the largest weight per key; this kernel sees at most 2048
// keys per row (64 tiles, dg_attn_api.hip), so at most 2^-10 of a row's mass moves: under the rounding of a 16-bit
// output (tests/test_gpu_parity.py builds the worst case).  The kernel for long key ranges (attn_mfma.hip) keeps a
// reference that never leads: at 33 024 keys the same bound would be 2^-6.
template <bool F16>
constexpr float kWsLead = F16 ? 4.0f : 0.0f;

typedef __bf16 ws_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 ws_f16x2 __attribute__((ext_vector_type(2)));
template <bool F16>
__device__ __forceinline__ float ws_add_pair(uint32_t pk, float acc) {
  if constexpr (F16) {
    const ws_f16x2 ones = {(_Float16)1.f, (_Float16)1.f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(ws_f16x2, pk), ones, acc, false);
  } else {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(ws_bf16x2, pk), __builtin_bit_cast(ws_bf16x2, 0x3f803f80u),
                                           acc, false);
  }
}

// all but the N most recent vector memory operations of the wave (N up to 63: vmcnt is bits 3:0 and 15:14)
template <int N>
__device__ __forceinline__ void ws_wait_vmem_but() {
  static_assert(N >= 0 && N < 64, "six bits of vmcnt");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
  asm volatile("" ::: "memory");
}

// One whole 32-key tile of K or V into this wave's buffer: NBLK instructions of 64 x 16 bytes, rows dense,
// 16-byte chunks XOR-swizzled (Lay<D>), rows outside [rmin, rmax] replaced by the nearest one inside.
template <int D, bool IS_V>
__device__ __forceinline__ void ws_issue_tile(const TileLoad& tl, uint32_t lane) {
  using L = Lay<D>;
  static_for<0, L::NBLK>([&](auto b_c) {
    constexpr int blk = decltype(b_c)::value;
    const uint32_t pch = blk * 64 + lane;
    const uint32_t r = pch / L::CPR, pc = pch % L::CPR;
    const uint32_t c = pc ^ (IS_V ? L::swz_v(r) : L::swz_k(r));
    lds_dma_16<blk * 1024>(tl.base, min(max(r, tl.rmin), tl.rmax) * tl.stride_b + c * 16u, tl.lds);
  });
}

template <int D, bool F16>
__global__ void __launch_bounds__(256) attn_wsplit_kernel(const AttnParams p_in) {
  const AttnParams p = resolve_step(p_in);
  using L = Lay<D>;
  static_assert(!L::PAD, "head_dim 512 does not fit: O alone would fill the register file");
  constexpr int NSTEP = D / 16, NDB = D / 32, NBLK = L::NBLK;
  constexpr int STG_ROW = D * 4 + 16;   // bytes of a staged fp32 row of O; the pad keeps 16-byte writes of 8 rows apart
  constexpr int TILE_BYTES = L::K_BYTES + L::V_BYTES;
  constexpr int SLICE = ((TILE_BYTES > 32 * STG_ROW ? TILE_BYTES : 32 * STG_ROW) + 1023) / 1024 * 1024;
  constexpr int OFF_Q = 4 * SLICE, OFF_ML = OFF_Q + L::K_BYTES, OFF_DUMP = OFF_ML + 4 * 32 * 2 * 4;
  constexpr int LDS_BYTES = OFF_DUMP + 4 * 256;
  static_assert(LDS_BYTES <= 160 * 1024, "LDS of one compute unit");
  __shared__ __attribute__((aligned(1024))) char smem[LDS_BYTES];
  float* const sml = (float*)(smem + OFF_ML);

  // ---- which (KV head, row tile) this workgroup owns: ids go round-robin over the 8 XCDs (each has its
  // own L2); the units, KV head first, are cut into 8 equal runs, so the row tiles of a head, which stream
  // the same keys, sit behind one L2 ----
  const uint32_t n_rt = (p.rows_total + kWsRows - 1) / kWsRows;
  const uint32_t n_units = p.hkv * n_rt;
  const uint32_t per_xcd = (n_units + 7u) >> 3;
  const uint32_t unit = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
  if (unit >= n_units) return;
  const uint32_t kvh = __builtin_amdgcn_readfirstlane(unit / n_rt);
  const uint32_t rt = __builtin_amdgcn_readfirstlane(unit % n_rt);

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t g2 = lane >> 5, l32 = lane & 31u, h16 = (lane >> 4) & 1u, i16 = lane & 15u;

  // ---- this lane's query row and its key bounds ----
  const uint32_t row0 = rt * kWsRows;
  const uint32_t r = row0 + l32;
  const bool row_ok = r < p.rows_total;
  const uint32_t tok = row_ok ? r / p.group : 0u;
  RowBounds rb = row_bounds(p, tok);
  if (!row_ok) {
    rb.lo = 0;
    rb.hi = 0;
    rb.extra = p.t_all;
  }
  // ---- bounds that hold for every row of the workgroup: which key tiles to visit, which need the mask ----
  uint32_t lo_min, lo_max, hi_min, hi_max;
  {
    const uint32_t last_row = min(row0 + kWsRows, p.rows_total) - 1u;
    const uint32_t tok_a = row0 / p.group, tok_b = last_row / p.group;
    const RowBounds ba = row_bounds(p, tok_a), bb = row_bounds(p, tok_b);
    lo_min = min(ba.lo, bb.lo);
    lo_max = max(ba.lo, bb.lo);
    hi_min = min(ba.hi, bb.hi);
    hi_max = max(ba.hi, bb.hi);
    if (tok_a < p.causal_rows && tok_b >= p.causal_rows) {  // both kinds of rows in the tile
      const RowBounds bc = row_bounds(p, p.causal_rows - 1u), bd = row_bounds(p, p.causal_rows);
      lo_min = min(lo_min, min(bc.lo, bd.lo));
      lo_max = max(lo_max, max(bc.lo, bd.lo));
      hi_min = min(hi_min, min(bc.hi, bd.hi));
      hi_max = max(hi_max, max(bc.hi, bd.hi));
    }
    if (tok_a < p.causal_rows && p.extra_lo < p.t_clip_hi) hi_max = p.t_clip_hi;
    if (row0 + kWsRows > p.rows_total) hi_min = 0;  // ragged tile: always take the masked path
    lo_min = __builtin_amdgcn_readfirstlane(lo_min);
    lo_max = __builtin_amdgcn_readfirstlane(lo_max);
    hi_min = __builtin_amdgcn_readfirstlane(hi_min);
    hi_max = __builtin_amdgcn_readfirstlane(hi_max);
  }
  // the key tiles these rows can see, cut into four equal runs, one per wave
  const uint32_t mt_begin = max(lo_min / kBlockN, p.tile_first);
  const uint32_t mt_end = max(min((hi_max + kBlockN - 1) / kBlockN, p.tile_end), mt_begin);
  const uint32_t per_wave = (mt_end - mt_begin + 3u) >> 2;
  const uint32_t tb = __builtin_amdgcn_readfirstlane(min(mt_begin + wave * per_wave, mt_end));
  const uint32_t te = __builtin_amdgcn_readfirstlane(min(tb + per_wave, mt_end));
  const uint32_t ntile = te - tb;

  const char* kbase = (const char*)p.k + (int64_t)kvh * p.k_head_stride * 2;
  const char* vbase = (const char*)p.v + (int64_t)kvh * p.v_head_stride * 2;
  const int64_t kstride_b = p.k_tok_stride * 2, vstride_b = p.v_tok_stride * 2;
  lds_char* const kb = (lds_char*)smem + wave * SLICE;
  lds_char* const vb = kb + L::K_BYTES;
  auto k_load = [&](uint32_t tile) {
    return make_tile_load<D, false, true>(kbase, kstride_b, tile * kBlockN, lo_min, p.t_all, p.ring_mask, kb, 0u, lane);
  };
  auto v_load = [&](uint32_t tile) {
    return make_tile_load<D, true, true>(vbase, vstride_b, tile * kBlockN, lo_min, p.t_all, p.ring_mask, vb, 0u, lane);
  };

  // Offsets of a tile's NBLK load instructions, per lane, for a tile whose 32 rows all exist (every tile but
  // the first one, when the range starts inside it, and the last one, when the keys end inside it): block
  // blk covers rows blk * 64 / CPR ..., lane l the 16-byte chunk l of the block, swizzled.  Worked out once;
  // the tile's base address is scalar.
  // The loads go out in groups that share one setting of M0 (lds_dma_16_group): four blocks of a K tile (its
  // loads are issued together), two blocks of a V tile (two go between a pair of score MFMAs); the offsets
  // carry the group's bias.
  constexpr int GK = NBLK >= 4 ? 4 : NBLK, GV = 2;
  static_assert(NBLK % GK == 0 && NBLK % GV == 0 && GK <= 4, "groups tile the blocks");
  uint32_t koff[NBLK], voff[NBLK];
#pragma unroll
  for (int blk = 0; blk < NBLK; ++blk) {
    const uint32_t pch = blk * 64 + lane;
    const uint32_t rr_ = pch / L::CPR, pc = pch % L::CPR;
    koff[blk] = rr_ * (uint32_t)kstride_b + ((pc ^ L::swz_k(rr_)) << 4) + kDmaBias - (uint32_t)(blk % GK) * 1024u;
    voff[blk] = rr_ * (uint32_t)vstride_b + ((pc ^ L::swz_v(rr_)) << 4) + kDmaBias - (uint32_t)(blk % GV) * 1024u;
  }
  // a tile with rows that must not be read (before the first visible key: dead ring slots; past the last key)
  auto tile_is_edge = [&](uint32_t tile) { return tile * kBlockN < lo_min || tile * kBlockN + kBlockN > p.t_all; };
  // one tile's loads: offsets from the table, or (a tile with rows that must not be read) worked out with the
  // clamp into a table of their own first; the branch is per tile, the loads themselves are the same code
  auto edge_table = [&](auto is_v_c, const TileLoad& tl, uint32_t (&tab)[NBLK]) {
    constexpr bool IS_V = decltype(is_v_c)::value;
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
      const uint32_t pch = blk * 64 + lane;
      const uint32_t rr_ = pch / L::CPR, pc = pch % L::CPR;
      const uint32_t c = pc ^ (IS_V ? L::swz_v(rr_) : L::swz_k(rr_));
      tab[blk] = min(max(rr_, tl.rmin), tl.rmax) * tl.stride_b + c * 16u + kDmaBias - (uint32_t)(blk % (IS_V ? GV : GK)) * 1024u;
    }
  };
  // group g of a tile's loads: blocks g G .. g G + G - 1
  auto issue_group = [&](auto is_v_c, auto g_c, const TileLoad& tl, const uint32_t (&tab)[NBLK]) {
    constexpr int G = decltype(is_v_c)::value ? GV : GK;
    constexpr int g = decltype(g_c)::value;
    lds_dma_16_group<G, g * G * 1024>(tl.base - kDmaBias, &tab[g * G], tl.lds);
  };
  using IsK = std::false_type;
  using IsV = std::true_type;
  constexpr int NGK = NBLK / GK, NGV = NBLK / GV;

  // ---- the first K and V tiles are on their way before anything waits for the query rows ----
  if (ntile > 0) {
    uint32_t tab[NBLK];
    const TileLoad ktl0 = k_load(tb);
    edge_table(IsK{}, ktl0, tab);
    static_for<0, NGK>([&](auto g_c) { issue_group(IsK{}, g_c, ktl0, tab); });
    const TileLoad vtl0 = v_load(tb);
    edge_table(IsV{}, vtl0, tab);
    static_for<0, NGV>([&](auto g_c) { issue_group(IsV{}, g_c, vtl0, tab); });
  }

  // ---- Q fragments: B operand of S^T = K.Q^T, lane = row, 8 consecutive d per step.  The 32 rows come in
  // through LDS as whole rows, in the layout of a K tile, a quarter of the 1 KiB blocks per wave; every wave
  // then reads all of them the way it reads K fragments. ----
  u32x4 qf[NSTEP];
  {
    lds_char* const qb = (lds_char*)smem + OFF_Q;
    const uint32_t rq = min(r, p.rows_total - 1u);   // rows past the last one repeat it (they are masked everywhere)
    const uint32_t q_row_off = ((rq / p.group * p.hq) + kvh * p.group + rq % p.group) * (uint32_t)(2 * D);
    static_for<0, (NBLK + 3) / 4>([&](auto b_c) {
      constexpr int bi = decltype(b_c)::value;
      const uint32_t blk = bi * 4 + wave;
      const uint32_t pch = blk * 64 + lane;
      const uint32_t rl = (pch / L::CPR) & 31u, pc = pch % L::CPR;
      const uint32_t c = pc ^ L::swz_k(rl);
      const uint32_t off = __shfl(q_row_off, (int)rl, 64) + c * 16u;
      if (NBLK >= 4 || blk < (uint32_t)NBLK) lds_dma_16<0>((const char*)p.q, off, (uint32_t)(size_t)qb + blk * 1024u);
    });
    // ---- while those are on their way: the rest of the key range is touched into the L2 ----
    // In a loop over many layers a layer's cache rows come from HBM every time, and with one buffer per
    // matrix a tile's loads have half a tile's time to land, which covers the L2 and not HBM (measured:
    // a sliding layer 20.6 us with the rows cached, 26.2 us from HBM, 22.4 us with the touches).  The workgroups of a KV head sit
    // behind one L2 and stream the same keys, so they share the work: NTOUCH instructions per wave, a
    // 128-byte line per lane, tile after tile (K lines, then V lines); a lane whose share lies past the range
    // repeats the last line.  Touches are loads into a dump area nobody reads; they are the newest loads at
    // the wait below, which leaves them out.
    constexpr int NTOUCH = 4;
    {
      constexpr uint32_t LPRW = 2 * D >= 128 ? 2 * D / 128 : 1;   // lines per key row
      constexpr uint32_t LPT = 32 * LPRW;                        // lines per tile and matrix
      // (the offsets below are 32-bit: a range or ring whose rows span 4 GiB goes without touches)
      const uint64_t span_rows = p.ring_mask ? (uint64_t)p.ring_mask + 1u : (uint64_t)(mt_end - mt_begin) * kBlockN;
      const bool fits = span_rows * (uint64_t)max(kstride_b, vstride_b) < (1ull << 32);
      const uint32_t n_lines = fits ? (mt_end - mt_begin) * 2u * LPT : 0u;
      const uint32_t dump = (uint32_t)(size_t)((lds_char*)smem + OFF_DUMP + wave * 256u);
      if (n_lines > 0) {
        static_for<0, NTOUCH>([&](auto t_c) {
          constexpr uint32_t t = decltype(t_c)::value;
          const uint32_t idx = min(t * (256u * n_rt) + rt * 256u + threadIdx.x, n_lines - 1u);
          const uint32_t tile_i = idx / (2u * LPT), rem = idx % (2u * LPT);
          const bool is_v = rem >= LPT;
          const uint32_t li = is_v ? rem - LPT : rem;
          const uint32_t pos = min(max((mt_begin + tile_i) * kBlockN + li / LPRW, lo_min), p.t_all - 1u);
          // (32-bit byte offsets: from the ring's first slot, or from the first position of the range)
          const uint32_t first = p.ring_mask ? 0u : mt_begin * kBlockN;
          const uint32_t rel = p.ring_mask ? (pos & p.ring_mask) : pos - min(first, pos);
          const uint32_t off_k = rel * (uint32_t)kstride_b + (li % LPRW) * 128u;
          const uint32_t off_v = rel * (uint32_t)vstride_b + (li % LPRW) * 128u;
          // one instruction per matrix would need two bases: the lanes of a wave straddle K and V lines only
          // at a tile's middle, so the base is chosen per wave from its first lane and the other lanes follow
          const bool wave_v = __builtin_amdgcn_readfirstlane((uint32_t)is_v) != 0u;
          const char* base = (wave_v ? vbase : kbase) + (int64_t)first * (wave_v ? vstride_b : kstride_b);
          lds_dma_touch(base, wave_v == is_v ? (wave_v ? off_v : off_k) : 0u, dump);
        });
      } else {
        static_for<0, NTOUCH>([&](auto) { lds_dma_touch(kbase, 0u, dump); });   // keeps the count of loads the wait assumes
      }
    }
    ws_wait_vmem_but<NTOUCH>();
    __syncthreads();
    const uint32_t q_lane_off = l32 * L::K_STRIDE;
    const uint32_t q_swz = L::swz_k(l32);
#pragma unroll
    for (int s = 0; s < NSTEP; ++s) {
      const u32x4 raw = *(lds_u32x4*)(qb + q_lane_off + ((((uint32_t)(2 * s) + g2) ^ q_swz) << 4));
      if (F16 && p.q_is_bf16) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          qf[s][e] = pack2<true>(__uint_as_float(raw[e] << 16), __uint_as_float(raw[e] & 0xffff0000u));
      } else {
        qf[s] = raw;
      }
    }
  }

  f32x16 o[NDB];
#pragma unroll
  for (int i = 0; i < NDB; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[i][e] = 0.f;
  float m_ref = -INFINITY;   // reference max of the row in use, log2 units (scale folded in)
  float m_run = -INFINITY;   // running max itself
  float l_part = 0.f, l_part2 = 0.f;   // this lane's share of the row sum (its 16 of every 32 keys)

  // per-lane LDS byte offsets of the fragment reads
  const uint32_t k_lane_off = l32 * L::K_STRIDE;
  const uint32_t k_swz = L::swz_k(l32);
  const uint32_t v_row = 4u * g2 + (i16 >> 2);
  const uint32_t v_swz = L::swz_v(v_row);
  const uint32_t v_lane_chunk = 2u * h16 + ((i16 & 3u) >> 1);
  const uint32_t v_lane_off = v_row * L::V_STRIDE + (i16 & 1u) * 8u;
  // K fragment of MFMA step st: A operand, lane = key row l32, 8 consecutive d at 16 st + 8 g2
  auto k_frag = [&](int st) -> u32x4 {
    return *(lds_u32x4*)(kb + k_lane_off + ((((uint32_t)(2 * st) + g2) ^ k_swz) << 4));
  };
  // V^T fragment of k-step ks, d-block db: k-slot j of lane half g2 is key 16 ks + 8 (j>>2) + 4 g2 + (j&3),
  // the order in which the score accumulator holds a lane's keys
  auto v_frag = [&](int ks, int db) -> u32x4 {
    const uint32_t off = v_lane_off + (uint32_t)(16 * ks) * L::V_STRIDE + (((uint32_t)(4 * db) + v_lane_chunk) ^ v_swz) * 16u;
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vb + off)));
    const u32x2 hi = __builtin_bit_cast(
        u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vb + off + 8 * L::V_STRIDE)));
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  };

  // S^T = K.Q^T of the tile in the K buffer.  The score MFMAs are assembly with an ordinary register tuple as
  // accumulator: left to the compiler they accumulate in the same register class as O, and O then moves
  // between the classes around every tile.  Fragment reads run PFK steps ahead of the MFMA that consumes them
  // (the loads between the MFMAs are assembly the compiler will not move LDS reads across, so the distance is
  // spelled out).  `between(st)` is what follows MFMA st in program order.
  f32x16 s;
  auto scores = [&](auto&& between) {
    constexpr int PFK = NSTEP < 4 ? NSTEP : 4;
    u32x4 kf[PFK];
#pragma unroll
    for (int i = 0; i < PFK; ++i) kf[i] = k_frag(i);
    static_for<0, NSTEP>([&](auto st_c) {
      constexpr int st = decltype(st_c)::value;
      if constexpr (st == 0) mfma_scores_first<F16>(s, kf[0], qf[0]);
      else if constexpr (st == NSTEP - 1) mfma_scores_last<F16>(s, kf[st % PFK], qf[st]);
      else mfma_scores_acc<F16>(s, kf[st % PFK], qf[st]);
      if constexpr (st + PFK < NSTEP) kf[st % PFK] = k_frag(st + PFK);
      between(st_c);
    });
    // every K fragment is in registers: the buffer may take the next tile
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };
  if (ntile > 0) scores([](auto) {});   // (K(tb) and V(tb) landed with the query rows)

  for (uint32_t jj = 0; jj < ntile; ++jj) {
    const uint32_t tile = tb + jj;
    const uint32_t t0 = tile * kBlockN;
    const bool more = jj + 1u < ntile;
    // The scores of tile jj are in s.  The K buffer takes tile jj + 1.
    const TileLoad ktl = k_load(min(tile + 1u, te - 1u));
    const bool k_edge = tile_is_edge(min(tile + 1u, te - 1u));

    // ---- online softmax with a lazily raised reference max ----
    if (__builtin_expect(!(t0 >= lo_max && t0 + kBlockN <= hi_min), 0)) {   // edge tile: mask
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t t = t0 + 8u * (e >> 2) + 4u * g2 + (e & 3);
        if (!key_visible(rb, t, p.t_clip_hi)) s[e] = -INFINITY;
      }
    }
    float tmax;
    {
      const float a0 = fmaxf(fmaxf(s[0], s[1]), s[2]), a1 = fmaxf(fmaxf(s[3], s[4]), s[5]);
      const float a2 = fmaxf(fmaxf(s[6], s[7]), s[8]), a3 = fmaxf(fmaxf(s[9], s[10]), s[11]);
      const float a4 = fmaxf(fmaxf(s[12], s[13]), s[14]);
      tmax = fmaxf(fmaxf(fmaxf(a0, a1), a2), fmaxf(fmaxf(a3, a4), s[15]));
    }
    // The scores of this tile are read (the K buffer was free since they existed): the next K tile's loads, all of
    // them here, behind the tile max and ahead of everything that depends on it.  (Spread through the softmax
    // in quarters they cost 0.3 us more per sliding layer, at the very top of the loop 0.1.)
    if (more) {
      if (__builtin_expect(k_edge, 0)) {   // (its own copy of the loads: the common path reads the table as it stands)
        uint32_t etab[NBLK];
        edge_table(IsK{}, ktl, etab);
        static_for<0, NGK>([&](auto g_c) { issue_group(IsK{}, g_c, ktl, etab); });
      } else {
        static_for<0, NGK>([&](auto g_c) { issue_group(IsK{}, g_c, ktl, koff); });
      }
    }
    tmax = max_across_halves(tmax) * p.scale_log2;
    const bool raise = __builtin_amdgcn_ballot_w64(tmax > m_ref + kWsTau<F16>) != 0ull;
    m_run = fmaxf(m_run, tmax);
    if (__builtin_expect(raise, 0)) {
      // one row has to raise its reference: every row moves up to its running max (the block is rescaled
      // anyway, and the next raise is then as far away as it can be)
      const float m_new = fmaxf(m_ref, m_run + kWsLead<F16>);
      const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_ref - m_new);
      const bool rescale = __builtin_amdgcn_ballot_w64(m_ref != -INFINITY && corr != 1.f) != 0ull;
      l_part *= corr;
      l_part2 *= corr;
      if (rescale) {   // O stays in the accumulation registers: spelled out, or the allocator moves all of it
#pragma unroll
        for (int i = 0; i < NDB; ++i)
#pragma unroll
          for (int e = 0; e < 16; e += 8) {
            float x0 = o[i][e], x1 = o[i][e + 1], x2 = o[i][e + 2], x3 = o[i][e + 3];
            float x4 = o[i][e + 4], x5 = o[i][e + 5], x6 = o[i][e + 6], x7 = o[i][e + 7];
            scale_acc8(x0, x1, x2, x3, x4, x5, x6, x7, corr);
            o[i][e] = x0;
            o[i][e + 1] = x1;
            o[i][e + 2] = x2;
            o[i][e + 3] = x3;
            o[i][e + 4] = x4;
            o[i][e + 5] = x5;
            o[i][e + 6] = x6;
            o[i][e + 7] = x7;
          }
        scale_acc_done();
      }
      m_ref = m_new;
    }
    // The probabilities are 2^(score - reference - offset): with bf16 the offset puts a weight 2^40 below the
    // reference (and so below the row's largest) under the smallest normal number, an exact zero.
    const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref + kWsPOff<F16>;
    u32x4 pk[2];
    static_for<0, 4>([&](auto q_c) {
      constexpr int q = decltype(q_c)::value;
      float ex[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) ex[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[4 * q + i], p.scale_log2, -m_use));
      pk[q >> 1][(2 * q) & 3] = pack2<F16>(ex[0], ex[1]);
      pk[q >> 1][(2 * q + 1) & 3] = pack2<F16>(ex[2], ex[3]);
    });
    // the row sum uses the rounded probabilities, the same numbers P.V multiplies
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      l_part = ws_add_pair<F16>(pk[ks][0], l_part);
      l_part2 = ws_add_pair<F16>(pk[ks][1], l_part2);
      l_part = ws_add_pair<F16>(pk[ks][2], l_part);
      l_part2 = ws_add_pair<F16>(pk[ks][3], l_part2);
    }

    // ---- O^T += V^T.P^T ----
    // V(jj) has landed (the loads of K(jj+1), issued after it, may still be on their way)
    if (more) ws_wait_vmem_but<NBLK>();
    else wait_vmem_all();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int db = 0; db < NDB; ++db) o[db] = mfma16<F16>(v_frag(ks, db), pk[ks], o[db]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the V buffer is free for the next tile's loads
    if (more) {
      // ---- scores of tile jj + 1 (K(jj+1), the only load outstanding, has landed), with the loads of
      // V(jj+1) between its MFMAs: they have the rest of the scores and the softmax to land ----
      wait_vmem_all();
      const TileLoad vtl = v_load(tile + 1u);
      uint32_t vtab[NBLK];
      if (__builtin_expect(tile_is_edge(tile + 1u), 0)) {
        edge_table(IsV{}, vtl, vtab);
      } else {
#pragma unroll
        for (int blk = 0; blk < NBLK; ++blk) vtab[blk] = voff[blk];
      }
      scores([&](auto st_c) {
        constexpr int st = decltype(st_c)::value;
        constexpr int first = (NSTEP - NGV) / 2;   // behind the middle MFMAs (behind the first ones: +0.15 us per
                                                   // sliding layer, behind the last ones +0.1, after them all +0.8)
        if constexpr (st >= first && st < first + NGV) issue_group(IsV{}, std::integral_constant<int, st - first>{}, vtl, vtab);
      });
    }
  }
  wait_vmem_all();   // (only when ntile == 0 is there nothing to wait for; cheap either way)

  // ---- the four waves' (m, l, O) of every row meet in LDS ----
  const float l_tot = sum_across_halves(l_part + l_part2);
  const float m_pub = m_ref + kWsPOff<F16>;   // the exponent the sums are relative to
  if (g2 == 0) {
    sml[(wave * 32u + l32) * 2u] = m_pub;
    sml[(wave * 32u + l32) * 2u + 1u] = l_tot;
  }
  {
    lds_char* const stg = kb;   // this wave's own slice: its tile buffers are free now
#pragma unroll
    for (int i = 0; i < NDB; ++i)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const f32x4 v4 = acc_read4<true>(o[i], 4 * q4);
        *(__attribute__((address_space(3))) f32x4*)(stg + l32 * STG_ROW + (32 * i + 8 * q4 + 4 * g2) * 4) = v4;
      }
  }
  __syncthreads();
  // wave w merges rows 8 w .. 8 w + 7 of the workgroup: a row is D / 4 lanes of four d each.  Everything the
  // passes need is asked of LDS first (the registers are free now), so that the passes do not each wait for a
  // chain of reads.
  constexpr int LPR = D / 4 < 64 ? D / 4 : 64;   // lanes per row
  constexpr int RPP = 64 / LPR;                  // rows per pass
  constexpr int NPASS = 8 / RPP;
  static_assert(D / 4 <= 64, "a row is at most one pass of the wave");
  const uint32_t dl = lane % LPR;                // which four d
  // The weights of the wave's 8 rows, one row per lane (the lanes past 7 repeat them): w_i = 2^(m_i - m) for
  // the waves that saw a key of the row, 1 / l, and the row's log-sum-exp.  The passes below take them from
  // the lane that holds their row instead of every lane working them out again for every row.
  float wrow[4], inv_row, lse_row;
  bool den_ok_row;
  {
    const uint32_t rl = wave * 8u + (lane & 7u);
    float mi[4], li[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      mi[i] = sml[(i * 32u + rl) * 2u];
      li[i] = sml[(i * 32u + rl) * 2u + 1u];
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) mx = li[i] > 0.f ? fmaxf(mx, mi[i]) : mx;
#pragma unroll
    for (int i = 0; i < 4; ++i) wrow[i] = li[i] > 0.f ? __builtin_amdgcn_exp2f(mi[i] - mx) : 0.f;
    const float den = (wrow[0] * li[0] + wrow[1] * li[1]) + (wrow[2] * li[2] + wrow[3] * li[3]);
    den_ok_row = den > 0.f;
    inv_row = den_ok_row ? __builtin_amdgcn_rcpf(den) : 0.f;
    lse_row = den_ok_row ? mx * kLn2 + __logf(den) : -INFINITY;
  }
  f32x4 part[NPASS][4];
#pragma unroll
  for (int pass = 0; pass < NPASS; ++pass) {
    const uint32_t rl = wave * 8u + pass * RPP + lane / LPR;   // row within the workgroup
#pragma unroll
    for (int i = 0; i < 4; ++i)
      part[pass][i] = *(__attribute__((address_space(3))) f32x4*)((lds_char*)smem + i * SLICE + rl * STG_ROW + dl * 16u);
  }
  // value of the lane that holds the row of this pass
  auto of_row = [&](float x, int pass) -> float {
    if constexpr (RPP == 1) return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(x), pass));
    else return __shfl(x, (int)(pass * RPP + lane / LPR), 64);
  };
  // (tok, head) of the wave's first row; with a whole row per pass the rows that follow are found by counting
  // (head in group + 1, carry into the canvas row) instead of a division per pass
  const uint32_t r_first = row0 + wave * 8u;
  uint32_t tok_s = __builtin_amdgcn_readfirstlane(r_first / p.group);
  uint32_t g_s = __builtin_amdgcn_readfirstlane(r_first % p.group);
  const bool f32_out = p.out_dtype == DT_F32, trunc_out = p.out_trunc != 0;
#pragma unroll
  for (int pass = 0; pass < NPASS; ++pass) {
    const uint32_t rr = r_first + pass * RPP + lane / LPR;
    uint32_t tok_o, g_o;
    if constexpr (RPP == 1) {
      tok_o = tok_s;
      g_o = g_s;
      g_s += 1u;
      if (g_s == p.group) {
        g_s = 0u;
        tok_s += 1u;
      }
    } else {
      tok_o = rr / p.group;
      g_o = rr % p.group;
    }
    const float inv = of_row(inv_row, pass);
    const float lse_v = of_row(lse_row, pass);
    // (a wave that saw no key of the row holds exact zeros there and gets weight zero)
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float w = of_row(wrow[i], pass);
      acc[0] = __builtin_fmaf(w, part[pass][i][0], acc[0]);
      acc[1] = __builtin_fmaf(w, part[pass][i][1], acc[1]);
      acc[2] = __builtin_fmaf(w, part[pass][i][2], acc[2]);
      acc[3] = __builtin_fmaf(w, part[pass][i][3], acc[3]);
    }
    if (rr >= p.rows_total) continue;
    const float y0 = acc[0] * inv, y1 = acc[1] * inv, y2 = acc[2] * inv, y3 = acc[3] * inv;
    const uint32_t qh_o = kvh * p.group + g_o;
    const size_t row_idx = (size_t)tok_o * p.hq + qh_o;
    if (p.lse && dl == 0) p.lse[row_idx] = lse_v;
    if (p.dbg) {
      const uint32_t tag = (tok_o << 16) | qh_o;
      if (dl == 0 && lse_v == -INFINITY) dbg_report(p.dbg, DBG_ERR_SOFTMAX_NORM_ZERO, DBG_KERNEL_ATTENTION, tag, tag);
      if (!(fabsf(y0) + fabsf(y1) + fabsf(y2) + fabsf(y3) <= 3.402823466e38f))   // NaN or infinity
        dbg_report(p.dbg, DBG_ERR_NONFINITE, DBG_KERNEL_ATTENTION, tag, dl * 4u);
    }
    // written through (wt_store.h): the next kernel reads these rows, and a kernel does not end before the
    // lines it left dirty in its L2 are written back
    if (f32_out) {
      const u32x4 v4 = {__float_as_uint(y0), __float_as_uint(y1), __float_as_uint(y2), __float_as_uint(y3)};
      if constexpr (RPP == 1) wt_store16(wt_window_wave((const float*)p.out + row_idx * D), dl * 16u, v4);
      else *(u32x4*)((float*)p.out + row_idx * D + dl * 4u) = v4;
    } else {
      u32x2 pk2;
      if (trunc_out) {
        pk2[0] = (__float_as_uint(y0) >> 16) | (__float_as_uint(y1) & 0xffff0000u);
        pk2[1] = (__float_as_uint(y2) >> 16) | (__float_as_uint(y3) & 0xffff0000u);
      } else {
        pk2[0] = pack2<false>(y0, y1);
        pk2[1] = pack2<false>(y2, y3);
      }
      if constexpr (RPP == 1) wt_store8(wt_window_wave((const uint16_t*)p.out + row_idx * D), dl * 8u, pk2);
      else *(u32x2*)((uint16_t*)p.out + row_idx * D + dl * 4u) = pk2;
    }
  }
}

template <int D, bool F16>
hipError_t launch_ws(const AttnParams& p, hipStream_t s) {
  const uint32_t n_units = p.hkv * ((p.rows_total + kWsRows - 1) / kWsRows);
  const uint32_t grid = ((n_units + 7u) / 8u) * 8u;
  hipLaunchKernelGGL((attn_wsplit_kernel<D, F16>), dim3(grid), dim3(256), 0, s, p);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_attn_wsplit(const AttnParams& p, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s) {
  const bool f16 = kv_dtype == DT_F16;
  switch (head_dim) {
    case 32: return f16 ? launch_ws<32, true>(p, s) : launch_ws<32, false>(p, s);
    case 64: return f16 ? launch_ws<64, true>(p, s) : launch_ws<64, false>(p, s);
    case 128: return f16 ? launch_ws<128, true>(p, s) : launch_ws<128, false>(p, s);
    case 256: return f16 ? launch_ws<256, true>(p, s) : launch_ws<256, false>(p, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace dg
