// Denoise-step attention on MFMA for gfx950 (MI355X).
//
// One workgroup (4 waves) owns 128 stacked query rows of one KV head and one key-range split.
// Stacked row = canvas_row * group + head_in_group, so the `group` query heads that share a KV
// head are the M dimension of the same tile and K/V are read once for all of them.
//
// Per 32-key tile every wave plays two roles:
//   row owner  (32 rows):  S^T = K.Q^T with v_mfma_f32_32x32x16 (bf16 or f16): A = K rows from
//              LDS (ds_read_b128), B = Q held in registers for the whole kernel.  Output lane =
//              query row, output registers = keys, so row max / row sum are per-lane scalars.
//              P = exp2(S*c - m) is rounded to the element type and written to LDS in exactly
//              the register image the next MFMA wants as its B operand.
//   d owner (a quarter of head_dim, all 128 rows):  O^T += V^T.P^T, A = V^T fragments read with
//              ds_read_b64_tr_b16 from the row-major V tile, B = P fragments from LDS.
// Splitting P.V over head_dim instead of rows is what keeps LDS traffic affordable: the
// transposing read runs at half the rate of ds_read_b128, and with a row split each of the four
// waves would read the whole V tile through it; with the d split each V fragment is read once
// per workgroup and the small P tile is what gets read four times.
//
// The tile loop is software-pipelined with one barrier per tile.  One wave per SIMD issues in
// order, so anything that is to overlap the matrix pipe has to sit between MFMAs in program
// order.  For tile j a wave issues, in this order:
//   score MFMAs of tile j+1, the softmax of tile j spread between them (its scores were
//   accumulated one tile earlier), ending with the store of P(j);
//   [barrier, waiting first for this wave's loads of V(j) and K(j+2)]
//   the first LDS reads of the P.V phase, then the last few score MFMAs of tile j+1, whose K
//   fragments were already in registers (they cover the latency of those reads);
//   the P.V MFMAs of tile j with, spread between them, the global loads of V(j+1) and K(j+3),
//   the copy of tile j+1's scores and the first K fragment reads of tile j+2.
// K and V tiles arrive by 16-byte direct-to-LDS loads into two buffers each; P, the rescale
// factors and the flags are double buffered too, which is what makes one barrier enough.
// The running max is only raised (and O rescaled) when some row's
// tile max exceeds it by more than 2^tau; the raise is broadcast to the d owners through LDS
// together with P.  Rescaling O costs about as much as the tile's P.V MFMAs, and with unit-RMS
// Q and K and no 1/sqrt(d) the scores of a row spread over tens of log2 units, so a small tau
// would rescale some row block on almost every tile.  Any reference below the true max is
// exact as long as nothing overflows.  bf16: tau = 120 with the probabilities stored as
// 2^(score - reference - 86), so P <= 2^34 and the fp32 sums stay below 2^34 * keys * |v|, far
// from 2^127; a weight more than 2^40 below the row's running max is stored as an exact zero.
// With f16 operands P itself has to stay below 65504: tau = 15.9, no offset.
#include "attn_params.h"
#include "mfma_tile.h"
#include "wt_store.h"

namespace dg {
namespace {

// log2 units by which a tile max may exceed the reference max before the reference is raised
// (a raise rescales a 32-row block of O, which costs about as much as a tile's P.V).  With the
// offset below the bf16 probabilities then reach 2^34 at most, and a row's sums 2^34 x keys x |v|.
template <bool F16>
constexpr float kTau = F16 ? 15.9f : 120.0f;   // f16: P <= 2^15.9 = 61147, below the largest half (65504)
// The probabilities are stored as 2^(score - reference - kPOff): with bf16 the offset moves
// their range to [2^-126, 2^34], so that a key whose weight is below 2^-40 of the reference
// (and therefore of the row's largest) underflows to an exact zero in the exponential itself.
// The reference lags the row's running max by up to kTau, so on top of that a weight is set to
// an exact zero when its score is more than kDrop below the running max.  Dropping those
// weights changes a row's sum by less than keys x 2^-40 of it, below the fp32 rounding of the
// accumulation; what it buys is power: on a long row all but a per cent or two of the keys are
// that small, a multiplier fed zeros draws little, and the clock this kernel runs at is set by
// the power of the matrix cores.  (f16 probabilities already underflow 2^-25 below 2^15.)
template <bool F16>
constexpr float kPOff = F16 ? 0.0f : 86.0f;
constexpr float kDrop = 40.0f;

// dst = src for a score tile, as instructions the compiler cannot move or merge away; part I of
// 8 copies elements 2 I and 2 I + 1
template <int I>
__device__ __forceinline__ void copy_scores_part(f32x16& dst, const f32x16& src) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  f32x2 d;
  const f32x2 v = {src[2 * I], src[2 * I + 1]};
  asm volatile("v_mov_b64 %0, %1" : "=v"(d) : "v"(v));
  dst[2 * I] = d[0];
  dst[2 * I + 1] = d[1];
}
__device__ __forceinline__ u32x4 opaque4(u32x4 v) {
  asm volatile("" : "+v"(v));
  return v;
}
// the value, made opaque to the optimiser (so that what is derived from it is recomputed where
// it is used instead of being kept in registers across the tile loop)
__device__ __forceinline__ uint32_t opaque(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}

// the value brought into the finite range of f16 (NaN stays NaN)
__device__ __forceinline__ float sat_f16(float x) { return __builtin_amdgcn_fmed3f(x, -65504.f, 65504.f); }

// acc + lo + hi of a packed pair, in one dot-product instruction
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <bool F16>
__device__ __forceinline__ float add_pair(uint32_t pk, float acc) {
  if constexpr (F16) {
    const f16x2_t ones = {(_Float16)1.f, (_Float16)1.f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, pk), ones, acc, false);
  } else {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pk), __builtin_bit_cast(bf16x2_t, 0x3f803f80u),
                                           acc, false);
  }
}

template <int D, bool F16, bool TOUCH>
__global__ void __launch_bounds__(256) attn_mfma_kernel(const AttnParams p_in) {
  const AttnParams p = resolve_step(p_in);
  using L = Lay<D>;
  constexpr int NSTEP = D / 16, NDB = D / 32;
  // P.V work split: DSPLIT groups of d-blocks x RSPLIT groups of row-blocks = 4 waves
  constexpr int DSPLIT = NDB < 4 ? NDB : 4, RSPLIT = 4 / DSPLIT;
  constexpr int NDBW = NDB / DSPLIT;   // d-blocks (32 wide) this wave accumulates
  constexpr int NRBW = 4 / RSPLIT;     // row-blocks (32 rows) this wave accumulates
  constexpr int NACC = NDBW * NRBW;
  // One LDS block, carved by hand so that the order of the buffers is fixed:
  //   K0 K1 | V0 V1 | P: [ks][row-block][lane] x 16 B | per-row rescale factor of this tile |
  //   "row-block raised its max this tile" flags | epilogue (m, l) per row
  // P, the rescale factors and the flags exist twice (tiles alternate), which is what lets the
  // tile loop run with a single barrier per tile.
  constexpr int OFF_K0 = 0, OFF_K1 = L::K_BYTES, OFF_V0 = 2 * L::K_BYTES, OFF_V1 = OFF_V0 + L::V_BYTES;
  constexpr int P_BYTES = 2 * 4 * 1024, CORR_BYTES = 4 * 32 * 4, FLAG_BYTES = 16;
  constexpr int OFF_P = 2 * L::K_BYTES + 2 * L::V_BYTES, OFF_CORR = OFF_P + 2 * P_BYTES;
  constexpr int OFF_FLAG = OFF_CORR + 2 * CORR_BYTES, OFF_ML = OFF_FLAG + 2 * FLAG_BYTES;
  // At head_dim 512, when the caller says the cache rows will come from HBM (AttnParams.touch_ahead,
  // which selects the TOUCH instance of the kernel: the other one has none of this in its loop),
  // the key and value tiles a workgroup will need are touched into the L2 PF_AHEAD tiles before their
  // loads to LDS are issued (with the rows in the memory-side cache after all the touches cost 2 %:
  // they sit in the same in-order queue as the tile loads).  Two tile buffers per matrix and one barrier per tile
  // leave a load one tile's time (1.7 us) to land, less for the loads issued late in the tile; that
  // covers the memory-side cache and not HBM under load: with the cache of a 32k-key layer not
  // resident (a schedule of 30 layers streams 1.1 GB per iteration) the workgroups took 14 % more
  // cycles at an unchanged clock.  The touch is the most recent load at every barrier of the tile
  // loop, which waits for all loads but that one, so a touch has until the barrier after the next.
  constexpr bool PREFETCH = TOUCH;
  static_assert(!TOUCH || D == 512, "a row of 1 KiB = 8 lines is assumed");
  constexpr int PF_AHEAD = 6;
  constexpr int OFF_DUMP = OFF_ML + 4 * 32 * 2 * 4;
  constexpr int LDS_BYTES = OFF_DUMP + (PREFETCH ? 256 : 0);
  static_assert(LDS_BYTES <= 160 * 1024, "LDS of one compute unit");
  static_assert(L::K_BYTES % 16 == 0 && L::V_BYTES % 16 == 0, "buffer alignment");
  __shared__ __attribute__((aligned(1024))) char smem[LDS_BYTES];
  float* const sml = (float*)(smem + OFF_ML);

  // ---- which (KV head, split, row tile) this workgroup owns ----
  // Workgroup ids go round-robin over the 8 XCDs, each with its own L2.  The units, ordered
  // (KV head, split) first and row tile second, are cut into 8 equal runs, one per XCD, so the
  // row tiles that stream the same keys sit behind one L2 and every XCD has work whatever
  // the number of (KV head, split) pairs.
  const uint32_t n_units = p.hkv * p.n_splits * p.n_mtiles;
  const uint32_t per_xcd = (n_units + 7u) >> 3;
  const uint32_t wg = blockIdx.x;
  const uint32_t unit = (wg & 7u) * per_xcd + (wg >> 3);
  if (unit >= n_units) return;
  // (the divisions by run-time values are done by the vector unit; readfirstlane tells the
  // compiler the results are the same in every lane, so everything derived from them stays in
  // scalar registers)
  const uint32_t stream = __builtin_amdgcn_readfirstlane(unit / p.n_mtiles);
  const uint32_t mt = __builtin_amdgcn_readfirstlane(unit % p.n_mtiles);
  const uint32_t kvh = __builtin_amdgcn_readfirstlane(stream / p.n_splits);
  const uint32_t split = __builtin_amdgcn_readfirstlane(stream % p.n_splits);

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t g2 = lane >> 5, l32 = lane & 31u, h16 = (lane >> 4) & 1u, i16 = lane & 15u;
  const uint32_t dgrp = wave % DSPLIT, rgrp = wave / DSPLIT;

  // ---- row-owner role: this lane's query row and its key bounds ----
  const uint32_t row0 = mt * kBlockM;
  const uint32_t r = row0 + wave * 32u + l32;
  const bool row_ok = r < p.rows_total;
  const uint32_t tok = row_ok ? r / p.group : 0u;
  const uint32_t qh = kvh * p.group + (row_ok ? r % p.group : 0u);
  RowBounds rb = row_bounds(p, tok);
  if (!row_ok) {
    rb.lo = 0;
    rb.hi = 0;
    rb.extra = p.t_all;
  }

  // ---- tile-uniform bounds: which key tiles to visit, which need the per-element mask ----
  uint32_t lo_min, lo_max, hi_min, hi_max;
  {
    const uint32_t last_row = min(row0 + kBlockM, p.rows_total) - 1u;
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
    if (row0 + kBlockM > p.rows_total) hi_min = 0;  // ragged tile: always take the masked path
    // all four are the same in every lane; say so, so that they live in scalar registers
    lo_min = __builtin_amdgcn_readfirstlane(lo_min);
    lo_max = __builtin_amdgcn_readfirstlane(lo_max);
    hi_min = __builtin_amdgcn_readfirstlane(hi_min);
    hi_max = __builtin_amdgcn_readfirstlane(hi_max);
  }
  // the key tiles this row tile can see, cut into n_splits equal runs (a causal or windowed row
  // tile sees only part of the launch's key range: cutting its own range keeps the splits even)
  const uint32_t mt_begin = max(lo_min / kBlockN, p.tile_first);
  const uint32_t mt_end = max(min((hi_max + kBlockN - 1) / kBlockN, p.tile_end), mt_begin);
  const uint32_t per_split = (mt_end - mt_begin + p.n_splits - 1u) / p.n_splits;
  const uint32_t tb = __builtin_amdgcn_readfirstlane(min(mt_begin + split * per_split, mt_end));
  const uint32_t te = __builtin_amdgcn_readfirstlane(min(tb + per_split, mt_end));
  const uint32_t ntile = te > tb ? te - tb : 0u;

  const char* kbase = (const char*)p.k + (int64_t)kvh * p.k_head_stride * 2;
  const char* vbase = (const char*)p.v + (int64_t)kvh * p.v_head_stride * 2;
  const int64_t kstride_b = p.k_tok_stride * 2, vstride_b = p.v_tok_stride * 2;
  // Touch this workgroup's share of key tile `tile` of the split (the last tile instead of one past it).
  // The row tiles of a (KV head, split) pair stream the same keys behind one L2, so they share the
  // work: a tile is 256 lines of K and 256 of V (a row is 1 KiB = 8 lines); with 16 row tiles or more,
  // row tile mt takes the sixteenth (mt mod 16) of them, 8 lines per wave in one instruction (the
  // other lanes repeat them); with fewer, an eighth.  Every workgroup touching whole tiles cost more
  // in the load pipeline than the misses it saved.
  struct Touch {
    const char* base;   // wave-uniform
    uint32_t voff;      // per lane
  };
  auto touch_address = [&](uint32_t tile, uint32_t ln) -> Touch {
    const uint32_t tp = min(tile, te - 1u) * kBlockN;
    const uint32_t sh = p.n_mtiles >= 16u ? 4u : 3u;   // log2 of the number of shares
    const uint32_t share = mt & ((1u << sh) - 1u);
    const bool is_v = (share >> (sh - 1u)) != 0u;      // the upper half of the shares are V's lines
    const uint32_t li = (share & ((1u << (sh - 1u)) - 1u)) * (512u >> sh) + wave * (128u >> sh) + (ln & ((128u >> sh) - 1u));
    const uint32_t row = min(li >> 3, p.t_all - 1u - tp);
    const int64_t stride_b = is_v ? vstride_b : kstride_b;
    const int64_t slot = (int64_t)kv_slot(p.ring_mask, tp);
    return Touch{(is_v ? vbase : kbase) + slot * stride_b, row * (uint32_t)stride_b + (li & 7u) * 128u};
  };
  auto touch = [&](const Touch& t) { lds_dma_touch(t.base, t.voff, (uint32_t)(size_t)(smem + OFF_DUMP)); };
  auto touch_tile = [&](uint32_t tile, uint32_t ln) { touch(touch_address(tile, ln)); };
  if constexpr (PREFETCH) {
    // tiles 0 .. 2 are loaded right away; 3 .. PF_AHEAD - 2 are touched here (the wait for the query rows
    // covers them), PF_AHEAD - 1 before the loop and PF_AHEAD + jj during tile jj
    if (ntile > 3) {
      static_for<3, PF_AHEAD - 1>([&](auto i_c) { touch_tile(tb + decltype(i_c)::value, lane); });
    }
  }

  // ---- Q fragments: B operand of S^T = K.Q^T, lane = row, 8 consecutive d per step ----
  // The operand layout gives a lane 16 bytes of its own row per step, so loading the fragments
  // straight from memory touches 32 bytes of 32 different cache lines per instruction, and the
  // four waves' 128 KiB pass through the compute unit's first-level cache several times over
  // (measured: 4.7 us until the rows had landed, 3.0 us this way).  Instead each wave brings its
  // 32 rows into LDS as whole rows, in the layout of a K tile (the tile buffers are not in use
  // yet), and reads the fragments from there the way it reads K fragments.
  u32x4 qf[NSTEP];
  {
    static_assert(4 * L::K_BYTES <= LDS_BYTES, "the four waves' query rows are staged in the tile buffers");
    lds_char* const qb = (lds_char*)smem + wave * L::K_BYTES;
    // byte offset of this lane's row (rows past the last one repeat it: finite values, and the
    // rows are masked everywhere); below 4 GiB, which the host checks
    const uint32_t rq = min(r, p.rows_total - 1u);
    const uint32_t q_row_off = ((rq / p.group * p.hq) + kvh * p.group + rq % p.group) * (uint32_t)(2 * D);
    if constexpr (L::PAD) {
      // one instruction = one row
      static_for<0, 32>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        const uint32_t off = __builtin_amdgcn_readlane(q_row_off, i);
        lds_dma_16<i * L::K_STRIDE>((const char*)p.q + off, lane * 16u, (uint32_t)(size_t)qb);
      });
    } else {
      // one instruction = 64 chunks of 16 bytes = 64 / CPR rows, swizzled like a K tile
      static_for<0, L::NBLK>([&](auto b_c) {
        constexpr int blk = decltype(b_c)::value;
        const uint32_t pch = blk * 64 + lane;
        const uint32_t rl = pch / L::CPR, pc = pch % L::CPR;
        const uint32_t c = pc ^ L::swz_k(rl);
        const uint32_t off = __shfl(q_row_off, (int)rl, 64) + c * 16u;
        lds_dma_16<blk * 1024>((const char*)p.q, off, (uint32_t)(size_t)qb);
      });
    }
    wait_vmem_all();
    const uint32_t q_lane_off = l32 * L::K_STRIDE + (L::PAD ? g2 * 16u : 0u);
    const uint32_t q_swz = L::swz_k(l32);
#pragma unroll
    for (int s = 0; s < NSTEP; ++s) {
      u32x4 raw;
      if constexpr (L::PAD) raw = *(lds_u32x4*)(qb + q_lane_off + 32 * s);
      else raw = *(lds_u32x4*)(qb + q_lane_off + ((((uint32_t)(2 * s) + g2) ^ q_swz) << 4));
      if (F16 && p.q_is_bf16) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          qf[s][e] = pack2<true>(__uint_as_float(raw[e] << 16), __uint_as_float(raw[e] & 0xffff0000u));
      } else {
        qf[s] = raw;
      }
    }
    // every wave has its fragments before the first tiles overwrite the rows
    __syncthreads();
  }

  // d-owner accumulators: o[i * NRBW + j] = O^T block (d-block dgrp*NDBW+i, row-block rgrp*NRBW+j);
  // register e of a block is d offset 8*(e>>2) + 4*g2 + (e&3), the lane is the row (l32).
  f32x16 o[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[i][e] = 0.f;
  float m_ref = -INFINITY;  // running reference max, log2 units (scale folded in)
  float m_run = -INFINITY;  // running max itself
  float x_drop = -INFINITY; // exponents below this are dropped: m_run - kDrop, relative to the reference in use
  float l_part = 0.f;       // this lane's share of the row sum (its 16 of every 32 keys),
  float l_part2 = 0.f;      // kept as two partial sums

  // per-lane LDS byte offsets of the fragment reads (everything else is a compile-time offset
  // in the padded layout, or one XOR with a per-lane constant in the swizzled one)
  const uint32_t k_lane_off = l32 * L::K_STRIDE + (L::PAD ? g2 * 16u : 0u);
  const uint32_t k_swz = L::swz_k(l32);
  const uint32_t v_row = 4u * g2 + (i16 >> 2);  // + 16*ks + 8*q, which keeps row&3
  const uint32_t v_swz = L::swz_v(v_row);
  const uint32_t v_lane_chunk = 2u * h16 + ((i16 & 3u) >> 1);
  const uint32_t v_lane_off = v_row * L::V_STRIDE + (i16 & 1u) * 8u + (L::PAD ? v_lane_chunk * 16u : 0u);

  constexpr int NLD = L::NLD;                    // load instructions per wave, tile and matrix
  constexpr int NQK = NSTEP, NPV = 2 * NACC;     // MFMAs per wave and tile in each phase
  constexpr int PFK = NQK < 4 ? NQK : 4;         // K fragment reads kept in flight ahead of the MFMAs
  constexpr int LD_EVERY = NPV / (2 * NLD);      // P.V MFMAs per tile load instruction
  static_assert(LD_EVERY >= 1 && 2 * NLD * LD_EVERY <= NPV, "tile loads must fit between the P.V MFMAs");

  // K fragment of MFMA step st: A operand, lane = key row l32, 8 consecutive d at 16*st + 8*g2
  auto k_frag = [&](lds_char* kb, int st) -> u32x4 {
    if constexpr (L::PAD) {
      return *(lds_u32x4*)(kb + k_lane_off + 32 * st);
    } else {
      const uint32_t c = (uint32_t)(2 * st) + g2;
      return *(lds_u32x4*)(kb + k_lane_off + ((c ^ k_swz) << 4));
    }
  };
  // V^T fragment for MFMA k-step ks of d-block db: k-slot j of lane half g2 is key
  // 16*ks + 8*(j>>2) + 4*g2 + (j&3), the order in which the score accumulator holds keys.
  auto v_frag = [&](lds_char* vb, int ks, uint32_t db) -> u32x4 {
    uint32_t off;
    if constexpr (L::PAD) {
      off = v_lane_off + (uint32_t)(16 * ks) * L::V_STRIDE + 64u * db;
    } else {
      const uint32_t c = 4u * db + v_lane_chunk;
      off = v_lane_off + (uint32_t)(16 * ks) * L::V_STRIDE + ((c ^ v_swz) << 4);
    }
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vb + off)));
    const u32x2 hi = __builtin_bit_cast(
        u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vb + off + 8 * L::V_STRIDE)));
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  };

  if (ntile > 0) {
    lds_char* const k0 = (lds_char*)(smem + OFF_K0);
    lds_char* const k1 = (lds_char*)(smem + OFF_K1);
    lds_char* const v0 = (lds_char*)(smem + OFF_V0);
    lds_char* const v1 = (lds_char*)(smem + OFF_V1);
    // Loads for a tile past the last one are not branched around: they fetch the last tile
    // again into a buffer nobody reads any more (or whose scores nobody uses).
    const uint32_t t_last = (te - 1u) * kBlockN;
    // (in the loop only tiles behind the workgroup's first one are loaded)
    auto k_load = [&](uint32_t t0, lds_char* buf, uint32_t ln) {
      return make_tile_load<D, false, false>(kbase, kstride_b, min(t0, t_last), 0u, p.t_all, p.ring_mask, buf, wave, ln);
    };
    auto v_load = [&](uint32_t t0, lds_char* buf, uint32_t ln) {
      return make_tile_load<D, true, false>(vbase, vstride_b, min(t0, t_last), 0u, p.t_all, p.ring_mask, buf, wave, ln);
    };
    auto k_load_first = [&](lds_char* buf) {
      return make_tile_load<D, false, true>(kbase, kstride_b, tb * kBlockN, lo_min, p.t_all, p.ring_mask, buf, wave, lane);
    };
    auto v_load_first = [&](lds_char* buf) {
      return make_tile_load<D, true, true>(vbase, vstride_b, tb * kBlockN, lo_min, p.t_all, p.ring_mask, buf, wave, lane);
    };

    // ---- softmax of one tile, cut into NCH pieces ----
    // The pieces of tile jj run between the score MFMAs of tile jj+1: one wave per SIMD issues
    // in order, so vector work only overlaps the matrix pipe if it sits between MFMAs in
    // program order.  A vector instruction that needs the result of the one before it waits
    // about 8 cycles, an independent one issues after 4, so every piece is written as a group of
    // independent operations (four scores at a time, two partial row sums).
    // State that lives across pieces:
    float tmax = 0.f, m_use = 0.f;
    float ex[4] = {0.f, 0.f, 0.f, 0.f};
    u32x4 pk4 = {0, 0, 0, 0};
    auto softmax_piece = [&](auto c_c, f32x16& s, uint32_t t0, uint32_t par) {
      constexpr int c = decltype(c_c)::value;
      if constexpr (c == 0) {
        // mask (edge tiles only)
        const bool masked = !(t0 >= lo_max && t0 + kBlockN <= hi_min);
        if (__builtin_expect(masked, 0)) {
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const uint32_t t = t0 + 8u * (e >> 2) + 4u * g2 + (e & 3);
            if (!key_visible(rb, t, p.t_clip_hi)) s[e] = -INFINITY;
          }
        }
      } else if constexpr (c == 1) {
        // tile max of the row, as a tree
        const float a0 = fmaxf(fmaxf(s[0], s[1]), s[2]), a1 = fmaxf(fmaxf(s[3], s[4]), s[5]);
        const float a2 = fmaxf(fmaxf(s[6], s[7]), s[8]), a3 = fmaxf(fmaxf(s[9], s[10]), s[11]);
        const float a4 = fmaxf(fmaxf(s[12], s[13]), s[14]);
        tmax = fmaxf(fmaxf(fmaxf(a0, a1), a2), fmaxf(fmaxf(a3, a4), s[15]));
      } else if constexpr (c == 2) {
        // online softmax with a lazily raised reference max
        tmax = max_across_halves(tmax) * p.scale_log2;
        const bool raise = __builtin_amdgcn_ballot_w64(tmax > m_ref + kTau<F16>) != 0ull;
        bool rescale = false;   // some row of the block has accumulated something that changes
        m_run = fmaxf(m_run, tmax);
        if (__builtin_expect(raise, 0)) {
          // When one row of the block has to raise its reference the whole block is rescaled anyway,
          // so every row moves its reference up to its running max: the next raise is then as far
          // away as it can be (with f16 operands, where the threshold is low, this halves the raises).
          const float m_new = fmaxf(m_ref, m_run);
          const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_ref - m_new);
          rescale = __builtin_amdgcn_ballot_w64(m_ref != -INFINITY && corr != 1.f) != 0ull;
          l_part *= corr;
          l_part2 *= corr;
          // the d owners rescale O after the barrier
          if (g2 == 0) ((float*)(smem + OFF_CORR + par * CORR_BYTES))[wave * 32u + l32] = corr;
          m_ref = m_new;
        }
        if (lane == 0) ((uint32_t*)(smem + OFF_FLAG + par * FLAG_BYTES))[wave] = rescale ? 1u : 0u;
        m_use = (m_ref == -INFINITY) ? 0.f : m_ref + kPOff<F16>;
        if constexpr (!F16) x_drop = m_run - kDrop - m_use;
      } else {
        // scores 4 q .. 4 q + 3 in two steps: (a) scale and subtract, first two exponentials;
        // (b) the other two exponentials, rounding to the MFMA operand type, and for every
        // second q the store of a k-step's B operand and its share of the row sum
        constexpr int q = (c - 3) / 2;
        if constexpr ((c - 3) % 2 == 0) {
#pragma unroll
          for (int i = 0; i < 4; ++i) ex[i] = __builtin_fmaf(s[4 * q + i], p.scale_log2, -m_use);
          const bool keep0 = F16 || ex[0] >= x_drop, keep1 = F16 || ex[1] >= x_drop;
          ex[0] = __builtin_amdgcn_exp2f(ex[0]);
          ex[1] = __builtin_amdgcn_exp2f(ex[1]);
          ex[0] = keep0 ? ex[0] : 0.f;
          ex[1] = keep1 ? ex[1] : 0.f;
        } else {
          const bool keep2 = F16 || ex[2] >= x_drop, keep3 = F16 || ex[3] >= x_drop;
          ex[2] = __builtin_amdgcn_exp2f(ex[2]);
          ex[3] = __builtin_amdgcn_exp2f(ex[3]);
          ex[2] = keep2 ? ex[2] : 0.f;
          ex[3] = keep3 ? ex[3] : 0.f;
          pk4[(2 * q) % 4] = pack2<F16>(ex[0], ex[1]);
          pk4[(2 * q + 1) % 4] = pack2<F16>(ex[2], ex[3]);
          if constexpr (q % 2 == 1) {
            // register image of the B operand of MFMA k-step q/2 for (row l32, lane half g2)
            *(lds_u32x4*)((lds_char*)(smem + OFF_P) + par * P_BYTES + (((uint32_t)(q / 2) * 4u + wave) * 64u + lane) * 16u) =
                pk4;
            // the row sum uses the rounded probabilities, the same numbers P.V multiplies
            l_part = add_pair<F16>(pk4[0], l_part);
            l_part2 = add_pair<F16>(pk4[1], l_part2);
            l_part = add_pair<F16>(pk4[2], l_part);
            l_part2 = add_pair<F16>(pk4[3], l_part2);
          }
        }
      }
    };
    constexpr int NCH = 3 + 8;   // pieces the softmax of a tile is cut into

    // S^T = K.Q^T, MFMA steps [ST0, ST1) of the tile in kb.  The K fragments of steps
    // 0 .. PFK-1 are already in (or on their way to) kf; fragment reads run PFK ahead of the
    // MFMA that consumes them.  With SOFTMAX, the softmax of the previous tile (scores in
    // s_prev) is spread over the steps below NSPLIT.  The scheduling barriers keep the
    // interleaving as written.
    constexpr int NSPLIT = NQK - PFK;   // steps before the tile's barrier; the rest need no more LDS reads
    u32x4 kf[PFK];
    auto kf_preload = [&](lds_char* kb) {
#pragma unroll
      for (int i = 0; i < PFK; ++i) kf[i] = k_frag(kb, i);
    };
    auto qk_steps = [&](auto st0_c, auto st1_c, lds_char* kb, auto softmax_c, auto wait_c, f32x16& s, f32x16& s_prev,
                        uint32_t t0_prev, uint32_t par, auto&& after) {
      constexpr bool SOFTMAX = decltype(softmax_c)::value, WAIT = decltype(wait_c)::value;
      static_for<decltype(st0_c)::value, decltype(st1_c)::value>([&](auto st_c) {
        constexpr int st = decltype(st_c)::value;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (st == 0) mfma_scores_first<F16>(s, kf[0], qf[0]);
        else if constexpr (WAIT && st == NQK - 1) mfma_scores_last<F16>(s, kf[st % PFK], qf[st]);
        else mfma_scores_acc<F16>(s, kf[st % PFK], qf[st]);
        if constexpr (st + PFK < NQK) kf[st % PFK] = k_frag(kb, st + PFK);
        if constexpr (SOFTMAX && st < NSPLIT) {
          // pieces [st NCH / NSPLIT, (st+1) NCH / NSPLIT) follow MFMA st
          static_for<st * NCH / (NSPLIT > 0 ? NSPLIT : 1), (st + 1) * NCH / (NSPLIT > 0 ? NSPLIT : 1)>(
              [&](auto c_c) {
                softmax_piece(c_c, s_prev, t0_prev, par); });
        }
        after(st_c);
      });
      __builtin_amdgcn_sched_barrier(0);
    };
    using I0 = std::integral_constant<int, 0>;
    using ISPLIT = std::integral_constant<int, NSPLIT>;
    using IQK = std::integral_constant<int, NQK>;

    issue_tile<D, false>(k_load_first(k0), wave, lane);
    issue_tile<D, false>(k_load((tb + 1) * kBlockN, k1, lane), wave, lane);
    issue_tile<D, true>(v_load_first(v0), wave, lane);
    wait_vmem_all();
    __syncthreads();
    // s_a: scores of the tile whose softmax is due; s_b: scores being accumulated for the next.
    // s_b is copied into s_a during each tile's P.V by copy_scores_part(), not by an assignment:
    // the compiler would merge the two and place its own copy right behind (or before) the last
    // score MFMA, reading the registers before the MFMA has written them.
    f32x16 s_a, s_b;
    kf_preload(k0);
    auto nothing = [](auto) {};
    qk_steps(I0{}, IQK{}, k0, std::false_type{}, std::true_type{}, s_a, s_b, 0u, 0u, nothing);
    __syncthreads();   // every wave is done with K(tb): its buffer takes K(tb+2)
    issue_tile<D, false>(k_load((tb + 2) * kBlockN, k0, lane), wave, lane);
    if constexpr (PREFETCH) touch_tile(tb + PF_AHEAD - 1, lane);
    kf_preload(k1);

    for (uint32_t jj = 0; jj < ntile; ++jj) {
      const uint32_t par = jj & 1u;
      const uint32_t t0 = (tb + jj) * kBlockN;
      lds_char* const kb_next = par ? k0 : k1;    // holds K(jj+1); takes K(jj+3) after the barrier
      lds_char* const kb_next2 = par ? k1 : k0;   // holds K(jj+2) once the barrier is passed
      lds_char* const vb_cur = par ? v1 : v0;     // holds V(jj)
      lds_char* const vb_free = par ? v0 : v1;    // takes V(jj+1)

      // ---- row-owner role: scores of the next tile, softmax of this one ----
      // (K(jj+1) has landed everywhere: its loads were waited for before the previous barrier,
      // and its first fragments were read during the previous tile's P.V.  For the last tile
      // the "next" scores are those of a repeated tile and go unused.)
      if constexpr (NSPLIT == 0)
        static_for<0, NCH>([&](auto c_c) { softmax_piece(c_c, s_a, t0, par); });
      qk_steps(I0{}, ISPLIT{}, kb_next, std::true_type{}, std::false_type{}, s_b, s_a, t0, par, nothing);
      // The one barrier of the tile.  Before it: this wave's loads of V(jj) and K(jj+2), issued
      // during the previous tile's P.V, have landed, its P is written and the last K fragments
      // of the tile are in registers (the barrier's fence waits for all three).  After it: P,
      // the rescale words and V(jj) of this tile are visible to the d owners; every wave is done
      // reading K(jj+1), V(jj-1) and the previous tile's P (which has its own buffer), so their
      // buffers can be refilled.
      if constexpr (PREFETCH) wait_vmem_but<1>();   // (the touch of the previous tile may be on its way)
      else wait_vmem_all();
      __syncthreads();

      // ---- d-owner role ----
      lds_char* const pbuf = (lds_char*)(smem + OFF_P) + par * P_BYTES;
      auto p_frag = [&](int ks, uint32_t rbk) -> u32x4 {
        return *(lds_u32x4*)(pbuf + (((uint32_t)ks * 4u + rbk) * 64u + lane) * 16u);
      };
      constexpr int NVF = 2 * NDBW;                    // V^T fragments per tile and wave
      constexpr int PFV = NVF - 1 < 3 ? NVF - 1 : 3;   // fragment reads in flight ahead of the MFMAs
      auto v_frag_n = [&](int f) { return v_frag(vb_cur, f / NDBW, dgrp * NDBW + f % NDBW); };
      // first reads of the P.V phase; the last score MFMAs of the next tile cover their latency
      u32x4 fl = *(lds_u32x4*)((lds_char*)(smem + OFF_FLAG) + par * FLAG_BYTES);
      u32x4 pbv[NRBW];
#pragma unroll
      for (int j = 0; j < NRBW; ++j) pbv[j] = p_frag(0, rgrp * NRBW + j);
      u32x4 va[PFV + 1];
#pragma unroll
      for (int f = 0; f <= PFV; ++f) va[f] = v_frag_n(f);
      // The descriptors of this tile's global loads are worked out between those MFMAs, not
      // behind the branch below, where nothing would overlap them.  The per-lane offsets are
      // re-derived in every iteration: hoisted out of the loop they would cost more live VGPRs
      // than this kernel has.
      const uint32_t lane_l = opaque(lane);
      TileLoad next_v, next_k;
      Touch next_touch{nullptr, 0u};
      qk_steps(ISPLIT{}, IQK{}, kb_next, std::true_type{}, std::false_type{}, s_b, s_a, t0, par, [&](auto st_c) {
        constexpr int st = decltype(st_c)::value;
        if constexpr (st == NSPLIT) next_v = pinned(v_load(t0 + kBlockN, vb_free, lane_l));
        if constexpr (st == (NSPLIT + 1 < NQK ? NSPLIT + 1 : NSPLIT))
          next_k = pinned(k_load(t0 + 3 * kBlockN, kb_next, lane_l));
      });
      // keep every use of the flags behind those MFMAs: they are what hides the latency of the read
      fl = opaque4(fl);
      if (__builtin_expect(__builtin_amdgcn_readfirstlane(fl[0] | fl[1] | fl[2] | fl[3]) != 0u, 0)) {
        // O lives in accumulator registers, which only MFMA and the accvgpr moves can touch.
        // Spelling the multiply out keeps the values in that register class on both sides of
        // this rarely taken branch; a plain `o[i] *= corr` makes the allocator shuttle all of
        // O through VGPRs and spill.
        const float* const scorr = (const float*)(smem + OFF_CORR + par * CORR_BYTES);
#pragma unroll
        for (int j = 0; j < NRBW; ++j) {
          const uint32_t rbk = rgrp * NRBW + j;
          if (__builtin_amdgcn_readfirstlane(fl[rbk]) == 0u) continue;
          const float corr = scorr[rbk * 32u + l32];
#pragma unroll
          for (int i = 0; i < NDBW; ++i)
#pragma unroll
            for (int e = 0; e < 16; e += 8) {
              f32x16& a = o[i * NRBW + j];
              float x0 = a[e], x1 = a[e + 1], x2 = a[e + 2], x3 = a[e + 3];
              float x4 = a[e + 4], x5 = a[e + 5], x6 = a[e + 6], x7 = a[e + 7];
              scale_acc8(x0, x1, x2, x3, x4, x5, x6, x7, corr);
              a[e] = x0;
              a[e + 1] = x1;
              a[e + 2] = x2;
              a[e + 3] = x3;
              a[e + 4] = x4;
              a[e + 5] = x5;
              a[e + 6] = x6;
              a[e + 7] = x7;
            }
          scale_acc_done();
        }
      }
      // O^T += V^T . P^T: per k-step, NDBW V^T fragments x NRBW P fragments.  The P fragments
      // of a k-step stay in registers for the whole step; V^T fragments are fetched PFV ahead
      // of the one that multiplies, and each P fragment of k-step 1 replaces its k-step 0
      // counterpart right after that one's last use.  Spread between the MFMAs: the global
      // loads of V(jj+1) and K(jj+3), alternating; the copy of the next tile's scores to where
      // the softmax expects them; behind the last MFMAs, the reads of the first K fragments of
      // tile jj+2 (pinned there: at the loop end the compiler would move them to the top of the
      // next iteration, in front of the MFMAs that wait for them).
      constexpr int COPY_AT = NPV >= 16 ? NPV / 2 : 0;   // MFMA index after which the copy starts
      static_for<0, NVF>([&](auto f_c) {
        constexpr int f = decltype(f_c)::value, ks = f / NDBW, i = f % NDBW;
        static_for<0, NRBW>([&](auto j_c) {
          constexpr int j = decltype(j_c)::value, n = f * NRBW + j;   // n: MFMA index within the tile
          __builtin_amdgcn_sched_barrier(0);
          o[i * NRBW + j] = mfma16<F16>(va[f % (PFV + 1)], pbv[j], o[i * NRBW + j]);
          if constexpr (ks == 0 && i == NDBW - 1) pbv[j] = p_frag(1, rgrp * NRBW + j);
          if constexpr (n % LD_EVERY == 0 && n / LD_EVERY < 2 * NLD) {
            constexpr int q = n / LD_EVERY;
            if constexpr (q % 2 == 0) issue_tile_part<D, true, q / 2>(next_v, wave, lane_l);
            else issue_tile_part<D, false, q / 2>(next_k, wave, lane_l);
          }
          if constexpr (NPV >= 16 && n >= COPY_AT && n < COPY_AT + 8) copy_scores_part<n - COPY_AT>(s_a, s_b);
          if constexpr (NPV >= PFK && n >= NPV - PFK) kf[n - (NPV - PFK)] = k_frag(kb_next2, n - (NPV - PFK));
          // the touch itself behind the tile's last load, its address worked out a few MFMAs earlier
          // (behind the last MFMA nothing would overlap the arithmetic)
          if constexpr (PREFETCH && n == NPV - 6) {
            next_touch = touch_address(tb + jj + PF_AHEAD, lane_l);
            uint64_t b = (uint64_t)next_touch.base;
            uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
            uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
            asm volatile("" : "+s"(lo), "+s"(hi), "+v"(next_touch.voff));
            next_touch.base = (const char*)(((uint64_t)hi << 32) | lo);
          }
          if constexpr (PREFETCH && n == NPV - 1) {
            static_assert(!PREFETCH || (2 * NLD - 1) * LD_EVERY < NPV - 1, "the touch follows the tile's last load");
            touch(next_touch);
          }
        });
        if constexpr (f + PFV + 1 < NVF) va[f % (PFV + 1)] = v_frag_n(f + PFV + 1);
      });
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (NPV < 16) static_for<0, 8>([&](auto i_c) { copy_scores_part<decltype(i_c)::value>(s_a, s_b); });
      if constexpr (NPV < PFK) kf_preload(kb_next2);
    }
    // the loads issued for tiles after the last one must not outlive this workgroup's LDS
    wait_vmem_all();
  }

  // ---- epilogue ----
  // row owners publish (m, l) of their rows; d owners normalise and store their slice of O
  const float l_tot = sum_across_halves(l_part + l_part2);
  const float m_pub = m_ref + kPOff<F16>;   // the exponent the sums are relative to
  // first partial row of this workgroup; partial rows and their (m, l) are written through (wt_store.h)
  const size_t wg_prow0 = ((size_t)split * p.hkv + kvh) * p.rows_pad + row0;
  __syncthreads();   // the last tile's readers are done with LDS
  if (g2 == 0) {
    sml[(wave * 32u + l32) * 2u] = m_pub;
    sml[(wave * 32u + l32) * 2u + 1u] = l_tot;
    if (p.n_splits > 1) {
      const u32x2 ml2 = {__float_as_uint(m_pub), __float_as_uint(l_tot)};
      wt_store8(wt_window(p.part_ml + wg_prow0 * 2), (r - row0) * 8u, ml2);
    } else if (row_ok) {
      if (p.lse) p.lse[(size_t)tok * p.hq + qh] = l_tot > 0.f ? m_pub * kLn2 + __logf(l_tot) : -INFINITY;
      if (p.dbg && !(l_tot > 0.f)) dbg_report(p.dbg, DBG_ERR_SOFTMAX_NORM_ZERO, DBG_KERNEL_ATTENTION, (tok << 16) | qh, (tok << 16) | qh);
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NRBW; ++j) {
    const uint32_t rbk = rgrp * NRBW + j;
    const uint32_t rr = row0 + rbk * 32u + l32;
    if (p.n_splits > 1 && p.part_half) {
      // Same route through LDS as below, for partial rows kept as f16: each accumulator is divided
      // by the split's row sum first (a weighted mean of V rows: no larger than the largest |V|),
      // and the merge weighs the rows by l 2^(m - m_max) instead of 2^(m - m_max).
      constexpr int STG_ROW = NDBW * 64 + 16;             // bytes of a staged row slice, padded
      constexpr int LPR = NDBW * 4, RPI = 64 / LPR;       // lanes per row slice (16 B each), rows per store
      lds_char* const stg = (lds_char*)smem + wave * (32 * STG_ROW);
      const float l_row = sml[(rbk * 32u + l32) * 2u + 1u];
      const float inv = l_row > 0.f ? 1.f / l_row : 0.f;
#pragma unroll
      for (int i = 0; i < NDBW; ++i) {
        const f32x16& a = o[i * NRBW + j];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const f32x4 x = acc_read4<D == 512>(a, 4 * q4);
          u32x2 h2;
          h2[0] = pack2<true>(sat_f16(x[0] * inv), sat_f16(x[1] * inv));
          h2[1] = pack2<true>(sat_f16(x[2] * inv), sat_f16(x[3] * inv));
          *(__attribute__((address_space(3))) u32x2*)(stg + l32 * STG_ROW + (32 * i + 8 * q4 + 4 * g2) * 2) = h2;
        }
      }
      const auto win = wt_window((const uint16_t*)p.part_o + wg_prow0 * D);
      const uint32_t po = ((rbk * 32u) * D + 32u * (dgrp * NDBW) + (lane % LPR) * 8u) * 2u;   // bytes
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const uint32_t rl = it * RPI + lane / LPR;        // row within the block
        const u32x4 v4 = *(lds_u32x4*)(stg + rl * STG_ROW + (lane % LPR) * 16);
        wt_store16(win, po + rl * (D * 2u), v4);
      }
      continue;
    }
    if (p.n_splits > 1) {
      // The accumulators hold a row per lane: stored as they are, every instruction would
      // scatter 32-byte pieces over 32 rows.  Each wave passes its 32 rows x (NDBW x 32) d through
      // its own piece of LDS (the tile buffers are free now) and writes whole rows instead.
      constexpr int STG_ROW = NDBW * 128 + 16;            // bytes; the pad keeps the 16-byte writes of 8 rows apart
      constexpr int LPR = NDBW * 8, RPI = 64 / LPR;       // lanes per row slice, rows per store instruction
      static_assert(4 * 32 * STG_ROW <= OFF_ML, "staging must not reach the (m, l) words");
      lds_char* const stg = (lds_char*)smem + wave * (32 * STG_ROW);
#pragma unroll
      for (int i = 0; i < NDBW; ++i) {
        const f32x16& a = o[i * NRBW + j];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const f32x4 v4 = acc_read4<D == 512>(a, 4 * q4);
          *(__attribute__((address_space(3))) f32x4*)(stg + l32 * STG_ROW + (32 * i + 8 * q4 + 4 * g2) * 4) = v4;
        }
      }
      const auto win = wt_window(p.part_o + wg_prow0 * D);
      const uint32_t po = ((rbk * 32u) * D + 32u * (dgrp * NDBW) + (lane % LPR) * 4u) * 4u;   // bytes
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const uint32_t rl = it * RPI + lane / LPR;        // row within the block
        const u32x4 v4 = *(lds_u32x4*)(stg + rl * STG_ROW + (lane % LPR) * 16);
        wt_store16(win, po + rl * (D * 4u), v4);
      }
      continue;
    }
    if (rr >= p.rows_total) continue;
    const float l_row = sml[(rbk * 32u + l32) * 2u + 1u];
    const float inv = l_row > 0.f ? 1.f / l_row : 0.f;
    const uint32_t tok_o = rr / p.group, qh_o = kvh * p.group + rr % p.group;
#pragma unroll
    for (int i = 0; i < NDBW; ++i) {
      const size_t idx0 = ((size_t)tok_o * p.hq + qh_o) * D + 32u * (dgrp * NDBW + i) + 4u * g2;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const f32x16& a = o[i * NRBW + j];
        const f32x4 x = acc_read4<D == 512>(a, 4 * q4);
        const float y0 = x[0] * inv, y1 = x[1] * inv;
        const float y2 = x[2] * inv, y3 = x[3] * inv;
        const size_t idx = idx0 + 8 * q4;
        if (p.dbg && !(fabsf(y0) + fabsf(y1) + fabsf(y2) + fabsf(y3) <= 3.402823466e38f))   // NaN or infinity
          dbg_report(p.dbg, DBG_ERR_NONFINITE, DBG_KERNEL_ATTENTION, (tok_o << 16) | qh_o, 32u * (dgrp * NDBW + i) + 4u * g2 + 8u * q4);
        if (p.out_dtype == DT_F32) {
          f32x4 v4 = {y0, y1, y2, y3};
          *(f32x4*)((float*)p.out + idx) = v4;
        } else {
          u32x2 pk;
          if (p.out_trunc) {
            pk[0] = (__float_as_uint(y0) >> 16) | (__float_as_uint(y1) & 0xffff0000u);
            pk[1] = (__float_as_uint(y2) >> 16) | (__float_as_uint(y3) & 0xffff0000u);
          } else {
            pk[0] = pack2<false>(y0, y1);
            pk[1] = pack2<false>(y2, y3);
          }
          *(u32x2*)((uint16_t*)p.out + idx) = pk;
        }
      }
    }
  }
}

template <int D, bool F16>
hipError_t launch_one(const AttnParams& p, hipStream_t s) {
  const uint32_t nstream = p.hkv * p.n_splits;
  const uint32_t grid = ((nstream * p.n_mtiles + 7u) / 8u) * 8u;
  if constexpr (D == 512) {
    if (p.touch_ahead) {
      hipLaunchKernelGGL((attn_mfma_kernel<D, F16, true>), dim3(grid), dim3(256), 0, s, p);
      return hipGetLastError();
    }
  }
  hipLaunchKernelGGL((attn_mfma_kernel<D, F16, false>), dim3(grid), dim3(256), 0, s, p);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_attn_mfma(const AttnParams& p, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s) {
  const bool f16 = kv_dtype == DT_F16;
  switch (head_dim) {
    case 32: return f16 ? launch_one<32, true>(p, s) : launch_one<32, false>(p, s);
    case 64: return f16 ? launch_one<64, true>(p, s) : launch_one<64, false>(p, s);
    case 128: return f16 ? launch_one<128, true>(p, s) : launch_one<128, false>(p, s);
    case 256: return f16 ? launch_one<256, true>(p, s) : launch_one<256, false>(p, s);
    case 512: return f16 ? launch_one<512, true>(p, s) : launch_one<512, false>(p, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace dg
