// Denoise-step attention on MFMA for gfx950 (MI355X).
//
// One workgroup (4 waves) owns 128 stacked query rows of one KV head and one key-range split.
// Stacked row = canvas_row * group + head_in_group, so the `group` query heads that share a KV
// head are the M dimension of the same tile and K/V are read once for all of them.
//
// Per 32-key tile:
//   S^T = K . Q^T   v_mfma_f32_32x32x16 (bf16 or f16): A = K rows from LDS (ds_read_b128),
//                   B = Q held in registers for the whole kernel.  Output lane = query row,
//                   output registers = keys, so row max / row sum are per-lane scalars.
//   P   = exp2(S*c - m)  in registers; its register layout already is the B operand of the
//                   next MFMA when keys are taken in the order the accumulator holds them.
//   O^T += V^T . P^T  A = V^T fragments read with ds_read_b64_tr_b16 from the row-major V tile.
// K and V tiles arrive by 16-byte direct-to-LDS loads, double buffered: tile j+2 of K and
// tile j+1 of V are in flight while tile j+1 of K and tile j of V are consumed.  QK^T of the
// next tile is issued before the softmax of the current one so the matrix pipe has work
// while the VALU computes exponentials.  The running max is only raised (and O rescaled)
// when some row's tile max exceeds it by more than 2^kTau, which in steady state is never.
#include "attn_params.h"

namespace dg {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
typedef __attribute__((address_space(3))) i16x4 lds_i16x4;
typedef __attribute__((address_space(1))) const void gbl_void;
typedef __attribute__((address_space(3))) void lds_void;

constexpr float kTau = 8.0f;  // log2 units: P never exceeds 2^8 before a rescale

// Optional per-phase cycle accounting (development builds only): every wave sums the cycles
// it spends in each phase of the tile loop and stores the sums at the end.
#ifdef DG_ATTN_PHASE_TIMING
#define DG_PHASE_DECL unsigned long long ph_t = clock64(), ph_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#define DG_PHASE(i)                          \
  {                                          \
    const unsigned long long now = clock64(); \
    ph_acc[i] += now - ph_t;                 \
    ph_t = now;                              \
  }
#define DG_PHASE_STORE                                                                    \
  if (p.phase_cycles && lane == 0) {                                                      \
    for (int i = 0; i < 8; ++i) p.phase_cycles[((size_t)blockIdx.x * 4 + wave) * 8 + i] = ph_acc[i]; \
  }
#else
#define DG_PHASE_DECL
#define DG_PHASE(i)
#define DG_PHASE_STORE
#endif

template <bool F16>
__device__ __forceinline__ f32x16 mfma16(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (F16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  }
}

// two floats -> packed pair of E (round to nearest even), low half = a
template <bool F16>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  if constexpr (F16) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, v);
  } else {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    b2 v = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, v);
  }
}
template <bool F16>
__device__ __forceinline__ float unpack_lo(uint32_t u) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)(u & 0xffffu));
  else return __uint_as_float(u << 16);
}
template <bool F16>
__device__ __forceinline__ float unpack_hi(uint32_t u) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16));
  else return __uint_as_float(u & 0xffff0000u);
}

// s_waitcnt vmcnt(0) as a builtin, so that the compiler's own wait-count bookkeeping sees it
// (gfx9 encoding: vmcnt = bits 3:0 and 15:14, expcnt = 6:4, lgkmcnt = 11:8; the other two
// counters are left at their maxima).
__device__ __forceinline__ void wait_vmem_all() {
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");
}

// value of lane l combined with lane l^32
__device__ __forceinline__ float max_across_halves(float x) {
  const uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_across_halves(float x) {
  const uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// 16-byte chunk swizzles of a tile row (CPR = chunks per row).  K is read as 32 rows x one
// chunk per half-wave, V as 8 rows x 4 chunks per transpose read; both patterns then fall
// on distinct banks.
template <int CPR>
__device__ __forceinline__ uint32_t swz_k(uint32_t row) {
  if constexpr (CPR >= 16) return row & 15u;
  else return (row / (16 / CPR)) & (CPR - 1);
}
template <int CPR>
__device__ __forceinline__ uint32_t swz_v(uint32_t row) {
  return ((row & 3u) << 2) & (CPR - 1);
}

// One 32-key tile's direct-to-LDS loads, described once per tile and issued one wave
// instruction at a time so the issue slots can be spread between MFMAs.  Each instruction
// fills one contiguous KiB of LDS (64 lanes x 16 B); the swizzle is applied by choosing which
// global chunk each lane fetches.  Keys past t_all re-read key t_all-1 (finite, masked later).
struct TileLoad {
  const char* base;   // head base + slot(t0) * row stride (wave-uniform)
  uint32_t stride_b;  // bytes between key rows
  uint32_t rmax;      // last valid row of the tile
  uint32_t lds;       // LDS byte address of the destination buffer
  bool on;
};

__device__ __forceinline__ TileLoad make_tile_load(const char* head_base, int64_t tok_stride_b, uint32_t t0,
                                                   uint32_t t_all, uint32_t ring_mask, lds_char* buf, bool on) {
  TileLoad tl;
  tl.base = head_base + (int64_t)kv_slot(ring_mask, t0) * tok_stride_b;
  tl.stride_b = (uint32_t)tok_stride_b;
  tl.rmax = t_all - 1u - t0;
  tl.lds = (uint32_t)(size_t)buf;
  tl.on = on;
  return tl;
}

// The load is written as assembly on purpose: the compiler orders every LDS read after a
// direct-to-LDS load it knows about with s_waitcnt vmcnt(0), which would expose the whole
// fetch latency once per tile.  The kernel waits for these loads itself, at the top of the
// tile loop, one iteration after they were issued.
template <int D, bool IS_V>
__device__ __forceinline__ void issue_tile_part(const TileLoad& tl, int k, uint32_t wave, uint32_t lane) {
  constexpr int CPR = D / 8;
  constexpr int NBLK = 32 * CPR / 64;
  if (!tl.on) return;
  const uint32_t blk = k * 4 + wave;
  if (NBLK < 4 && blk >= (uint32_t)NBLK) return;
  const uint32_t pch = blk * 64 + lane;
  const uint32_t r = pch / CPR, pc = pch % CPR;
  const uint32_t c = pc ^ (IS_V ? swz_v<CPR>(r) : swz_k<CPR>(r));
  const uint32_t voff = min(r, tl.rmax) * tl.stride_b + c * 16u;
  // both are wave-uniform by construction; readfirstlane tells the compiler so
  const uint32_t dst = __builtin_amdgcn_readfirstlane(tl.lds + blk * 1024u);
  const uint64_t b = (uint64_t)tl.base;
  // (readfirstlane returns a signed int: without the casts the low half would be sign-extended
  // over the high half)
  const uint64_t base = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32)) << 32) |
                        (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff), "s"(base)
               : "memory");
}

template <int D, bool IS_V>
__device__ __forceinline__ void issue_tile(const TileLoad& tl, uint32_t wave, uint32_t lane) {
  constexpr int NLD = (32 * (D / 8) / 64 + 3) / 4;
#pragma unroll
  for (int k = 0; k < NLD; ++k) issue_tile_part<D, IS_V>(tl, k, wave, lane);
}

// PIPE: issue Q.K^T of tile j+1 before the softmax of tile j (needs a second score tile in
// registers; used where the register file has room for it).
template <int D, bool F16, bool PIPE>
__global__ void __launch_bounds__(256) attn_mfma_kernel(const AttnParams p) {
  constexpr int CPR = D / 8, ROWB = 2 * D, TILEB = kBlockN * ROWB, NSTEP = D / 16, NDB = D / 32;
  __shared__ __attribute__((aligned(1024))) char sk0[TILEB];
  __shared__ __attribute__((aligned(1024))) char sk1[TILEB];
  __shared__ __attribute__((aligned(1024))) char sv0[TILEB];
  __shared__ __attribute__((aligned(1024))) char sv1[TILEB];

  // ---- which (KV head, split, row tile) this workgroup owns ----
  // Workgroup ids go round-robin over the 8 XCDs.  All row tiles of one (KV head, split)
  // stream the same keys, so they are given ids with the same id%8 and share one L2.
  const uint32_t nstream = p.hkv * p.n_splits;
  const uint32_t wg = blockIdx.x;
  const uint32_t slot_in_xcd = wg >> 3;
  const uint32_t stream = (slot_in_xcd / p.n_mtiles) * 8u + (wg & 7u);
  const uint32_t mt = slot_in_xcd % p.n_mtiles;
  if (stream >= nstream) return;
  const uint32_t kvh = stream / p.n_splits, split = stream % p.n_splits;

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t g2 = lane >> 5, l32 = lane & 31u, h16 = (lane >> 4) & 1u, i16 = lane & 15u;

  // ---- this lane's query row and its key bounds ----
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
    if (tok_a < p.causal_rows && p.extra_lo < p.t_all) hi_max = p.t_all;
    if (row0 + kBlockM > p.rows_total) hi_min = 0;  // ragged tile: always take the masked path
  }
  const uint32_t split_begin = p.tile_first + split * p.tiles_per_split;
  const uint32_t split_end = min(split_begin + p.tiles_per_split, p.tile_end);
  const uint32_t tb = max(lo_min / kBlockN, split_begin);
  const uint32_t te = min((hi_max + kBlockN - 1) / kBlockN, split_end);
  const uint32_t ntile = te > tb ? te - tb : 0u;

  // ---- Q fragments: B operand of S^T = K.Q^T, lane = row, 8 consecutive d per step ----
  u32x4 qf[NSTEP];
  {
    const size_t qoff = ((size_t)tok * p.hq + qh) * D + 8u * g2;
    if (F16 && p.q_is_bf16) {
      const uint16_t* qp = (const uint16_t*)p.q + qoff;
#pragma unroll
      for (int s = 0; s < NSTEP; ++s) {
        u32x4 raw = row_ok ? *(const u32x4*)(qp + 16 * s) : u32x4{0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 4; ++e)
          qf[s][e] = pack2<true>(__uint_as_float(raw[e] << 16), __uint_as_float(raw[e] & 0xffff0000u));
      }
    } else {
      const uint16_t* qp = (const uint16_t*)p.q + qoff;
#pragma unroll
      for (int s = 0; s < NSTEP; ++s) qf[s] = row_ok ? *(const u32x4*)(qp + 16 * s) : u32x4{0, 0, 0, 0};
    }
  }

  f32x16 o[NDB];
#pragma unroll
  for (int i = 0; i < NDB; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[i][e] = 0.f;
  float m_ref = -INFINITY;  // running reference max, log2 units (scale folded in)
  float l_part = 0.f;       // this lane's share of the row sum (its 16 of every 32 keys)

  const char* kbase = (const char*)p.k + (int64_t)kvh * p.k_head_stride * 2;
  const char* vbase = (const char*)p.v + (int64_t)kvh * p.v_head_stride * 2;
  const int64_t kstride_b = p.k_tok_stride * 2, vstride_b = p.v_tok_stride * 2;

  // per-lane LDS byte offsets of the fragment reads
  const uint32_t k_row_off = l32 * ROWB;
  const uint32_t k_swz = swz_k<CPR>(l32);
  const uint32_t v_row = 4u * g2 + (i16 >> 2);  // + 16*ks + 8*q, which keeps row&3
  const uint32_t v_swz = swz_v<CPR>(v_row);
  const uint32_t v_lane_chunk = 2u * h16 + ((i16 & 3u) >> 1);
  const uint32_t v_lane_off = v_row * ROWB + (i16 & 1u) * 8u;

  constexpr int NLD = (32 * CPR / 64 + 3) / 4;   // load instructions per wave, tile and matrix
  constexpr int NQK = NSTEP, NPV = 2 * NDB;      // MFMAs per tile in each phase
  constexpr int PFK = NQK < 4 ? NQK : 4;         // fragment reads kept in flight ahead of the MFMAs
  constexpr int PFV = NPV < 4 ? NPV : 4;
  constexpr int LDK_EVERY = NQK / NLD, LDV_EVERY = NPV / NLD;

  auto k_frag = [&](lds_char* kb, int st) -> u32x4 {
    const uint32_t c = (uint32_t)(2 * st) + g2;
    return *(lds_u32x4*)(kb + k_row_off + ((c ^ k_swz) << 4));
  };
  auto v_frag = [&](lds_char* vb, int i) -> u32x4 {   // i = ks * NDB + db
    const int ks = i / NDB, db = i % NDB;
    const uint32_t c = (uint32_t)(4 * db) + v_lane_chunk;
    const uint32_t off = v_lane_off + (uint32_t)(16 * ks) * ROWB + ((c ^ v_swz) << 4);
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vb + off)));
    const u32x2 hi =
        __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vb + off + 8 * ROWB)));
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  };

  // S^T = K.Q^T for one tile.  PFK fragment reads run ahead of the MFMA that consumes them and
  // the next K tile's global loads are issued one instruction every LDK_EVERY MFMAs; the
  // scheduling barriers keep that interleaving.
  auto qk_tile = [&](lds_char* kb, const TileLoad& next_k, uint32_t ld_lane) -> f32x16 {
    f32x16 s;
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.f;
    u32x4 kf[PFK];
#pragma unroll
    for (int i = 0; i < PFK; ++i) kf[i] = k_frag(kb, i);
#pragma unroll
    for (int st = 0; st < NQK; ++st) {
      __builtin_amdgcn_sched_barrier(0);
      s = mfma16<F16>(kf[st % PFK], qf[st], s);
      if (st + PFK < NQK) kf[st % PFK] = k_frag(kb, st + PFK);
      if (st % LDK_EVERY == 0 && st / LDK_EVERY < NLD) issue_tile_part<D, false>(next_k, st / LDK_EVERY, wave, ld_lane);
    }
    __builtin_amdgcn_sched_barrier(0);
    return s;
  };

  DG_PHASE_DECL
  if (ntile > 0) {
    lds_char* const k0 = (lds_char*)sk0;
    lds_char* const k1 = (lds_char*)sk1;
    lds_char* const v0 = (lds_char*)sv0;
    lds_char* const v1 = (lds_char*)sv1;
    const TileLoad none = make_tile_load(kbase, kstride_b, tb * kBlockN, p.t_all, p.ring_mask, k0, false);

    issue_tile<D, false>(make_tile_load(kbase, kstride_b, tb * kBlockN, p.t_all, p.ring_mask, k0, true), wave, lane);
    if (ntile > 1)
      issue_tile<D, false>(make_tile_load(kbase, kstride_b, (tb + 1) * kBlockN, p.t_all, p.ring_mask, k1, true), wave, lane);
    issue_tile<D, true>(make_tile_load(vbase, vstride_b, tb * kBlockN, p.t_all, p.ring_mask, v0, true), wave, lane);
    wait_vmem_all();
    __syncthreads();
    f32x16 s_cur;
    if constexpr (PIPE) {
      // K(tb+2) goes where K(tb) sits, so it cannot be issued before this first tile is consumed
      s_cur = qk_tile(k0, none, lane);
    }
    DG_PHASE(0)

    for (uint32_t jj = 0; jj < ntile; ++jj) {
      const uint32_t t0 = (tb + jj) * kBlockN;
      lds_char* const kb_even = (jj & 1u) ? k1 : k0;   // holds K(jj)
      lds_char* const kb_odd = (jj & 1u) ? k0 : k1;    // holds K(jj+1)
      lds_char* const vb_cur = (jj & 1u) ? v1 : v0;    // holds V(jj)
      lds_char* const vb_free = (jj & 1u) ? v0 : v1;   // refill with V(jj+1)

      // The tiles this iteration reads have landed everywhere, and every wave is done with
      // the buffers this iteration refills.
      wait_vmem_all();
      DG_PHASE(1)
      __syncthreads();
      DG_PHASE(2)
      // Re-derive the per-lane global offsets of the tile loads inside every iteration: hoisted
      // out of the loop they would cost sixteen more live VGPRs than this kernel has.
      uint32_t lane_l = lane;
      asm volatile("" : "+v"(lane_l));
      // PIPE: K(jj) was consumed one iteration ago, its buffer takes K(jj+2).
      // otherwise: K(jj+1) goes to the other buffer (the prologue already fetched K(tb+1)).
      const TileLoad next_k =
          PIPE ? make_tile_load(kbase, kstride_b, t0 + 2 * kBlockN, p.t_all, p.ring_mask, kb_even, jj + 2 < ntile)
               : make_tile_load(kbase, kstride_b, t0 + kBlockN, p.t_all, p.ring_mask, kb_odd,
                                jj >= 1 && jj + 1 < ntile);
      const TileLoad next_v =
          make_tile_load(vbase, vstride_b, t0 + kBlockN, p.t_all, p.ring_mask, vb_free, jj + 1 < ntile);
      DG_PHASE(3)
      f32x16 s_next;
      if constexpr (PIPE) {
        if (jj + 1 < ntile) s_next = qk_tile(kb_odd, next_k, lane_l);
      } else {
        s_cur = qk_tile(kb_even, next_k, lane_l);
      }
#ifdef DG_ATTN_PHASE_TIMING
      asm volatile("s_nop 0" ::"v"(s_cur[0]), "v"(s_cur[15]));  // the scores have to exist before the clock is read
#endif
      DG_PHASE(4)

      // ---- mask (edge tiles only) ----
      const bool masked = !(t0 >= lo_max && t0 + kBlockN <= hi_min);
      if (masked) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const uint32_t t = t0 + 8u * (e >> 2) + 4u * g2 + (e & 3);
          if (!key_visible(rb, t, p.t_all)) s_cur[e] = -INFINITY;
        }
      }
      // ---- online softmax with a lazily raised reference max ----
      float tmax = s_cur[0];
#pragma unroll
      for (int e = 1; e < 16; ++e) tmax = fmaxf(tmax, s_cur[e]);
      tmax = max_across_halves(tmax) * p.scale_log2;
      if (__builtin_amdgcn_ballot_w64(tmax > m_ref + kTau) != 0ull) {
        const float m_new = fmaxf(m_ref, tmax);
        const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_ref - m_new);
        l_part *= corr;
        // O lives in accumulator registers, which only MFMA and the accvgpr moves can touch.
        // Spelling the multiply out keeps the values in that register class on both sides
        // of this rarely taken branch; a plain `o[i] *= corr` makes the allocator shuttle
        // all of O through VGPRs and spill.
#pragma unroll
        for (int i = 0; i < NDB; ++i)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            float tmp;
            float x = o[i][e];
            asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\tv_accvgpr_write_b32 %0, %1"
                         : "+a"(x), "=&v"(tmp)
                         : "v"(corr));
            o[i][e] = x;
          }
        m_ref = m_new;
      }
      const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref;
      u32x4 pf[2];
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_cur[e], p.scale_log2, -m_use));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_cur[e + 1], p.scale_log2, -m_use));
        const uint32_t pk = pack2<F16>(p0, p1);
        pf[e >> 3][(e >> 1) & 3] = pk;
        // the row sum uses the rounded probabilities, the same numbers P.V multiplies
        l_part += unpack_lo<F16>(pk) + unpack_hi<F16>(pk);
      }
      DG_PHASE(5)

      // ---- O^T += V^T . P^T, V(jj+1)'s global loads spread between the MFMAs ----
      {
        u32x4 vf[PFV];
#pragma unroll
        for (int i = 0; i < PFV; ++i) vf[i] = v_frag(vb_cur, i);
#pragma unroll
        for (int i = 0; i < NPV; ++i) {
          __builtin_amdgcn_sched_barrier(0);
          o[i % NDB] = mfma16<F16>(vf[i % PFV], pf[i / NDB], o[i % NDB]);
          if (i + PFV < NPV) vf[i % PFV] = v_frag(vb_cur, i + PFV);
          if (i % LDV_EVERY == 0 && i / LDV_EVERY < NLD) issue_tile_part<D, true>(next_v, i / LDV_EVERY, wave, lane_l);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#ifdef DG_ATTN_PHASE_TIMING
      asm volatile("s_nop 0" ::"a"(o[0][0]), "a"(o[NDB - 1][15]));
#endif
      DG_PHASE(6)
      if constexpr (PIPE) {
        if (jj + 1 < ntile) s_cur = s_next;
      }
    }
  }

  // ---- epilogue ----
  DG_PHASE_STORE
  const float l_tot = sum_across_halves(l_part);
  if (p.n_splits > 1) {
    const size_t prow = ((size_t)split * p.hkv + kvh) * p.rows_pad + r;
    float* po = p.part_o + prow * D + 4u * g2;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 v4 = {o[db][4 * q4], o[db][4 * q4 + 1], o[db][4 * q4 + 2], o[db][4 * q4 + 3]};
        *(f32x4*)(po + 32 * db + 8 * q4) = v4;
      }
    if (g2 == 0) {
      p.part_ml[prow * 2] = m_ref;
      p.part_ml[prow * 2 + 1] = l_tot;
    }
    return;
  }
  if (!row_ok) return;
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  const size_t ooff = ((size_t)tok * p.hq + qh) * D + 4u * g2;
  if (g2 == 0) {
    if (p.lse) p.lse[(size_t)tok * p.hq + qh] = l_tot > 0.f ? m_ref * kLn2 + __logf(l_tot) : -INFINITY;
    if (p.dbg && !(l_tot > 0.f)) dbg_report(p.dbg, 1u, (tok << 16) | qh, __float_as_uint(l_tot));
  }
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const float y0 = o[db][4 * q4] * inv, y1 = o[db][4 * q4 + 1] * inv;
      const float y2 = o[db][4 * q4 + 2] * inv, y3 = o[db][4 * q4 + 3] * inv;
      const size_t idx = ooff + 32 * db + 8 * q4;
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

template <int D, bool F16>
hipError_t launch_one(const AttnParams& p, hipStream_t s) {
  const uint32_t nstream = p.hkv * p.n_splits;
  const uint32_t grid = ((nstream + 7u) / 8u) * p.n_mtiles * 8u;
  constexpr bool kPipe = D < 512;  // at D=512 the second score tile does not fit next to O and Q
  hipLaunchKernelGGL((attn_mfma_kernel<D, F16, kPipe>), dim3(grid), dim3(256), 0, s, p);
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
