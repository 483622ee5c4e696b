// Building blocks shared by the MFMA kernels for gfx950: vector typedefs, the 32x32x16 MFMA
// wrapper, packed-pair conversions, wait-count helpers, and the LDS tile layout with its
// direct-to-LDS loader (one 32-key tile of K or V per call sequence).
#pragma once
#include "attn_params.h"

#include <type_traits>

namespace dg {
namespace {

// compile-time loop: f(std::integral_constant<int, I>) for I in [I0, N)
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

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

// Score MFMAs, written as assembly so that their accumulator is an ordinary VGPR tuple.  O fills
// all 256 accumulation registers at head_dim 512; the compiler gives every MFMA of such a
// kernel an accumulation-register destination, which made it park one block of O in VGPRs
// around each tile's score MFMAs (48 register moves per tile and wave).
// The compiler does not know these are MFMAs, so the one hazard it would otherwise cover is
// handled here: the last score MFMA of a tile (mfma_scores_last) is followed by the wait
// states a non-MFMA read of the scores needs.  Back-to-back MFMAs that accumulate into the same registers need
// no wait states, and operands that come from LDS are covered by the s_waitcnt the compiler
// inserts for the asm operands.
template <bool F16>
__device__ __forceinline__ void mfma_scores_first(f32x16& s, u32x4 a, u32x4 b) {
  if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(s) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(s) : "v"(a), "v"(b));
}
template <bool F16>
__device__ __forceinline__ void mfma_scores_acc(f32x16& s, u32x4 a, u32x4 b) {
  if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(s) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s) : "v"(a), "v"(b));
}
// Last score MFMA of a tile, followed by 12 wait states: what the compiler's own hazard recogniser keeps between
// an MFMA of this shape (8 passes) and a VALU read of its result on this target.  They are part of the same asm
// statement so that no compiler-made register copy of the scores can land between the MFMA and the wait.
template <bool F16>
__device__ __forceinline__ void mfma_scores_last(f32x16& s, u32x4 a, u32x4 b) {
  if constexpr (F16)
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\ts_nop 11" : "+v"(s) : "v"(a), "v"(b));
  else
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\ts_nop 11" : "+v"(s) : "v"(a), "v"(b));
}

// x *= c for values that live in accumulation registers, without the register allocator moving
// them into the VGPR class.  Eight at a time: eight independent read / multiply / write chains in flight.
__device__ __forceinline__ void scale_acc8(float& x0, float& x1, float& x2, float& x3, float& x4, float& x5, float& x6,
                                           float& x7, float c) {
  float t0, t1, t2, t3, t4, t5, t6, t7;
  asm volatile(
      "v_accvgpr_read_b32 %8, %0\n\tv_accvgpr_read_b32 %9, %1\n\tv_accvgpr_read_b32 %10, %2\n\tv_accvgpr_read_b32 %11, %3\n\t"
      "v_accvgpr_read_b32 %12, %4\n\tv_accvgpr_read_b32 %13, %5\n\tv_accvgpr_read_b32 %14, %6\n\tv_accvgpr_read_b32 %15, %7\n\t"
      "v_mul_f32 %8, %8, %16\n\tv_mul_f32 %9, %9, %16\n\tv_mul_f32 %10, %10, %16\n\tv_mul_f32 %11, %11, %16\n\t"
      "v_mul_f32 %12, %12, %16\n\tv_mul_f32 %13, %13, %16\n\tv_mul_f32 %14, %14, %16\n\tv_mul_f32 %15, %15, %16\n\t"
      "v_accvgpr_write_b32 %0, %8\n\tv_accvgpr_write_b32 %1, %9\n\tv_accvgpr_write_b32 %2, %10\n\tv_accvgpr_write_b32 %3, %11\n\t"
      "v_accvgpr_write_b32 %4, %12\n\tv_accvgpr_write_b32 %5, %13\n\tv_accvgpr_write_b32 %6, %14\n\tv_accvgpr_write_b32 %7, %15"
      : "+a"(x0), "+a"(x1), "+a"(x2), "+a"(x3), "+a"(x4), "+a"(x5), "+a"(x6), "+a"(x7), "=&v"(t0), "=&v"(t1), "=&v"(t2),
        "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7)
      : "v"(c));
}
// Behind the last scale_acc8 of a rescale: the compiler does not see those writes, and an MFMA that accumulates into
// the registers must keep clear of them.  Once per rescale, not once per group of registers (a rescale of a 32-row block
// is 16 groups at head_dim 256, and with an f16 cache a sliding layer's wave rescales every third tile).
__device__ __forceinline__ void scale_acc_done() { asm volatile("s_nop 3"); }
// Four values out of accumulation registers.  Spelled out so that the epilogue takes O from where
// the tile loop left it, a few registers at a time: left to itself the compiler moves all of O
// into VGPRs at the loop's exit, runs out of them and parks part of O in scratch memory, and the
// reloads then queue behind the epilogue's own stores (one memory counter serves both), which
// made every 32-row block wait for the previous block's stores to complete.
template <bool FROM_ACC>
__device__ __forceinline__ f32x4 acc_read4(const f32x16& a, int e) {
  if constexpr (!FROM_ACC) return f32x4{a[e], a[e + 1], a[e + 2], a[e + 3]};   // smaller head_dim: O does not fill the registers
  float t0, t1, t2, t3;
  asm volatile("v_accvgpr_read_b32 %0, %4\n\tv_accvgpr_read_b32 %1, %5\n\tv_accvgpr_read_b32 %2, %6\n\tv_accvgpr_read_b32 %3, %7"
               : "=v"(t0), "=v"(t1), "=v"(t2), "=v"(t3)
               : "a"(a[e]), "a"(a[e + 1]), "a"(a[e + 2]), "a"(a[e + 3]));
  return f32x4{t0, t1, t2, t3};
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

// s_waitcnt as a builtin, so that the compiler's own wait-count bookkeeping sees it (gfx9
// encoding: vmcnt = bits 3:0 and 15:14, expcnt = 6:4, lgkmcnt = 11:8; the other two counters are
// left at their maxima).
__device__ __forceinline__ void wait_vmem_all() {
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");
}

// all but the N most recent vector memory operations of the wave (they complete in order)
template <int N>
__device__ __forceinline__ void wait_vmem_but() {
  static_assert(N >= 0 && N < 16, "low four bits of vmcnt");
  __builtin_amdgcn_s_waitcnt(0x0F70 | N);
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

// LDS layout of one 32-key tile of K or V (rows = keys, head_dim contiguous, 16-byte chunks).
//
// head_dim 512: a row is exactly the KiB one direct-to-LDS instruction writes, so rows can be
// padded apart: K rows by 16 B (32 rows x one chunk per half-wave fall on distinct banks),
// V rows by 64 B (the 8 rows x 4 chunks of a transposing read do).  Every fragment address is
// then one per-lane base plus a compile-time offset, and the global side of a load is one
// row: a scalar address plus lane*16.
// smaller head_dim: several rows share an instruction's KiB, so rows stay dense and the 16-byte
// chunks are XOR-swizzled instead (the swizzle is applied by choosing which global chunk each
// lane fetches).
template <int D>
struct Lay {
  static constexpr int CPR = D / 8;          // chunks per row
  static constexpr int ROWB = 2 * D;         // bytes per row
  static constexpr bool PAD = CPR == 64;
  static constexpr int K_STRIDE = PAD ? ROWB + 16 : ROWB;
  static constexpr int V_STRIDE = PAD ? ROWB + 64 : ROWB;
  static constexpr int K_BYTES = 32 * K_STRIDE, V_BYTES = 32 * V_STRIDE;
  static constexpr int NBLK = 32 * CPR / 64;   // KiB blocks (= load instructions) per tile
  static constexpr int NLD = (NBLK + 3) / 4;   // load instructions per wave and tile
  static __device__ __forceinline__ uint32_t swz_k(uint32_t row) {
    if constexpr (PAD) return 0u;
    else if constexpr (CPR >= 16) return row & 15u;
    else return (row / (16 / CPR)) & (CPR - 1);
  }
  static __device__ __forceinline__ uint32_t swz_v(uint32_t row) {
    if constexpr (PAD) return 0u;
    else return ((row & 3u) << 2) & (CPR - 1);
  }
};

// One tile's direct-to-LDS loads, described once per tile and issued one wave instruction at a
// time so the issue slots can be spread between MFMAs.  Rows of the tile outside
// [t_min, t_all) are replaced by the nearest row inside: those keys are masked for every query
// row of the workgroup, but what their slots hold (dead ring slots, memory past the cache) may
// not be finite, and 0 * NaN would poison P.V.
struct TileLoad {
  const char* base;   // head base + slot(t0) * row stride (wave-uniform)
  uint32_t stride_b;  // bytes between key rows in global memory
  uint32_t rmin;      // first row of the tile that may be read
  uint32_t rmax;      // last row of the tile that may be read
  uint32_t lds;       // LDS byte address of the destination buffer (padded layout: of this wave's first row)
  // padded layout only, per lane: byte offsets from base of this lane's chunk in the first and
  // the last row that may be read, and in the row of this wave's load 0
  uint32_t lo_l, hi_l, raw0;
};

// FIRST: the tile may begin before t_min (only the first tile a workgroup visits can).
template <int D, bool IS_V, bool FIRST>
__device__ __forceinline__ TileLoad make_tile_load(const char* head_base, int64_t tok_stride_b, uint32_t t0,
                                                   uint32_t t_min, uint32_t t_all, uint32_t ring_mask, lds_char* buf,
                                                   uint32_t wave, uint32_t lane) {
  using L = Lay<D>;
  TileLoad tl;
  tl.base = head_base + (int64_t)kv_slot(ring_mask, t0) * tok_stride_b;
  tl.stride_b = (uint32_t)tok_stride_b;
  tl.rmax = min(t_all - 1u - t0, (uint32_t)kBlockN - 1u);
  // (a first visible key at or past t_all, i.e. rows that see nothing, must not move the clamp
  // past the last key that exists)
  tl.rmin = FIRST && t_min > t0 ? min(t_min - t0, tl.rmax) : 0u;
  tl.lds = (uint32_t)(size_t)buf;
  if constexpr (L::PAD) {
    tl.lds += wave * (IS_V ? L::V_STRIDE : L::K_STRIDE);
    tl.lo_l = tl.rmin * tl.stride_b + lane * 16u;
    tl.hi_l = tl.rmax * tl.stride_b + lane * 16u;
    tl.raw0 = wave * tl.stride_b + lane * 16u;
  }
  return tl;
}

// The descriptor with every field computed at this point of the program (the compiler would
// otherwise sink the arithmetic to the first use, which sits behind a branch where nothing
// overlaps it).
__device__ __forceinline__ TileLoad pinned(TileLoad tl) {
  uint64_t b = (uint64_t)tl.base;
  uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
  uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  uint32_t lds = (uint32_t)__builtin_amdgcn_readfirstlane(tl.lds);
  asm volatile("" : "+s"(lo), "+s"(hi), "+s"(lds), "+v"(tl.lo_l), "+v"(tl.hi_l), "+v"(tl.raw0));
  tl.base = (const char*)(((uint64_t)hi << 32) | lo);
  tl.lds = lds;
  return tl;
}

// The loads are written as assembly on purpose: the compiler orders every LDS read after a
// direct-to-LDS load it knows about with s_waitcnt vmcnt(0), which would expose the whole
// fetch latency once per tile.  The kernel waits for these loads itself (wait_vmem_all).
// All scalar operands are wave-uniform by construction; readfirstlane tells the compiler so
// (it returns a signed int: without the casts the low half of the address would be
// sign-extended over the high half).
__device__ __forceinline__ uint64_t uniform_address(const char* base_uniform) {
  const uint64_t b = (uint64_t)base_uniform;
  return ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32)) << 32) |
         (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
}
// lane l: 16 bytes from base + voff -> LDS byte (lds_dst + LDS_IMM) + 16 * l
template <int LDS_IMM>
__device__ __forceinline__ void lds_dma_16(const char* base_uniform, uint32_t voff, uint32_t lds_dst_uniform) {
  const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane(lds_dst_uniform);
  const uint64_t base = uniform_address(base_uniform);
  if constexpr (LDS_IMM == 0) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff), "s"(base)
                 : "memory");
  } else {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff),
                 "s"(base), "n"(LDS_IMM)
                 : "memory", "scc");
  }
}

// G consecutive KiB blocks of a tile with one setting of M0: block g goes to LDS byte (lds_dst + LDS_IMM) + 1024 g
// + 16 * l.  The instruction's immediate offset moves the LDS address AND the memory address, so the caller's
// per-lane offsets are biased: voff[g] = (byte offset from the tile's base) + kDmaBias - 1024 g, and the base passed
// here is the tile's base minus kDmaBias (the bias keeps every voff non-negative whatever row a clamp picked).
// Saves an M0 write and the wait state behind it for every block but the first.
constexpr uint32_t kDmaBias = 4096;
template <int G, int LDS_IMM>
__device__ __forceinline__ void lds_dma_16_group(const char* base_minus_bias_uniform, const uint32_t* voff,
                                                 uint32_t lds_dst_uniform) {
  static_assert(G == 1 || G == 2 || G == 4, "immediate offsets reach 3 KiB");
  const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane(lds_dst_uniform);
  const uint64_t base = uniform_address(base_minus_bias_uniform);
  if constexpr (G == 1) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff[0]), "s"(base),
                 "n"(LDS_IMM)
                 : "memory", "scc");
  } else if constexpr (G == 2) {
    asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %3\n\t"
                 "global_load_lds_dwordx4 %2, %3 offset:1024" ::"s"(dst),
                 "v"(voff[0]), "v"(voff[1]), "s"(base), "n"(LDS_IMM)
                 : "memory", "scc");
  } else {
    asm volatile("s_add_u32 m0, %0, %6\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %5\n\t"
                 "global_load_lds_dwordx4 %2, %5 offset:1024\n\tglobal_load_lds_dwordx4 %3, %5 offset:2048\n\t"
                 "global_load_lds_dwordx4 %4, %5 offset:3072" ::"s"(dst),
                 "v"(voff[0]), "v"(voff[1]), "v"(voff[2]), "v"(voff[3]), "s"(base), "n"(LDS_IMM)
                 : "memory", "scc");
  }
}

// lane l: 4 bytes from base + voff -> a dump area in LDS (64 words) that nobody reads.  What the load
// is for is its side effect: the 128-byte line it touches is in the L2 afterwards.  A load without a
// register destination, so nothing has to stay reserved until it lands.
__device__ __forceinline__ void lds_dma_touch(const char* base_uniform, uint32_t voff, uint32_t lds_dump_uniform) {
  const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane(lds_dump_uniform);
  const uint64_t base = uniform_address(base_uniform);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(dst), "v"(voff), "s"(base) : "memory");
}

template <int D, bool IS_V, int K>
__device__ __forceinline__ void issue_tile_part(const TileLoad& tl, uint32_t wave, uint32_t lane) {
  using L = Lay<D>;
  if (L::NBLK < 4 && K * 4 + wave >= (uint32_t)L::NBLK) return;
  if constexpr (L::PAD) {
    // one instruction = one key row (row 4 K + wave): everything but the clamp of the row is
    // either per tile or a compile-time constant
    uint32_t voff;
    asm("v_med3_u32 %0, %1, %2, %3" : "=v"(voff) : "v"(tl.raw0 + (uint32_t)(4 * K) * tl.stride_b), "v"(tl.lo_l), "v"(tl.hi_l));
    lds_dma_16<4 * K * (IS_V ? L::V_STRIDE : L::K_STRIDE)>(tl.base, voff, tl.lds);
  } else {
    const uint32_t blk = K * 4 + wave;
    const uint32_t pch = blk * 64 + lane;
    const uint32_t r = pch / L::CPR, pc = pch % L::CPR;
    const uint32_t c = pc ^ (IS_V ? L::swz_v(r) : L::swz_k(r));
    lds_dma_16<0>(tl.base, min(max(r, tl.rmin), tl.rmax) * tl.stride_b + c * 16u, tl.lds + blk * 1024u);
  }
}

template <int D, bool IS_V, int K = 0>
__device__ __forceinline__ void issue_tile(const TileLoad& tl, uint32_t wave, uint32_t lane) {
  if constexpr (K < Lay<D>::NLD) {
    issue_tile_part<D, IS_V, K>(tl, wave, lane);
    issue_tile<D, IS_V, K + 1>(tl, wave, lane);
  }
}

}  // namespace
}  // namespace dg
