// Kernel-side argument block and mask arithmetic shared by every attention kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dg {

enum : uint32_t { DT_BF16 = 0, DT_F16 = 1, DT_F32 = 2 };

constexpr uint32_t kMaxSplits = 64;   // key-range splits per launch: the merge gives each a lane
constexpr int kBlockM = 128;   // stacked query rows per workgroup (4 waves x 32)
constexpr int kBlockN = 32;    // keys per tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Stacked row r of a KV head = tok * group + g: the `group` query heads that share one KV
// head sit next to each other, so a 128-row tile covers 128/group consecutive canvas rows.
struct AttnParams {
  const void* q;       // [canvas][hq][D], element type = KV element type unless q_is_bf16
  const void* k;       // layer region + K offset (element type E)
  const void* v;       // layer region + V offset
  void* out;           // [canvas][hq][D]
  float* lse;          // [canvas][hq] or null
  float* part_o;       // [split][hkv][rows_pad][D]: unnormalised fp32 accumulators, or (part_half) the same
                       // index space in f16 holding accumulators divided by the split's row sum
  float* part_ml;      // [split][hkv][rows_pad][2] (m in log2 units, l)
  uint32_t* dbg;       // 4 words, first-writer-wins, or null
  const uint32_t* step_dev;   // device copy of the reference's StepParams, or null: when set, kv_len is read from its
                              // first word when the kernel runs (resolve_step) and the kv_len below is the largest
                              // prefix the launch was planned for
  int64_t k_tok_stride, k_head_stride, v_tok_stride, v_head_stride;  // elements
  uint32_t canvas, hq, hkv, group;
  uint32_t kv_len, t_all;
  uint32_t causal_rows;
  uint32_t win_m1;       // window-1, or 0xffffffff when unwindowed
  uint32_t lo_nc;        // first visible key of a non-causal row
  uint32_t extra_lo;     // causal rows also see keys >= extra_lo (t_all = none)
  uint32_t ring_mask;
  uint32_t t_clip_lo, t_clip_hi;   // only keys in [t_clip_lo, t_clip_hi) count (a key-range partial); the whole range: 0, t_all
  uint32_t rows_total, rows_pad, n_mtiles;
  uint32_t n_splits, tile_first, tiles_per_split, tile_end;
  uint32_t q_is_bf16;    // Q holds bf16 although E is f16 (reference: bf16 activations, f16 cache)
  uint32_t out_dtype, out_trunc;
  uint32_t part_half;    // split partials are normalised f16 rows instead of unnormalised fp32 ones
  uint32_t touch_ahead;  // head_dim 512: touch key/value tiles into the L2 some tiles before they are loaded
  uint32_t lo_explicit;  // lo_nc was given by the caller (not the window rule)
  uint32_t sees_masked;  // causal rows also see the canvas keys behind the causal rows
  float scale_log2;      // softmax_scale * log2(e)
};

// One pass of top-k sparse attention over canvas rows [tok0, tok0 + ntok).
constexpr int kTopkMaxK = 1024;   // most keys a row may keep
struct TopkParams {
  AttnParams a;          // tensors, strides and mask constants of the whole call
  float* s_plane;        // scores [hq][ntok][t_pad], fp32
  uint32_t tok0, ntok;
  uint32_t t_pad;        // floats per score row, a multiple of the key tile
  uint32_t n_mtiles;     // 128-row tiles of stacked rows in this pass
  uint32_t n_splits;     // key-range splits of the score kernel (no merge needed)
  uint32_t tile_first, tile_end;
  uint32_t k_cfg[4];     // (fixed k | chunk grid, divisor, k_min, k_max)
  float scale;
};

// Merging attention states of key-range partials (dg_attn_merge).  A state holds, per row
// (row = canvas row * n_q_heads + query head), m and l in two planes of `rows` floats and then, from
// the next 16-byte boundary, head_dim accumulators `acc` per row, with
//   output row = acc / l,   log-sum-exp of the row's scores = m + ln l   (natural log; l = 0: no key seen).
constexpr uint32_t kMaxStates = 16;
__host__ __device__ inline size_t state_acc_offset(size_t rows) { return (2 * rows + 3) & ~(size_t)3; }   // floats
struct StateMergeParams {
  const float* states[kMaxStates];
  uint32_t n, rows, hd, hq;
  void* out;            // [rows][head_dim] of out_dtype, or null
  float* lse;           // [rows] or null
  float* state_out;     // a state, or null; may be one of `states` (a row is read before it is written)
  uint32_t out_dtype, out_trunc;
  uint32_t* dbg;
};

// The reference binds StepParams as a device buffer (src/metal/step_kernel/enc.rs:2177-2220, buffer 4), so the
// prefix length a recorded command sequence works on is read when it runs.  With step_dev set, the same here:
// kv_len comes from device memory (clamped to the prefix the launch was planned for: grid, split count and
// workspace follow that maximum) and everything derived from it is worked out again, the way the host does it
// in make_plan.  The key range is the whole one (a key-range partial takes kv_len from the host).
__device__ __forceinline__ AttnParams resolve_step(const AttnParams& in) {
  AttnParams p = in;
  if (in.step_dev == nullptr) return p;
  const uint32_t kv = (uint32_t)__builtin_amdgcn_readfirstlane((int)min(in.step_dev[0], in.kv_len));
  p.kv_len = kv;
  p.t_all = kv + p.canvas;
  const bool windowed = p.win_m1 != 0xffffffffu;
  if (!p.lo_explicit) p.lo_nc = (windowed && kv > p.win_m1) ? kv - p.win_m1 : 0u;
  p.lo_nc = min(p.lo_nc, p.t_all);
  p.extra_lo = p.sees_masked ? min(kv + p.causal_rows, p.t_all) : p.t_all;
  uint32_t lo_all = 0xffffffffu;
  if (p.causal_rows < p.canvas) lo_all = min(lo_all, p.lo_nc);
  if (p.causal_rows > 0u) lo_all = min(lo_all, (windowed && kv > p.win_m1) ? kv - p.win_m1 : 0u);
  lo_all = min(lo_all, p.t_all);
  p.t_clip_lo = 0u;
  p.t_clip_hi = p.t_all;
  p.tile_first = lo_all / (uint32_t)kBlockN;
  p.tile_end = max(p.tile_first, (p.t_all + (uint32_t)kBlockN - 1u) / (uint32_t)kBlockN);
  return p;
}

struct RowBounds {
  uint32_t lo, hi, extra;  // visible iff (lo <= t < hi) or (extra <= t), and t < t_all
};

// Reference rules: causal rows see [max(0,qpos-(window-1)), qpos]; the other rows see
// [lo_nc, t_all) where lo_nc = max(0, kv_len-(window-1)) unless the caller set it.
__device__ __forceinline__ RowBounds row_bounds(const AttnParams& p, uint32_t tok) {
  RowBounds b;
  const bool causal = tok < p.causal_rows;
  const uint32_t qpos = p.kv_len + tok;
  if (causal) {
    b.hi = min(p.t_all, qpos + 1u);
    b.lo = (p.win_m1 != 0xffffffffu && qpos > p.win_m1) ? qpos - p.win_m1 : 0u;
    b.extra = p.extra_lo;
  } else {
    b.hi = p.t_all;
    b.lo = p.lo_nc;
    b.extra = p.t_all;
  }
  b.lo = max(b.lo, p.t_clip_lo);
  b.hi = min(b.hi, p.t_clip_hi);
  b.extra = max(b.extra, p.t_clip_lo);   // (keys at or past t_clip_hi are cut by key_visible's last argument)
  return b;
}

__device__ __forceinline__ bool key_visible(const RowBounds& b, uint32_t t, uint32_t t_all) {
  return t < t_all && ((t >= b.lo && t < b.hi) || t >= b.extra);
}

__device__ __forceinline__ uint32_t kv_slot(uint32_t ring_mask, uint32_t t) {
  return ring_mask ? (t & ring_mask) : t;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __uint_as_float((uint32_t)b << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f, bool trunc) {
  uint32_t u = __float_as_uint(f);
  if (!trunc) {
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
  }
  return (uint16_t)(u >> 16);
}

// The reference's DebugStatus vocabulary (src/shaders/include/debug_status.metal:8-19 error codes,
// src/shaders/include/dgq_kernels.metal:33-34 kernel ids), decoded on the host by
// src/metal/debug_status.rs:33-75.  include/dg_attn.h carries the same numbers as DG_DBG_*.
enum : uint32_t {
  DBG_ERR_SOFTMAX_NORM_ZERO = 3u,   // a row's softmax denominator was not > 0; value = (tok << 16) | query head
  DBG_ERR_NONFINITE = 4u,           // a result was NaN or infinite; value = element index (attention) / canvas row (producer)
  DBG_ERR_BAD_DIM = 8u,
  DBG_KERNEL_QK_ROPE_KV = 25u,
  DBG_KERNEL_ATTENTION = 26u,
};

// first-writer-wins status record, like the reference's debug_set_error (debug_status.metal:38-52).
// tg is (tok << 16) | query head of the row at fault (the reference's call sites pass 0 there).
__device__ __forceinline__ void dbg_report(uint32_t* dbg, uint32_t code, uint32_t kernel_id, uint32_t tg,
                                           uint32_t value) {
  if (dbg == nullptr) return;
  if (atomicCAS(dbg, 0u, code) == 0u) {
    dbg[1] = kernel_id;
    dbg[2] = tg;
    dbg[3] = value;
  }
}

// host-side launchers (defined next to their kernels)
hipError_t launch_attn_scalar(const AttnParams& p, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s);
hipError_t launch_attn_mfma(const AttnParams& p, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s);
hipError_t launch_attn_wsplit(const AttnParams& p, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s);
hipError_t launch_attn_merge(const AttnParams& p, uint32_t head_dim, bool streamed, hipStream_t s);
hipError_t launch_state_merge(const StateMergeParams& p, hipStream_t s);
// l[row] = 1 where m[row] is finite, else 0: completes a state whose rows are already normalised
hipError_t launch_state_unit_l(float* m_plane, float* l_plane, uint32_t rows, hipStream_t s);
hipError_t launch_convert(const void* src, uint32_t src_dtype, void* dst, uint32_t dst_dtype, size_t n, hipStream_t s);
// gathers keys [0,t_all) of a strided (possibly ring) cache into planes [hkv][t_all][D] of dst_dtype
hipError_t launch_kv_gather(const void* src, uint32_t src_dtype, void* dst, uint32_t dst_dtype, uint32_t hkv,
                            uint32_t t_all, uint32_t head_dim, int64_t tok_stride, int64_t head_stride,
                            uint32_t ring_mask, hipStream_t s);

hipError_t launch_topk_scores(const TopkParams& tp, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s);
hipError_t launch_topk_select(const TopkParams& tp, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s);

hipError_t launch_calib_copy(void* dst, const void* src, size_t bytes, hipStream_t s);
hipError_t launch_calib_mfma(float* sink, uint32_t workgroups, uint32_t iters, uint32_t operand_mode, hipStream_t s);

}  // namespace dg
