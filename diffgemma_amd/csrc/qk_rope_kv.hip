// The producer of the cache rows attention reads: per-head RMSNorm + RoPE + KV-cache write for
// the canvas rows of one layer (reference: src/shaders/attn/qk_rope_kv/qk_rope_kv.metal:29-149,
// CPU twin src/shaders/attn/cpu.rs:78-145).
//
// One wave per (canvas row, head), heads = Hq query heads, then Hkv key heads, then Hkv value
// heads, exactly the reference's grid (enc.rs:1794-1804).  The row (at most 1 KiB) is read once
// with up to 16-byte loads, normalised in registers, staged in LDS where each lane rotates one
// pair (d, hd/2 + d) per pass (cos and sin of the row's angles once per workgroup of four heads), and written once: Q (and K, unless V aliases it) back in place as bf16, K
// and V into the cache at slot(pos) in the cache's element type.  HBM-bound by construction:
// every byte moves once; at 256 canvas rows the launch is a few megabytes, i.e. latency-bound.
#include "attn_params.h"
#include "wt_store.h"
#include "../../include/dg_attn.h"

#include <hip/hip_fp16.h>

#include <cmath>

namespace dg {
namespace {

struct RopeParams {
  uint16_t* q;           // [canvas][hq][hd] bf16, in place
  uint16_t* k;           // [canvas][hkv][hd] bf16, in place unless v_from_k
  const uint16_t* v;     // [canvas][hkv][hd] bf16 (unused when v_from_k)
  void* kc;              // cache region + K offset
  void* vc;              // cache region + V offset
  const uint16_t* qw;    // [hd] bf16 norm weights
  const uint16_t* kw;
  uint32_t* dbg;
  const uint32_t* step_dev;   // device copy of the reference's StepParams, or null: kv_len (word 0) and kv_write_end
                              // (word 11) are then read from it when the kernel runs
  int64_t k_tok_stride, k_head_stride, v_tok_stride, v_head_stride;  // elements
  uint32_t canvas, hq, hkv, hd;
  uint32_t kv_len, kv_write_end, ring_mask;
  uint32_t is_full, v_from_k, kv_dtype, qk_trunc;
  // theta^(-2 d / hd) for d < rot/2, computed on the host with the C library's powf: the angle
  // pos * inv_freq is an fp32 product, and at pos ~ 1e5 one unit in the last place of inv_freq
  // moves it by a hundredth of a radian, so the table is what makes the rotation reproduce the
  // reference's CPU twin (cpu.rs:35,57) instead of depending on the device's pow
  float inv_freq[256];
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

constexpr float kRmsEps = 1e-6f;   // cpu.rs:3, attention_device.metal:10

// One row of `hd` bf16 elements, `per` = hd/64 consecutive ones per lane, moved with the widest
// access the count allows (16 bytes at hd 512).
template <int PER>
__device__ __forceinline__ void load_row(const uint16_t* src, float (&x)[8]) {
  if constexpr (PER == 8) {
    const uint4 r = *(const uint4*)src;
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = __uint_as_float(w[i] << 16);
      x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  } else if constexpr (PER == 4) {
    const uint2 r = *(const uint2*)src;
    x[0] = __uint_as_float(r.x << 16);
    x[1] = __uint_as_float(r.x & 0xffff0000u);
    x[2] = __uint_as_float(r.y << 16);
    x[3] = __uint_as_float(r.y & 0xffff0000u);
  } else if constexpr (PER == 2) {
    const uint32_t r = *(const uint32_t*)src;
    x[0] = __uint_as_float(r << 16);
    x[1] = __uint_as_float(r & 0xffff0000u);
  } else {
    x[0] = bf16_bits_to_f32(src[0]);
  }
}

// `per` consecutive elements as 16-bit storage values, packed and written with one store at element
// `d0` of the row that starts at `row` (the same row for the whole wave).  Written through: the
// attention kernel that follows reads these rows from every XCD (wt_store.h).
template <int PER>
__device__ __forceinline__ void store_row16(uint16_t* row, uint32_t d0, const uint16_t (&h)[8]) {
  const auto win = wt_window_wave(row);
  if constexpr (PER == 8) {
    const wt_u32x4 v = {h[0] | (uint32_t)h[1] << 16, h[2] | (uint32_t)h[3] << 16, h[4] | (uint32_t)h[5] << 16,
                        h[6] | (uint32_t)h[7] << 16};
    wt_store16(win, d0 * 2u, v);
  } else if constexpr (PER == 4) {
    const wt_u32x2 v = {h[0] | (uint32_t)h[1] << 16, h[2] | (uint32_t)h[3] << 16};
    wt_store8(win, d0 * 2u, v);
  } else if constexpr (PER == 2) {
    wt_store4(win, d0 * 2u, h[0] | (uint32_t)h[1] << 16);
  } else {
    wt_store2(win, d0 * 2u, h[0]);
  }
}

__device__ __forceinline__ uint16_t cache_bits(uint32_t dt, float v) {
  if (dt == DT_F16) return __builtin_bit_cast(uint16_t, (_Float16)v);   // kv_store: half(v), round to nearest
  return f32_to_bf16_bits(v, false);
}

template <int PER>
__global__ void __launch_bounds__(256) qk_rope_kv_kernel(const RopeParams p) {
  __shared__ float stage[4][512];
  __shared__ float cos_t[256], sin_t[256];
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t tok = blockIdx.x, h_raw = blockIdx.y * 4 + wave;
  const uint32_t n_heads = p.hq + 2 * p.hkv;
  const bool head_ok = h_raw < n_heads;
  const uint32_t h = head_ok ? h_raw : n_heads - 1u;   // (a wave without a head of its own stays for the barrier below)
  const uint32_t hd = p.hd;
  const bool is_q = h < p.hq, is_k = !is_q && h < p.hq + p.hkv;
  const uint32_t hh = is_q ? h : (h - p.hq) % p.hkv;
  // (the reference binds StepParams as a device buffer, qk_rope_kv.metal:30-38: read at execution time)
  const uint32_t kv_len = p.step_dev ? (uint32_t)__builtin_amdgcn_readfirstlane((int)p.step_dev[0]) : p.kv_len;
  const uint32_t kv_write_end = p.step_dev ? (uint32_t)__builtin_amdgcn_readfirstlane((int)p.step_dev[11]) : p.kv_write_end;
  const uint32_t pos = kv_len + tok;
  const bool kv_write = pos < kv_write_end;
  const int64_t slot = p.ring_mask ? (pos & p.ring_mask) : pos;

  uint16_t* row_inplace = is_q ? p.q + ((size_t)tok * p.hq + hh) * hd : p.k + ((size_t)tok * p.hkv + hh) * hd;
  const uint16_t* src = (is_q || is_k) ? row_inplace
                                       : (p.v_from_k ? p.k : p.v) + ((size_t)tok * p.hkv + hh) * hd;

  // lane owns elements [PER*lane, PER*lane + PER); at hd < 64 only the first hd lanes own one
  const uint32_t d0 = lane * PER;
  const bool active = d0 < hd;
  float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (active) load_row<PER>(src + d0, x);
  // (the norm weights too, now: asked for where they are used, behind the row sum, they were a second trip to
  // memory on the wave's critical path)
  float w[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (active && (is_q || is_k)) load_row<PER>((is_q ? p.qw : p.kw) + d0, w);
  // The angles depend on the position only: the workgroup's four heads share one table of cos and sin,
  // one pair per thread, worked out while the rows are on their way (rotation, cpu.rs:31-65: pairs
  // (d, hd/2 + d) for d < rot/2; split-half: rot = hd, theta 1e4; proportional: rot = hd/4, theta 1e6,
  // everything else is left alone).
  const uint32_t half_rot = p.is_full ? hd / 8 : hd / 2, off = hd / 2;
  if (threadIdx.x < half_rot) {
    float sn, cs;
    sincosf((float)pos * p.inv_freq[threadIdx.x], &sn, &cs);
    cos_t[threadIdx.x] = cs;
    sin_t[threadIdx.x] = sn;
  }
  __syncthreads();
  if (!head_ok) return;   // the whole wave leaves; nothing below synchronises across waves
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) ss += x[i] * x[i];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)hd + kRmsEps);
  if (lane == 0 && !(inv == inv && fabsf(inv) != INFINITY))
    dbg_report(p.dbg, DBG_ERR_NONFINITE, DBG_KERNEL_QK_ROPE_KV, (tok << 16) | h, tok);   // (qk_rope_kv.metal:77: tag = canvas row)

  uint16_t bits[8];
  if (!is_q && !is_k) {   // V: normalise without weight, write to the cache (cpu.rs:110-122)
    if (kv_write && active) {
#pragma unroll
      for (int i = 0; i < PER; ++i) bits[i] = cache_bits(p.kv_dtype, x[i] * inv);
      store_row16<PER>((uint16_t*)p.vc + slot * p.v_tok_stride + (int64_t)hh * p.v_head_stride, d0, bits);
    }
    return;
  }

  float* st = stage[wave];
  if (active) {
#pragma unroll
    for (int i = 0; i < PER; ++i) st[d0 + i] = x[i] * (inv * w[i]);   // x * (inv * w), the CPU twin's order (cpu.rs:71-74)
  }
  __builtin_amdgcn_wave_barrier();   // the stage is private to the wave, whose LDS operations execute in order

  // one pair per lane and pass
  for (uint32_t dd = lane; dd < half_rot; dd += 64) {
    const float s = sin_t[dd], c = cos_t[dd];
    const float x0 = st[dd], x1 = st[dd + off];
    st[dd] = x0 * c - x1 * s;
    st[dd + off] = x0 * s + x1 * c;
  }
  __builtin_amdgcn_wave_barrier();
  if (!active) return;
  float y[8];
#pragma unroll
  for (int i = 0; i < PER; ++i) y[i] = st[d0 + i];
  if (is_k && kv_write) {
#pragma unroll
    for (int i = 0; i < PER; ++i) bits[i] = cache_bits(p.kv_dtype, y[i]);
    store_row16<PER>((uint16_t*)p.kc + slot * p.k_tok_stride + (int64_t)hh * p.k_head_stride, d0, bits);
  }
  // Q always goes back in place; K only when V does not alias the raw k projection (cpu.rs:137-143)
  if (is_q || !p.v_from_k) {
#pragma unroll
    for (int i = 0; i < PER; ++i) bits[i] = f32_to_bf16_bits(y[i], p.qk_trunc != 0);
    store_row16<PER>(row_inplace, d0, bits);
  }
}

}  // namespace
}  // namespace dg

extern "C" {

static int rope_launch(const dg_rope_desc* d, const dg_step_params* step_dev, void* q, void* k, const void* v, void* kv_base,
                       const void* q_norm_w, const void* k_norm_w, dg_debug_status* dbg, void* stream) {
  if (!d || !q || !k || !kv_base || !q_norm_w || !k_norm_w) return DG_ERR_NULL;
  if (((uintptr_t)step_dev % 4) != 0) return DG_ERR_LAYOUT;
  if (!d->v_from_k && !v) return DG_ERR_NULL;
  const uint32_t hd = d->head_dim;
  if (!(hd == 32 || hd == 64 || hd == 128 || hd == 256 || hd == 512)) return DG_ERR_SHAPE;
  if (d->canvas == 0 || d->n_q_heads == 0 || d->n_kv_heads == 0) return DG_ERR_SHAPE;
  if (d->kv_dtype != DG_F16 && d->kv_dtype != DG_BF16) return DG_ERR_DTYPE;
  if (d->kv_ring_mask != 0 && ((d->kv_ring_mask + 1) & d->kv_ring_mask) != 0) return DG_ERR_LAYOUT;
  if ((uint64_t)d->kv_len + d->canvas > 0xffffffffull) return DG_ERR_SHAPE;
  if (d->kv_region_bytes % 2 != 0) return DG_ERR_LAYOUT;
  if (d->k_tok_stride < (int64_t)hd || d->v_tok_stride < (int64_t)hd || d->k_head_stride < (int64_t)hd ||
      d->v_head_stride < (int64_t)hd)
    return DG_ERR_LAYOUT;
  dg::RopeParams p{};
  p.q = (uint16_t*)q;
  p.k = (uint16_t*)k;
  p.v = (const uint16_t*)v;
  char* region = (char*)kv_base + d->kv_region_bytes;
  p.kc = region;
  p.vc = region + d->v_base_off * 2;
  p.qw = (const uint16_t*)q_norm_w;
  p.kw = (const uint16_t*)k_norm_w;
  p.dbg = (uint32_t*)dbg;
  p.step_dev = (const uint32_t*)step_dev;
  p.k_tok_stride = d->k_tok_stride;
  p.k_head_stride = d->k_head_stride;
  p.v_tok_stride = d->v_tok_stride;
  p.v_head_stride = d->v_head_stride;
  p.canvas = d->canvas;
  p.hq = d->n_q_heads;
  p.hkv = d->n_kv_heads;
  p.hd = hd;
  p.kv_len = d->kv_len;
  p.kv_write_end = d->kv_write_end;
  p.ring_mask = d->kv_ring_mask;
  p.is_full = d->is_full ? 1u : 0u;
  p.v_from_k = d->v_from_k ? 1u : 0u;
  p.kv_dtype = d->kv_dtype == DG_F16 ? dg::DT_F16 : dg::DT_BF16;
  p.qk_trunc = (d->flags & DG_ROPE_F_QK_TRUNCATE) ? 1u : 0u;
  const float theta = d->is_full ? 1.0e6f : 1.0e4f;        // cpu.rs:25-27
  const uint32_t half_rot = d->is_full ? hd / 8 : hd / 2;  // rot = hd/4 or hd (cpu.rs:17-23)
  for (uint32_t dd = 0; dd < half_rot; ++dd) p.inv_freq[dd] = std::pow(theta, -2.0f * (float)dd / (float)hd);
  const uint32_t n_heads = d->n_q_heads + 2 * d->n_kv_heads;
  // vector accesses of `per` elements: rows and the cache region must be aligned to them
  const uint32_t per = hd >= 64 ? hd / 64 : 1;
  const uintptr_t align = 2 * per;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)p.kc | (uintptr_t)p.vc | (uintptr_t)q_norm_w | (uintptr_t)k_norm_w |
       (d->v_from_k ? 0 : (uintptr_t)v)) % align != 0)
    return DG_ERR_LAYOUT;
  if ((d->k_tok_stride | d->k_head_stride | d->v_tok_stride | d->v_head_stride) % per != 0) return DG_ERR_LAYOUT;
  const dim3 grid(d->canvas, (n_heads + 3) / 4), block(256);
  hipStream_t s = (hipStream_t)stream;
  switch (per) {
    case 8: hipLaunchKernelGGL(dg::qk_rope_kv_kernel<8>, grid, block, 0, s, p); break;
    case 4: hipLaunchKernelGGL(dg::qk_rope_kv_kernel<4>, grid, block, 0, s, p); break;
    case 2: hipLaunchKernelGGL(dg::qk_rope_kv_kernel<2>, grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL(dg::qk_rope_kv_kernel<1>, grid, block, 0, s, p); break;
  }
  return hipGetLastError() == hipSuccess ? DG_OK : DG_ERR_LAUNCH;
}

int dg_qk_rope_kv(const dg_rope_desc* d, void* q, void* k, const void* v, void* kv_base, const void* q_norm_w,
                  const void* k_norm_w, dg_debug_status* dbg, void* stream) {
  return rope_launch(d, nullptr, q, k, v, kv_base, q_norm_w, k_norm_w, dbg, stream);
}

int dg_qk_rope_kv_dev(const dg_rope_desc* d, const dg_step_params* step_dev, void* q, void* k, const void* v, void* kv_base,
                      const void* q_norm_w, const void* k_norm_w, dg_debug_status* dbg, void* stream) {
  if (!step_dev) return DG_ERR_NULL;
  return rope_launch(d, step_dev, q, k, v, kv_base, q_norm_w, k_norm_w, dbg, stream);
}

// The reference's argument block -> descriptor; kv_len / kv_write_end from the host copy of P, or (P == null) left to
// the device copy.
static void rope_desc_from_reference(const dg_layer_offsets* L, const dg_step_params* P, const dg_attn_dims* dims,
                                     dg_rope_desc* out) {
  dg_rope_desc d{};
  d.canvas = dims->canvas;
  d.n_q_heads = dims->n_q_heads;
  d.n_kv_heads = L->n_kv_heads;
  d.head_dim = L->head_dim;
  d.kv_len = P ? P->kv_len : 0u;
  d.kv_write_end = P ? P->kv_write_end : 0xffffffffu;
  d.kv_ring_mask = L->kv_ring_mask;
  d.is_full = L->is_full;
  d.v_from_k = L->v_proj == 0 ? 1u : 0u;
  d.kv_dtype = DG_F16;
  d.flags = DG_ROPE_F_QK_TRUNCATE;   // arena_store truncates (common.metal:16-18)
  d.kv_region_bytes = L->kv_region;
  const int64_t row = (int64_t)L->n_kv_heads * L->head_dim;   // slot-major [slot][K: Hkv*d | V: Hkv*d]
  d.k_tok_stride = 2 * row;
  d.k_head_stride = L->head_dim;
  d.v_base_off = row;
  d.v_tok_stride = 2 * row;
  d.v_head_stride = L->head_dim;
  *out = d;
}

int dg_qk_rope_kv_dispatch(void* q, void* k, void* v, void* kvcache, const void* blob, const dg_layer_offsets* L,
                           const dg_step_params* P, const dg_attn_dims* dims, dg_debug_status* dbg, void* stream) {
  if (!L || !P || !dims || !blob) return DG_ERR_NULL;
  dg_rope_desc d;
  rope_desc_from_reference(L, P, dims, &d);
  return dg_qk_rope_kv(&d, q, k, v, kvcache, (const char*)blob + L->q_norm, (const char*)blob + L->k_norm, dbg, stream);
}

int dg_qk_rope_kv_dispatch_dev(void* q, void* k, void* v, void* kvcache, const void* blob, const dg_layer_offsets* L,
                               const dg_step_params* P_dev, const dg_attn_dims* dims, dg_debug_status* dbg, void* stream) {
  if (!L || !P_dev || !dims || !blob) return DG_ERR_NULL;
  dg_rope_desc d;
  rope_desc_from_reference(L, nullptr, dims, &d);
  return dg_qk_rope_kv_dev(&d, P_dev, q, k, v, kvcache, (const char*)blob + L->q_norm, (const char*)blob + L->k_norm, dbg,
                           stream);
}

}  // extern "C"
