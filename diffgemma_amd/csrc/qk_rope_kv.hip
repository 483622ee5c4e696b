// The producer of the cache rows attention reads: per-head RMSNorm + RoPE + KV-cache write for
// the canvas rows of one layer (reference: src/shaders/attn/qk_rope_kv/qk_rope_kv.metal:29-149,
// CPU twin src/shaders/attn/cpu.rs:78-145).
//
// One wave per (canvas row, head), heads = Hq query heads, then Hkv key heads, then Hkv value
// heads, exactly the reference's grid (enc.rs:1794-1804).  The row (at most 1 KiB) is read once
// with 16-byte loads, normalised in registers, staged in LDS so the rotation can pair element d
// with its partner, and written once: Q (and K, unless V aliases it) back in place as bf16, K
// and V into the cache at slot(pos) in the cache's element type.  HBM-bound by construction:
// every byte moves once; at 256 canvas rows the launch is a few megabytes, i.e. latency-bound.
#include "attn_params.h"
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

__device__ __forceinline__ void store_cache(void* base, uint32_t dt, int64_t idx, float v) {
  if (dt == DT_F16) ((_Float16*)base)[idx] = (_Float16)v;           // kv_store: half(v), round to nearest
  else ((uint16_t*)base)[idx] = f32_to_bf16_bits(v, false);
}

constexpr float kRmsEps = 1e-6f;   // cpu.rs:3, attention_device.metal:10

__global__ void __launch_bounds__(256) qk_rope_kv_kernel(const RopeParams p) {
  __shared__ float stage[4][512];
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t tok = blockIdx.x, h = blockIdx.y * 4 + wave;
  const uint32_t n_heads = p.hq + 2 * p.hkv;
  if (h >= n_heads) return;   // whole wave leaves; no barrier below involves it
  const uint32_t hd = p.hd;
  const bool is_q = h < p.hq, is_k = !is_q && h < p.hq + p.hkv;
  const uint32_t hh = is_q ? h : (h - p.hq) % p.hkv;
  const uint32_t pos = p.kv_len + tok;
  const bool kv_write = pos < p.kv_write_end;
  const int64_t slot = p.ring_mask ? (pos & p.ring_mask) : pos;

  uint16_t* row_inplace = is_q ? p.q + ((size_t)tok * p.hq + hh) * hd : p.k + ((size_t)tok * p.hkv + hh) * hd;
  const uint16_t* src = (is_q || is_k) ? row_inplace
                                       : (p.v_from_k ? p.k : p.v) + ((size_t)tok * p.hkv + hh) * hd;

  // lane owns elements [per*lane, per*lane + per), per = hd/64 (1 element for the first hd lanes if hd < 64)
  const uint32_t per = hd >= 64 ? hd / 64 : 1;
  const uint32_t d0 = lane * per;
  const bool active = d0 < hd;
  float x[8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x[i] = 0.f;
    if (active && (uint32_t)i < per) {
      x[i] = bf16_bits_to_f32(src[d0 + i]);
      ss += x[i] * x[i];
    }
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)hd + kRmsEps);
  if (lane == 0 && !(inv == inv && fabsf(inv) != INFINITY)) dbg_report(p.dbg, DG_DBG_ROPE_NONFINITE, (tok << 16) | h, __float_as_uint(inv));

  if (!is_q && !is_k) {   // V: normalise without weight, write to the cache (cpu.rs:110-122)
    if (kv_write && active) {
      const int64_t base = slot * p.v_tok_stride + (int64_t)hh * p.v_head_stride;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if ((uint32_t)i < per) store_cache(p.vc, p.kv_dtype, base + d0 + i, x[i] * inv);
    }
    return;
  }

  const uint16_t* w = is_q ? p.qw : p.kw;
  float* st = stage[wave];
#pragma unroll
  for (int i = 0; i < 8; ++i)
    if (active && (uint32_t)i < per) {
      x[i] *= inv * bf16_bits_to_f32(w[d0 + i]);   // x * (inv * w), the CPU twin's order (cpu.rs:71-74)
      st[d0 + i] = x[i];
    }
  __builtin_amdgcn_wave_barrier();   // the stage is private to the wave, whose LDS operations execute in order

  // rotation (cpu.rs:31-65): split-half pairs (d, d + rot/2) over the whole head with theta 1e4;
  // proportional pairs (d, hd/2 + d) for d < rot/2 = hd/8 with theta 1e6, the rest is left alone
  const uint32_t half_rot = p.is_full ? hd / 8 : hd / 2;
  const uint32_t partner_off = hd / 2;     // both schemes pair d with d + hd/2 (split-half: rot/2 = hd/2)
  float y[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    y[i] = x[i];
    if (active && (uint32_t)i < per) {
      const uint32_t d = d0 + i;
      const bool first = d < half_rot, second = d >= partner_off && d < partner_off + half_rot;
      if (first || second) {
        const uint32_t dd = first ? d : d - partner_off;
        const float a = (float)pos * p.inv_freq[dd];
        const float c = cosf(a), s = sinf(a);
        const float x0 = st[dd], x1 = st[dd + partner_off];
        y[i] = first ? x0 * c - x1 * s : x0 * s + x1 * c;
      }
    }
  }
  if (!active) return;
  if (is_k && kv_write) {
    const int64_t base = slot * p.k_tok_stride + (int64_t)hh * p.k_head_stride;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if ((uint32_t)i < per) store_cache(p.kc, p.kv_dtype, base + d0 + i, y[i]);
  }
  // Q always goes back in place; K only when V does not alias the raw k projection (cpu.rs:137-143)
  if (is_q || !p.v_from_k) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if ((uint32_t)i < per) row_inplace[d0 + i] = f32_to_bf16_bits(y[i], p.qk_trunc != 0);
  }
}

}  // namespace
}  // namespace dg

extern "C" {

int dg_qk_rope_kv(const dg_rope_desc* d, void* q, void* k, const void* v, void* kv_base, const void* q_norm_w,
                  const void* k_norm_w, dg_debug_status* dbg, void* stream) {
  if (!d || !q || !k || !kv_base || !q_norm_w || !k_norm_w) return DG_ERR_NULL;
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
  hipLaunchKernelGGL(dg::qk_rope_kv_kernel, dim3(d->canvas, (n_heads + 3) / 4), dim3(256), 0, (hipStream_t)stream, p);
  return hipGetLastError() == hipSuccess ? DG_OK : DG_ERR_LAUNCH;
}

int dg_qk_rope_kv_dispatch(void* q, void* k, void* v, void* kvcache, const void* blob, const dg_layer_offsets* L,
                           const dg_step_params* P, const dg_attn_dims* dims, dg_debug_status* dbg, void* stream) {
  if (!L || !P || !dims || !blob) return DG_ERR_NULL;
  dg_rope_desc d{};
  d.canvas = dims->canvas;
  d.n_q_heads = dims->n_q_heads;
  d.n_kv_heads = L->n_kv_heads;
  d.head_dim = L->head_dim;
  d.kv_len = P->kv_len;
  d.kv_write_end = P->kv_write_end;
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
  return dg_qk_rope_kv(&d, q, k, v, kvcache, (const char*)blob + L->q_norm, (const char*)blob + L->k_norm, dbg, stream);
}

}  // extern "C"
