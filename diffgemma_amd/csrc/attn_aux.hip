// Auxiliary kernels: the scalar cross-check kernel, the split merge, dtype conversion.
#include "attn_params.h"
#include "wt_store.h"

#include <hip/hip_fp16.h>

namespace dg {

namespace {

template <typename T>
__device__ __forceinline__ float load_elem(const T* p, int64_t i);
template <>
__device__ __forceinline__ float load_elem<uint16_t>(const uint16_t* p, int64_t i) {  // bf16 bits
  return bf16_bits_to_f32(p[i]);
}
template <>
__device__ __forceinline__ float load_elem<_Float16>(const _Float16* p, int64_t i) {
  return (float)p[i];
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// NaN or infinity (a comparison with NaN is false)
__device__ __forceinline__ bool nonfinite(float y) { return !(fabsf(y) <= 3.402823466e38f); }

__device__ __forceinline__ void store_out(const AttnParams& p, size_t idx, float y) {
  if (p.out_dtype == DT_F32) {
    ((float*)p.out)[idx] = y;
  } else if (p.out_dtype == DT_BF16) {
    ((uint16_t*)p.out)[idx] = f32_to_bf16_bits(y, p.out_trunc != 0);
  } else {
    ((_Float16*)p.out)[idx] = (_Float16)y;
  }
}

// One wave per (canvas row, query head); keys streamed one at a time with the online
// softmax recurrence.  Slow on purpose: it shares nothing with the MFMA kernel except the
// mask arithmetic, which is what makes it a useful on-device cross-check.
template <typename KT>
__global__ void __launch_bounds__(64) attn_scalar_kernel(const AttnParams p, const uint32_t hd) {
  const uint32_t tok = blockIdx.x, qh = blockIdx.y, lane = threadIdx.x;
  const uint32_t kvh = qh / p.group;
  const RowBounds b = row_bounds(p, tok);
  const KT* kbase = (const KT*)p.k + (int64_t)kvh * p.k_head_stride;
  const KT* vbase = (const KT*)p.v + (int64_t)kvh * p.v_head_stride;
  const size_t qoff = ((size_t)tok * p.hq + qh) * hd;
  float qv[8], acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t d = lane + 64u * i;
    acc[i] = 0.f;
    qv[i] = 0.f;
    if (d < hd) {
      qv[i] = p.q_is_bf16 ? bf16_bits_to_f32(((const uint16_t*)p.q)[qoff + d])
                          : load_elem<KT>((const KT*)p.q, (int64_t)(qoff + d));
    }
  }
  float m = -INFINITY, l = 0.f;
  for (uint32_t t = b.lo; t < p.t_clip_hi; ++t) {
    if (!key_visible(b, t, p.t_clip_hi)) {
      if (t >= b.hi && b.extra >= p.t_clip_hi) break;
      continue;
    }
    const int64_t slot = kv_slot(p.ring_mask, t);
    const KT* kk = kbase + slot * p.k_tok_stride;
    const KT* vv = vbase + slot * p.v_tok_stride;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t d = lane + 64u * i;
      if (d < hd) s += qv[i] * load_elem<KT>(kk, d);
    }
    s = wave_sum(s) * p.scale_log2;
    const float mn = fmaxf(m, s);
    const float corr = exp2f(m - mn);
    const float pr = exp2f(s - mn);
    l = l * corr + pr;
    m = mn;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t d = lane + 64u * i;
      if (d < hd) acc[i] = acc[i] * corr + pr * load_elem<KT>(vv, d);
    }
  }
  if (lane == 0) {
    if (!(l > 0.f)) dbg_report(p.dbg, DBG_ERR_SOFTMAX_NORM_ZERO, DBG_KERNEL_ATTENTION, (tok << 16) | qh, (tok << 16) | qh);
    if (p.lse) p.lse[(size_t)tok * p.hq + qh] = l > 0.f ? m * kLn2 + logf(l) : -INFINITY;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t d = lane + 64u * i;
    if (d < hd) {
      const float y = l > 0.f ? acc[i] / l : 0.f;
      if (p.dbg && nonfinite(y)) dbg_report(p.dbg, DBG_ERR_NONFINITE, DBG_KERNEL_ATTENTION, (tok << 16) | qh, d);
      store_out(p, qoff + d, y);
    }
  }
}

// One wave per stacked row: combines the per-split (m, l, O) triples.
// The split weights are worked out first (they are the same for the whole row); the O partials
// are then streamed with four splits' loads in flight per lane, which is what lets the kernel
// run at memory speed: the partials of a 32k-prefix global layer are tens of megabytes.
static_assert(kMaxSplits <= 64, "one lane per split");
__global__ void __launch_bounds__(256) attn_merge_kernel(const AttnParams p, const uint32_t hd) {
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t gr = blockIdx.x * 4 + wave;  // global stacked row over all KV heads
  if (gr >= p.hkv * p.rows_total) return;
  const uint32_t kvh = gr / p.rows_total, r = gr % p.rows_total;
  const uint32_t tok = r / p.group, qh = kvh * p.group + r % p.group;
  const size_t split_stride = (size_t)p.hkv * p.rows_pad;
  const size_t row = (size_t)kvh * p.rows_pad + r;
  // lane s holds split s's (m, l); the row's weights come from wave reductions
  float ms = -INFINITY, ls = 0.f;
  if (lane < p.n_splits) {
    const float2 ml = *(const float2*)(p.part_ml + ((size_t)lane * split_stride + row) * 2);
    ms = ml.x;
    ls = ml.y;
  }
  float mx = ms;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  float wl = ls > 0.f ? ls * exp2f(ms - mx) : 0.f;   // l_s * 2^(m_s - m)
  const float den = wave_sum(wl);
  const float inv = den > 0.f ? 1.f / den : 0.f;
  const float w_mine = ls > 0.f ? exp2f(ms - mx) * inv : 0.f;   // weight of split `lane`
  const size_t ooff = ((size_t)tok * p.hq + qh) * hd;
  const size_t sstride = split_stride * hd;
  if (p.part_half) {
    // normalised f16 partial rows: O = sum_s (l_s 2^(m_s - m) / den) O_s; eight d per lane and load
    const float w_half = wl * inv;
    const uint16_t* const hbase = (const uint16_t*)p.part_o + row * hd;
    // (every lane runs the loop, idle ones on chunk 0: the weight shuffles below read lanes
    // that would otherwise be switched off when head_dim / 8 is below the split count)
    for (uint32_t d8_0 = 0; d8_0 < hd / 8; d8_0 += 64) {
      const bool live = d8_0 + lane < hd / 8;
      const uint32_t d8 = live ? d8_0 + lane : 0u;
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      // Splits whose weight is below 2^-24 of the row's total are left out: what they would add is
      // under the fp32 rounding of the sum (the weights add up to 1, |O_s| <= the largest |V|), and
      // on a peaked row, where one split holds nearly all of the mass, most of the partial rows are
      // then never fetched.  The others are summed in ascending order, four loads in flight.
      uint64_t todo = __builtin_amdgcn_ballot_w64(lane < p.n_splits && w_half >= 5.9604645e-8f);
      while (todo != 0ull) {
        uint32_t idx[4];
        uint32_t cnt = 0;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          idx[u] = todo != 0ull ? (uint32_t)__builtin_ctzll(todo) : idx[0];
          cnt += todo != 0ull ? 1u : 0u;
          todo &= todo - 1ull;
        }
        uint4 a[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) a[u] = ((const uint4*)(hbase + idx[u] * sstride))[d8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if ((uint32_t)u >= cnt) break;
          const float w = __shfl(w_half, (int)idx[u], 64);
          const uint32_t wd[4] = {a[u].x, a[u].y, a[u].z, a[u].w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            acc[2 * e] += w * (float)__builtin_bit_cast(_Float16, (uint16_t)(wd[e] & 0xffffu));
            acc[2 * e + 1] += w * (float)__builtin_bit_cast(_Float16, (uint16_t)(wd[e] >> 16));
          }
        }
      }
      if (!live) continue;
      if (p.dbg) {
        bool bad = false;
#pragma unroll
        for (int e = 0; e < 8; ++e) bad = bad || nonfinite(acc[e]);
        if (bad) dbg_report(p.dbg, DBG_ERR_NONFINITE, DBG_KERNEL_ATTENTION, (tok << 16) | qh, d8 * 8u);
      }
      if (p.out_dtype == DT_BF16) {   // eight bf16 in one 16-byte store
        const bool tr = p.out_trunc != 0;
        uint4 pk;
        pk.x = (uint32_t)f32_to_bf16_bits(acc[0], tr) | ((uint32_t)f32_to_bf16_bits(acc[1], tr) << 16);
        pk.y = (uint32_t)f32_to_bf16_bits(acc[2], tr) | ((uint32_t)f32_to_bf16_bits(acc[3], tr) << 16);
        pk.z = (uint32_t)f32_to_bf16_bits(acc[4], tr) | ((uint32_t)f32_to_bf16_bits(acc[5], tr) << 16);
        pk.w = (uint32_t)f32_to_bf16_bits(acc[6], tr) | ((uint32_t)f32_to_bf16_bits(acc[7], tr) << 16);
        const wt_u32x4 pk4 = {pk.x, pk.y, pk.z, pk.w};
        wt_store16(wt_window_wave((const uint16_t*)p.out + ooff), d8 * 16u, pk4);   // written through: wt_store.h
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) store_out(p, ooff + d8 * 8 + e, acc[e]);
      }
    }
    if (lane == 0) {
      if (!(den > 0.f)) dbg_report(p.dbg, DBG_ERR_SOFTMAX_NORM_ZERO, DBG_KERNEL_ATTENTION, (tok << 16) | qh, (tok << 16) | qh);
      if (p.lse) p.lse[(size_t)tok * p.hq + qh] = den > 0.f ? mx * kLn2 + logf(den) : -INFINITY;
    }
    return;
  }
  const float* const base = p.part_o + row * hd;
  for (uint32_t d4_0 = 0; d4_0 < hd / 4; d4_0 += 64) {   // idle lanes run along, see above
    const bool live = d4_0 + lane < hd / 4;
    const uint32_t d4 = live ? d4_0 + lane : 0u;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    uint32_t s = 0;
    for (; s + 4 <= p.n_splits; s += 4) {
      const float4 a0 = ((const float4*)(base + (s + 0) * sstride))[d4];
      const float4 a1 = ((const float4*)(base + (s + 1) * sstride))[d4];
      const float4 a2 = ((const float4*)(base + (s + 2) * sstride))[d4];
      const float4 a3 = ((const float4*)(base + (s + 3) * sstride))[d4];
      const float w0 = __shfl(w_mine, s + 0, 64), w1 = __shfl(w_mine, s + 1, 64);
      const float w2 = __shfl(w_mine, s + 2, 64), w3 = __shfl(w_mine, s + 3, 64);
      o.x += w0 * a0.x + w1 * a1.x + w2 * a2.x + w3 * a3.x;
      o.y += w0 * a0.y + w1 * a1.y + w2 * a2.y + w3 * a3.y;
      o.z += w0 * a0.z + w1 * a1.z + w2 * a2.z + w3 * a3.z;
      o.w += w0 * a0.w + w1 * a1.w + w2 * a2.w + w3 * a3.w;
    }
    for (; s < p.n_splits; ++s) {
      const float4 a = ((const float4*)(base + s * sstride))[d4];
      const float w = __shfl(w_mine, s, 64);
      o.x += w * a.x;
      o.y += w * a.y;
      o.z += w * a.z;
      o.w += w * a.w;
    }
    if (!live) continue;
    if (p.dbg && (nonfinite(o.x) || nonfinite(o.y) || nonfinite(o.z) || nonfinite(o.w)))
      dbg_report(p.dbg, DBG_ERR_NONFINITE, DBG_KERNEL_ATTENTION, (tok << 16) | qh, d4 * 4u);
    if (p.out_dtype == DT_F32) {
      const wt_u32x4 o4 = {__float_as_uint(o.x), __float_as_uint(o.y), __float_as_uint(o.z), __float_as_uint(o.w)};
      wt_store16(wt_window_wave((const float*)p.out + ooff), d4 * 16u, o4);
    } else if (p.out_dtype == DT_BF16) {   // four bf16 in one 8-byte store
      const bool tr = p.out_trunc != 0;
      uint2 pk;
      pk.x = (uint32_t)f32_to_bf16_bits(o.x, tr) | ((uint32_t)f32_to_bf16_bits(o.y, tr) << 16);
      pk.y = (uint32_t)f32_to_bf16_bits(o.z, tr) | ((uint32_t)f32_to_bf16_bits(o.w, tr) << 16);
      const wt_u32x2 pk2 = {pk.x, pk.y};
      wt_store8(wt_window_wave((const uint16_t*)p.out + ooff), d4 * 8u, pk2);
    } else {
      store_out(p, ooff + d4 * 4 + 0, o.x);
      store_out(p, ooff + d4 * 4 + 1, o.y);
      store_out(p, ooff + d4 * 4 + 2, o.z);
      store_out(p, ooff + d4 * 4 + 3, o.w);
    }
  }
  if (lane == 0) {
    if (!(den > 0.f)) dbg_report(p.dbg, DBG_ERR_SOFTMAX_NORM_ZERO, DBG_KERNEL_ATTENTION, (tok << 16) | qh, (tok << 16) | qh);
    if (p.lse) p.lse[(size_t)tok * p.hq + qh] = den > 0.f ? mx * kLn2 + logf(den) : -INFINITY;
  }
}

// The same merge for at most 8 splits of f16 partial rows whose total is small (a sliding layer:
// 6 splits x 4096 rows x 512 bytes): there the kernel is as long as one wave's chain of memory round
// trips, not bandwidth.  So a wave asks for everything at once, the (m, l) pairs and the partial rows
// of all splits (an absent split repeats the last one, weight zero), instead of weights first and
// only the rows of splits that count; and the weights come from lane-to-scalar reads, every lane
// doing the same arithmetic, instead of a dozen dependent shuffles.  The sum of the weights pairs
// its terms as the butterfly over the lanes does, ((0+4)+(2+6))+((1+5)+(3+7)), and the rows are
// added in the same order with the same cut, so both kernels give the same bits.
constexpr uint32_t kMergeFewSplits = 8;
__global__ void __launch_bounds__(256) attn_merge_few_kernel(const AttnParams p, const uint32_t hd) {
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t gr = blockIdx.x * 4 + wave;  // global stacked row over all KV heads
  if (gr >= p.hkv * p.rows_total) return;
  const uint32_t kvh = gr / p.rows_total, r = gr % p.rows_total;
  const uint32_t tok = r / p.group, qh = kvh * p.group + r % p.group;
  const size_t split_stride = (size_t)p.hkv * p.rows_pad;
  const size_t row = (size_t)kvh * p.rows_pad + r;
  const uint32_t n = p.n_splits;
  const float2 ml = *(const float2*)(p.part_ml + ((size_t)min(lane, n - 1u) * split_stride + row) * 2);
  const bool live = lane < hd / 8;
  const uint32_t d8 = live ? lane : 0u;
  const uint16_t* const hbase = (const uint16_t*)p.part_o + row * hd;
  const size_t sstride = split_stride * hd;
  uint4 a[kMergeFewSplits];
#pragma unroll
  for (uint32_t u = 0; u < kMergeFewSplits; ++u) a[u] = ((const uint4*)(hbase + min(u, n - 1u) * sstride))[d8];
  float msu[kMergeFewSplits], wlu[kMergeFewSplits];
  float mx = -INFINITY;
#pragma unroll
  for (uint32_t u = 0; u < kMergeFewSplits; ++u) {
    msu[u] = u < n ? __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(ml.x), (int)u)) : -INFINITY;
    mx = fmaxf(mx, msu[u]);
  }
#pragma unroll
  for (uint32_t u = 0; u < kMergeFewSplits; ++u) {
    const float lsu = u < n ? __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(ml.y), (int)u)) : 0.f;
    wlu[u] = lsu > 0.f ? lsu * exp2f(msu[u] - mx) : 0.f;
  }
  const float den = ((wlu[0] + wlu[4]) + (wlu[2] + wlu[6])) + ((wlu[1] + wlu[5]) + (wlu[3] + wlu[7]));
  const float inv = den > 0.f ? 1.f / den : 0.f;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (uint32_t u = 0; u < kMergeFewSplits; ++u) {
    const float w = wlu[u] * inv;
    if (u < n && w >= 5.9604645e-8f) {   // the same in every lane
      const uint32_t wd[4] = {a[u].x, a[u].y, a[u].z, a[u].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] += w * (float)__builtin_bit_cast(_Float16, (uint16_t)(wd[e] & 0xffffu));
        acc[2 * e + 1] += w * (float)__builtin_bit_cast(_Float16, (uint16_t)(wd[e] >> 16));
      }
    }
  }
  const size_t ooff = ((size_t)tok * p.hq + qh) * hd;
  if (live) {
    if (p.dbg) {
      bool bad = false;
#pragma unroll
      for (int e = 0; e < 8; ++e) bad = bad || nonfinite(acc[e]);
      if (bad) dbg_report(p.dbg, DBG_ERR_NONFINITE, DBG_KERNEL_ATTENTION, (tok << 16) | qh, d8 * 8u);
    }
    if (p.out_dtype == DT_BF16) {
      const bool tr = p.out_trunc != 0;
      const wt_u32x4 pk4 = {(uint32_t)f32_to_bf16_bits(acc[0], tr) | ((uint32_t)f32_to_bf16_bits(acc[1], tr) << 16),
                            (uint32_t)f32_to_bf16_bits(acc[2], tr) | ((uint32_t)f32_to_bf16_bits(acc[3], tr) << 16),
                            (uint32_t)f32_to_bf16_bits(acc[4], tr) | ((uint32_t)f32_to_bf16_bits(acc[5], tr) << 16),
                            (uint32_t)f32_to_bf16_bits(acc[6], tr) | ((uint32_t)f32_to_bf16_bits(acc[7], tr) << 16)};
      wt_store16(wt_window_wave((const uint16_t*)p.out + ooff), d8 * 16u, pk4);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) store_out(p, ooff + d8 * 8 + e, acc[e]);
    }
  }
  if (lane == 0) {
    if (!(den > 0.f)) dbg_report(p.dbg, DBG_ERR_SOFTMAX_NORM_ZERO, DBG_KERNEL_ATTENTION, (tok << 16) | qh, (tok << 16) | qh);
    if (p.lse) p.lse[(size_t)tok * p.hq + qh] = den > 0.f ? mx * kLn2 + logf(den) : -INFINITY;
  }
}

__device__ __forceinline__ float load_any(const void* src, uint32_t dt, size_t i) {
  if (dt == DT_F32) return ((const float*)src)[i];
  if (dt == DT_BF16) return bf16_bits_to_f32(((const uint16_t*)src)[i]);
  return (float)((const _Float16*)src)[i];
}
// f32 -> f16 the way the reference's host wrapper rounds what it puts into the cache
// (src/shaders/common/f16.rs:28-47): clamp to +-65504, flush subnormals to a signed zero, truncate
// the mantissa; NaN stays NaN.
__device__ __forceinline__ uint16_t f32_to_f16_bits_trunc(float v) {
  const uint32_t raw = __float_as_uint(v);
  const uint32_t sign = (raw >> 16) & 0x8000u;
  if (v != v) return (uint16_t)(sign | 0x7E00u);
  const uint32_t bits = __float_as_uint(fminf(fmaxf(v, -65504.f), 65504.f));
  const int32_t new_exp = (int32_t)((bits >> 23) & 0xffu) - 127 + 15;
  if (new_exp <= 0) return (uint16_t)sign;
  return (uint16_t)(sign | ((uint32_t)new_exp << 10) | ((bits & 0x7fffffu) >> 13));
}
// f32 sources are rounded like the reference's wrapper around its CPU attention does
// (src/shaders/attn/attention/mod.rs:218-240): bf16 and f16 by truncation.  16-bit sources are
// copied exactly when the types match and widened/narrowed by the hardware conversion otherwise.
__device__ __forceinline__ void store_any(void* dst, uint32_t dt, size_t i, float v, bool from_f32) {
  if (dt == DT_F32) ((float*)dst)[i] = v;
  else if (dt == DT_BF16) ((uint16_t*)dst)[i] = f32_to_bf16_bits(v, from_f32);
  else if (from_f32) ((uint16_t*)dst)[i] = f32_to_f16_bits_trunc(v);
  else ((_Float16*)dst)[i] = (_Float16)v;
}

__global__ void convert_kernel(const void* src, uint32_t sdt, void* dst, uint32_t ddt, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    store_any(dst, ddt, i, load_any(src, sdt, i), sdt == DT_F32);
}

__global__ void kv_gather_kernel(const void* src, uint32_t sdt, void* dst, uint32_t ddt, uint32_t hkv,
                                 uint32_t t_all, uint32_t hd, int64_t tok_stride, int64_t head_stride,
                                 uint32_t ring_mask) {
  const size_t n = (size_t)hkv * t_all * hd;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const uint32_t d = (uint32_t)(i % hd);
    const uint32_t t = (uint32_t)((i / hd) % t_all);
    const uint32_t h = (uint32_t)(i / ((size_t)hd * t_all));
    const int64_t s = (int64_t)kv_slot(ring_mask, t) * tok_stride + (int64_t)h * head_stride + d;
    store_any(dst, ddt, i, load_any(src, sdt, (size_t)s), sdt == DT_F32);
  }
}

// plain 16-byte copy of known size: the yardstick the HBM byte counters are scaled by
__global__ void calib_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// Nothing but MFMAs: four independent 32x32x16 bf16 accumulators per wave, one wave per SIMD.
// What this sustains is the ceiling the attention kernel's MFMA rate is compared with on the
// machine at hand.  The published peak assumes the maximum clock; the clock the chip holds
// depends on the power the multipliers draw, which depends on the operand values: with
// RANDOM operands (eight fragments per side of sign/exponent/mantissa noise around unit
// magnitude, cycled) the same instruction stream runs at a clearly lower clock than with the
// near-constant ones.
typedef float calib_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 calib_bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t calib_u32x4 __attribute__((ext_vector_type(4)));
// MODE 0: near-constant operands; 1: random; 2 / 3: random, with 3 of 4 / 19 of 20 elements of
// the B operand zero (what the probabilities of a long attention row look like once negligible
// weights are dropped).
template <int MODE>
__global__ void __launch_bounds__(256) calib_mfma_kernel(float* sink, uint32_t iters) {
  constexpr bool RANDOM = MODE != 0;
  calib_u32x4 a[8], b[8];
  uint32_t seed = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  auto noise_pair = [&]() -> uint32_t {   // two bf16 of random sign, magnitude in [2^-7, 2)
    seed ^= seed << 13;
    seed ^= seed >> 17;
    seed ^= seed << 5;
    const uint32_t lo = ((seed & 1u) << 15) | ((120u + ((seed >> 1) & 7u)) << 7) | ((seed >> 4) & 0x7fu);
    const uint32_t hi = (((seed >> 11) & 1u) << 15) | ((120u + ((seed >> 12) & 7u)) << 7) | ((seed >> 15) & 0x7fu);
    return lo | (hi << 16);
  };
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // near-constant: 1 + k/128 and 1/2 - k/256 for small k (a few mantissa bits set)
      a[i][e] = RANDOM ? noise_pair() : 0x3f803f80u + ((threadIdx.x + e) & 3u);
      b[i][e] = RANDOM ? noise_pair() : 0x3f003f00u - ((threadIdx.x * 3u + e) & 3u);
      if (MODE >= 2) {   // zero each half of the pair with probability 3/4 or 19/20
        const uint32_t keep = MODE == 2 ? 64u : 13u;   // of 256
        const uint32_t r = noise_pair();
        if ((r & 255u) >= keep) b[i][e] &= 0xffff0000u;
        if (((r >> 8) & 255u) >= keep) b[i][e] &= 0x0000ffffu;
      }
    }
#pragma unroll
  for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(a[i]), "+v"(b[i]));   // keep sixteen distinct fragments
  calib_f32x16 c0, c1, c2, c3;
#pragma unroll
  for (int e = 0; e < 16; ++e) c0[e] = c1[e] = c2[e] = c3[e] = 0.f;
  auto fa = [&](int i) { return __builtin_bit_cast(calib_bf16x8, a[i & 7]); };
  auto fb = [&](int i) { return __builtin_bit_cast(calib_bf16x8, b[(i * 3) & 7]); };
  for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa(4 * u), fb(4 * u), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa(4 * u + 1), fb(4 * u + 1), c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa(4 * u + 2), fb(4 * u + 2), c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa(4 * u + 3), fb(4 * u + 3), c3, 0, 0, 0);
    }
  }
  float acc = 0.f;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc += c0[e] + c1[e] + c2[e] + c3[e];
  if (acc == 123.456f) sink[blockIdx.x * 256 + threadIdx.x] = acc;   // keeps the MFMAs alive
}

}  // namespace

hipError_t launch_calib_mfma(float* sink, uint32_t workgroups, uint32_t iters, uint32_t operand_mode, hipStream_t s) {
  const dim3 grid(workgroups), block(256);
  switch (operand_mode) {
    case 0: hipLaunchKernelGGL(calib_mfma_kernel<0>, grid, block, 0, s, sink, iters); break;
    case 1: hipLaunchKernelGGL(calib_mfma_kernel<1>, grid, block, 0, s, sink, iters); break;
    case 2: hipLaunchKernelGGL(calib_mfma_kernel<2>, grid, block, 0, s, sink, iters); break;
    case 3: hipLaunchKernelGGL(calib_mfma_kernel<3>, grid, block, 0, s, sink, iters); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_calib_copy(void* dst, const void* src, size_t bytes, hipStream_t s) {
  const size_t n16 = bytes / 16;
  if (n16 == 0) return hipSuccess;
  hipLaunchKernelGGL(calib_copy_kernel, dim3(4096), dim3(256), 0, s, (const uint4*)src, (uint4*)dst, n16);
  return hipGetLastError();
}

hipError_t launch_attn_scalar(const AttnParams& p, uint32_t head_dim, uint32_t kv_dtype, hipStream_t s) {
  dim3 grid(p.canvas, p.hq, 1), block(64, 1, 1);
  if (kv_dtype == DT_BF16)
    hipLaunchKernelGGL(attn_scalar_kernel<uint16_t>, grid, block, 0, s, p, head_dim);
  else
    hipLaunchKernelGGL(attn_scalar_kernel<_Float16>, grid, block, 0, s, p, head_dim);
  return hipGetLastError();
}

// One wave per (canvas row, query head): the closed form  m = max m_i,  l = sum l_i e^(m_i - m),
// acc = sum acc_i e^(m_i - m)  over the states that saw a key, written as the final row (acc / l)
// and/or as a state again, in the normal form (m + ln l, 1, acc / l).
__global__ void __launch_bounds__(256) attn_state_merge_kernel(const StateMergeParams p) {
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * 4 + wave;
  if (row >= p.rows) return;
  // The (m, l) pairs of the row are read once, before anything is written: state_out may be one of the
  // inputs, and lane 0 overwrites the row's (m, l) there at the end.  Every lane derives the same
  // weights from them and keeps them in registers for the accumulator loop.
  float w[kMaxStates], lw[kMaxStates];
  float mx = -INFINITY;
#pragma unroll
  for (uint32_t i = 0; i < kMaxStates; ++i) {
    w[i] = -INFINITY;   // the exponent m for now; a state that saw no key of the row does not count
    lw[i] = 0.f;
    if (i < p.n) {
      const float m_i = p.states[i][row], l_i = p.states[i][p.rows + row];
      if (l_i > 0.f) {
        w[i] = m_i;
        lw[i] = l_i;
      }
    }
    mx = fmaxf(mx, w[i]);
  }
  float den = 0.f;
#pragma unroll
  for (uint32_t i = 0; i < kMaxStates; ++i) {
    w[i] = lw[i] > 0.f ? __expf(w[i] - mx) : 0.f;   // weight of the state's accumulators
    den += lw[i] * w[i];
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  const size_t acc0 = state_acc_offset(p.rows) + (size_t)row * p.hd;
  for (uint32_t d = lane * 4u; d < p.hd; d += 256u) {
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (uint32_t i = 0; i < kMaxStates; ++i) {
      if (i >= p.n || lw[i] == 0.f) continue;   // the same in every lane
      const float4 a = *(const float4*)(p.states[i] + acc0 + d);
      o.x = __builtin_fmaf(w[i], a.x, o.x);
      o.y = __builtin_fmaf(w[i], a.y, o.y);
      o.z = __builtin_fmaf(w[i], a.z, o.z);
      o.w = __builtin_fmaf(w[i], a.w, o.w);
    }
    o.x *= inv; o.y *= inv; o.z *= inv; o.w *= inv;
    if (p.dbg && (nonfinite(o.x) || nonfinite(o.y) || nonfinite(o.z) || nonfinite(o.w)))
      dbg_report(p.dbg, DBG_ERR_NONFINITE, DBG_KERNEL_ATTENTION, ((row / p.hq) << 16) | (row % p.hq), d);
    if (p.state_out) *(float4*)(p.state_out + acc0 + d) = o;
    if (p.out) {
      const size_t idx = (size_t)row * p.hd + d;
      if (p.out_dtype == DT_F32) {
        *(float4*)((float*)p.out + idx) = o;
      } else if (p.out_dtype == DT_BF16) {
        const bool tr = p.out_trunc != 0;
        uint2 pk;
        pk.x = (uint32_t)f32_to_bf16_bits(o.x, tr) | ((uint32_t)f32_to_bf16_bits(o.y, tr) << 16);
        pk.y = (uint32_t)f32_to_bf16_bits(o.z, tr) | ((uint32_t)f32_to_bf16_bits(o.w, tr) << 16);
        *(uint2*)((uint16_t*)p.out + idx) = pk;
      } else {
        _Float16* const h = (_Float16*)p.out + idx;
        h[0] = (_Float16)o.x; h[1] = (_Float16)o.y; h[2] = (_Float16)o.z; h[3] = (_Float16)o.w;
      }
    }
  }
  if (lane == 0) {
    const float lse = den > 0.f ? mx + __logf(den) : -INFINITY;
    const uint32_t tag = ((row / p.hq) << 16) | (row % p.hq);
    if (p.dbg && p.out && !(den > 0.f)) dbg_report(p.dbg, DBG_ERR_SOFTMAX_NORM_ZERO, DBG_KERNEL_ATTENTION, tag, tag);
    if (p.lse) p.lse[row] = lse;
    if (p.state_out) {
      p.state_out[row] = lse;
      p.state_out[p.rows + row] = den > 0.f ? 1.f : 0.f;
    }
  }
}

__global__ void __launch_bounds__(256) state_unit_l_kernel(const float* m_plane, float* l_plane, uint32_t rows) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i < rows) l_plane[i] = m_plane[i] == -INFINITY ? 0.f : 1.f;   // (a NaN stays visible: l = 1)
}

hipError_t launch_state_unit_l(float* m_plane, float* l_plane, uint32_t rows, hipStream_t s) {
  hipLaunchKernelGGL(state_unit_l_kernel, dim3((rows + 255) / 256), dim3(256), 0, s, m_plane, l_plane, rows);
  return hipGetLastError();
}

hipError_t launch_state_merge(const StateMergeParams& p, hipStream_t s) {
  hipLaunchKernelGGL(attn_state_merge_kernel, dim3((p.rows + 3) / 4), dim3(256), 0, s, p);
  return hipGetLastError();
}

hipError_t launch_attn_merge(const AttnParams& p, uint32_t head_dim, bool streamed, hipStream_t s) {
  const uint32_t rows = p.hkv * p.rows_total;
  // a few splits of a small workspace: the variant that asks for every partial row up front
  const size_t part_bytes = (size_t)p.n_splits * p.hkv * p.rows_pad * head_dim * 2;
  if (!streamed && p.part_half && p.n_splits <= kMergeFewSplits && head_dim % 8 == 0 && head_dim <= 512 && part_bytes < ((size_t)32 << 20))
    hipLaunchKernelGGL(attn_merge_few_kernel, dim3((rows + 3) / 4), dim3(256), 0, s, p, head_dim);
  else
    hipLaunchKernelGGL(attn_merge_kernel, dim3((rows + 3) / 4), dim3(256), 0, s, p, head_dim);
  return hipGetLastError();
}

hipError_t launch_convert(const void* src, uint32_t sdt, void* dst, uint32_t ddt, size_t n, hipStream_t s) {
  if (n == 0) return hipSuccess;
  const size_t blocks = (n + 255) / 256;
  hipLaunchKernelGGL(convert_kernel, dim3((unsigned)(blocks > 4096 ? 4096 : blocks)), dim3(256), 0, s, src, sdt, dst,
                     ddt, n);
  return hipGetLastError();
}

hipError_t launch_kv_gather(const void* src, uint32_t sdt, void* dst, uint32_t ddt, uint32_t hkv, uint32_t t_all,
                            uint32_t hd, int64_t tok_stride, int64_t head_stride, uint32_t ring_mask,
                            hipStream_t s) {
  const size_t n = (size_t)hkv * t_all * hd;
  if (n == 0) return hipSuccess;
  const size_t blocks = (n + 255) / 256;
  hipLaunchKernelGGL(kv_gather_kernel, dim3((unsigned)(blocks > 8192 ? 8192 : blocks)), dim3(256), 0, s, src, sdt, dst,
                     ddt, hkv, t_all, hd, tok_stride, head_stride, ring_mask);
  return hipGetLastError();
}

}  // namespace dg
