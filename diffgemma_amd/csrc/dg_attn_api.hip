// extern "C" boundary of libdg_attn_hip.so: descriptor validation, launch planning, and the
// reference-shaped dispatch entry.  No allocation, no host synchronisation, no exceptions.
#include "../../include/dg_attn.h"
#include "../../include/dg_attn_bench.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <mutex>
#include <vector>

#include "attn_params.h"

namespace {

using dg::kMaxSplits;
constexpr size_t kAlign = 256;
// most key tiles (of 32 keys) a row tile may see for the one-launch kernel to be chosen.  Step time in us,
// one launch | split kernel + merge, 256-row canvas, 8 KV heads: head_dim 256: 40 tiles 19.8 | 23.4,
// 72 tiles 28.5 | 27.5, 104 tiles 37.8 | 28.7; head_dim 128: 40 tiles 12.7 | 15.1, 72 tiles 18.9 | 19.3,
// 104 tiles 25.0 | 21.4; head_dim 64: 40 tiles 11.6 | 13.4, 72 tiles 18.0 | 16.4.
#ifndef DG_WSPLIT_MAX_TILES
#define DG_WSPLIT_MAX_TILES 64
#endif
constexpr uint32_t kWsplitMaxTiles = DG_WSPLIT_MAX_TILES;
static_assert(kWsplitMaxTiles <= 64, "attn_wsplit.hip's leading reference for f16 probabilities is sized for at most 2048 keys per row");

inline size_t align_up(size_t x) { return (x + kAlign - 1) / kAlign * kAlign; }
inline uint32_t elem_size(uint32_t dt) { return dt == DG_F32 ? 4u : 2u; }
inline bool is_pow2(uint64_t x) { return x && !(x & (x - 1)); }

struct DeviceInfo {
  int checked = 0;  // 0 unknown, 1 ok, -1 wrong arch
  int cus = 256;
};

// Device memory of dg_attn_forward_static, the entry point that may not allocate: what
// dg_attn_forward takes as its workspace argument (split partial rows, converted copies of f32
// inputs) lives here instead.  Every device the library runs on holds its own copy at its own
// address until the process ends; the name below is only a host-side handle, the device address
// is looked up once per device (static_scratch_ptr) and that pointer is what kernels are given.
constexpr size_t kStaticScratchBytes = DG_ATTN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
void* g_scratch_ptr[64] = {};
DeviceInfo g_dev[64];
thread_local uint32_t* g_tls_dbg = nullptr;
std::mutex g_dev_mu;

// Which caches this thread's calls streamed lately, to tell whether a call's key/value rows can still be in the
// memory-side cache (256 MB on MI355X): a cache is taken to be cold when other caches of more than 200 MiB in total
// were streamed since its last use, or on its first use when it is large.  Decides only which instance of the
// head_dim 512 kernel runs (the one that touches tiles into the L2 ahead of their loads: same bits, other timing);
// under graph capture the decision recorded is the one made at capture.
struct CacheMemo {
  const void* region = nullptr;
  uint64_t streamed_at_last_use = 0;
};
thread_local CacheMemo g_memo[16];
thread_local uint64_t g_streamed = 0;

bool cache_is_cold(const void* region, uint64_t bytes) {
  int idx = -1, oldest = 0;
  for (int i = 0; i < 16; ++i) {
    if (g_memo[i].region == region) idx = i;
    if (g_memo[i].streamed_at_last_use < g_memo[oldest].streamed_at_last_use) oldest = i;
  }
  bool cold;
  if (idx < 0) {
    cold = bytes >= (32ull << 20);
    idx = oldest;
    g_memo[idx].region = region;
  } else {
    cold = g_streamed - g_memo[idx].streamed_at_last_use > (200ull << 20);
  }
  g_streamed += bytes;
  g_memo[idx].streamed_at_last_use = g_streamed;
  return cold;
}

struct ProfState {
  std::vector<hipEvent_t> ev;
  uint32_t used = 0;
  bool active = false;
};
thread_local ProfState g_prof;

int device_info(DeviceInfo* out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return DG_ERR_DEVICE;
  std::lock_guard<std::mutex> lock(g_dev_mu);
  DeviceInfo& di = g_dev[dev];
  if (di.checked == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return DG_ERR_DEVICE;
    di.checked = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
    di.cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }
  if (di.checked < 0) return DG_ERR_DEVICE;
  *out = di;
  return DG_OK;
}

// Compute units the launch plans are made for: those of the current device when it is a
// gfx950 part, else (no device: host-side sizing and tests) the 256 of an MI355X.  Sizing calls
// and launches use the same number, so a workspace sized by the library always fits its launch.
int plan_cus() {
  DeviceInfo di;
  return device_info(&di) == DG_OK ? di.cus : 256;
}

// Address of `scratch` on the current device, looked up the first time the device is seen.
int static_scratch_ptr(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return DG_ERR_DEVICE;
  std::lock_guard<std::mutex> lock(g_dev_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return DG_ERR_DEVICE;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return DG_OK;
}

// Everything the launch needs that can be derived on the host without a device.
struct Plan {
  uint32_t group = 0, rows_total = 0, n_mtiles = 0, rows_pad = 0;
  uint32_t t_all = 0, lo_nc = 0, extra_lo = 0, win_m1 = 0xffffffffu;
  uint32_t clip_lo = 0, clip_hi = 0;   // keys that count: [clip_lo, clip_hi); the whole range unless a partial is asked for
  uint32_t tile_first = 0, tile_end = 0, tiles_per_split = 0, n_splits = 1;
  uint32_t e_dtype = DG_BF16;   // element type the kernels compute in (bf16 or f16)
  bool convert_q = false, gather_kv = false, q_is_bf16 = false;
  bool scalar = false;
  bool wsplit = false;          // short key range, head_dim <= 256: keys split over the waves of a workgroup, one launch
  bool part_half = false;       // split partial rows travel as normalised f16 rows
  size_t off_q = 0, off_kv = 0, off_part_o = 0, off_part_ml = 0, total = 0;
  float scale = 1.0f;
};

int make_plan(const dg_attn_desc* d, int cus, Plan* pl, const uint32_t* key_range = nullptr) {
  if (!d) return DG_ERR_NULL;
  const uint32_t hd = d->head_dim;
  if (d->canvas == 0 || d->canvas > 65536 || d->n_q_heads == 0 || d->n_kv_heads == 0) return DG_ERR_SHAPE;
  if (d->n_q_heads % d->n_kv_heads != 0 || d->n_q_heads > 65535) return DG_ERR_SHAPE;
  if (d->kernel > DG_KERNEL_MFMA) return DG_ERR_UNSUPPORTED;
  pl->scalar = d->kernel == DG_KERNEL_SCALAR;
  if (pl->scalar) {
    if (hd == 0 || hd > 512 || hd % 8 != 0) return DG_ERR_SHAPE;
  } else if (hd != 32 && hd != 64 && hd != 128 && hd != 256 && hd != 512) {
    return DG_ERR_SHAPE;
  }
  if ((uint64_t)d->kv_len + d->canvas > 0x7fffffffull) return DG_ERR_SHAPE;
  // the kernels address query rows with 32-bit byte offsets
  if ((uint64_t)d->canvas * d->n_q_heads * hd * 2ull >= (1ull << 32)) return DG_ERR_SHAPE;
  if (d->q_dtype > DG_F32 || d->kv_dtype > DG_F32 || d->out_dtype > DG_F32) return DG_ERR_DTYPE;
  if (d->out_dtype == DG_F16) return DG_ERR_DTYPE;
  if (d->causal_rows > d->canvas) return DG_ERR_MASK;
  if (d->kv_ring_mask != 0) {
    if (!is_pow2((uint64_t)d->kv_ring_mask + 1) || d->kv_ring_mask + 1 < (uint32_t)dg::kBlockN) return DG_ERR_LAYOUT;
  }
  pl->t_all = d->kv_len + d->canvas;
  if ((d->flags & DG_ATTN_F_T_LO_EXPLICIT) && d->t_lo > pl->t_all) return DG_ERR_MASK;
  if (!(d->softmax_scale >= 0.0f)) return DG_ERR_MASK;
  pl->scale = d->softmax_scale == 0.0f ? 1.0f : d->softmax_scale;

  // element type: the cache decides; f32 anywhere is brought down to f16 first
  pl->e_dtype = d->kv_dtype == DG_BF16 ? DG_BF16 : DG_F16;
  pl->gather_kv = d->kv_dtype == DG_F32;
  if (d->q_dtype == DG_F32) {
    // f32 queries become bf16 by truncation, the reference wrapper's rounding of Q
    // (src/shaders/attn/attention/mod.rs:218-240), whatever the cache holds
    pl->convert_q = true;
    pl->q_is_bf16 = pl->e_dtype == DG_F16;
  } else if (d->q_dtype == DG_BF16 && pl->e_dtype == DG_F16) {
    pl->q_is_bf16 = true;  // bf16 activations over an f16 cache: the reference's own pairing
  } else if (d->q_dtype != pl->e_dtype) {
    return DG_ERR_DTYPE;   // f16 Q over a bf16 cache
  }

  if (!pl->gather_kv) {
    // rows must be 16-byte addressable for the direct-to-LDS loads
    const int64_t s[5] = {d->k_tok_stride, d->k_head_stride, d->v_base_off, d->v_tok_stride, d->v_head_stride};
    for (int64_t x : s)
      if (x < 0 || x % 8 != 0) return DG_ERR_LAYOUT;
    if (d->kv_region_bytes % 16 != 0) return DG_ERR_LAYOUT;
    if (d->k_tok_stride < (int64_t)hd || d->v_tok_stride < (int64_t)hd) return DG_ERR_LAYOUT;
    if (d->k_tok_stride * 2 * dg::kBlockN >= (1ll << 31) || d->v_tok_stride * 2 * dg::kBlockN >= (1ll << 31))
      return DG_ERR_LAYOUT;
  } else {
    if (d->k_tok_stride < 0 || d->k_head_stride < 0 || d->v_base_off < 0 || d->v_tok_stride < 0 ||
        d->v_head_stride < 0)
      return DG_ERR_LAYOUT;
  }

  pl->group = d->n_q_heads / d->n_kv_heads;
  pl->rows_total = d->canvas * pl->group;
  pl->n_mtiles = (pl->rows_total + dg::kBlockM - 1) / dg::kBlockM;
  pl->rows_pad = pl->n_mtiles * dg::kBlockM;

  // mask constants (reference rules, src/shaders/attn/attention/attention.metal:49-63)
  pl->win_m1 = d->window ? d->window - 1u : 0xffffffffu;
  pl->lo_nc = (d->window && d->kv_len > d->window - 1u) ? d->kv_len - (d->window - 1u) : 0u;
  if (d->flags & DG_ATTN_F_T_LO_EXPLICIT) pl->lo_nc = d->t_lo;
  pl->extra_lo = (d->flags & DG_ATTN_F_CAUSAL_SEES_MASKED) ? std::min(d->kv_len + d->causal_rows, pl->t_all) : pl->t_all;

  // key tiles any row can see
  uint32_t lo_all = 0xffffffffu;
  if (d->causal_rows < d->canvas) lo_all = std::min(lo_all, pl->lo_nc);
  if (d->causal_rows > 0) {
    const uint32_t qpos0 = d->kv_len;
    lo_all = std::min(lo_all, (d->window && qpos0 > d->window - 1u) ? qpos0 - (d->window - 1u) : 0u);
  }
  lo_all = std::min(lo_all, pl->t_all);
  // a ring must hold every visible position at once, or two of them share a slot
  if (d->kv_ring_mask != 0 && pl->t_all - lo_all > d->kv_ring_mask + 1u) return DG_ERR_LAYOUT;
  pl->clip_lo = 0;
  pl->clip_hi = pl->t_all;
  if (key_range) {
    if (key_range[0] > key_range[1]) return DG_ERR_MASK;
    pl->clip_lo = std::min(key_range[0], pl->t_all);
    pl->clip_hi = std::min(key_range[1], pl->t_all);
    lo_all = std::max(lo_all, pl->clip_lo);
  }
  pl->tile_first = lo_all / dg::kBlockN;
  pl->tile_end = std::max(pl->tile_first, (pl->clip_hi + dg::kBlockN - 1) / dg::kBlockN);
  const uint32_t ntiles = std::max(1u, pl->tile_end - pl->tile_first);

  // A short key range at head_dim <= 256 (a sliding-window layer) runs as one launch in which the four waves
  // of a workgroup split the keys and merge in LDS (attn_wsplit.hip): every workgroup then streams all keys
  // its rows see, which pays while that is a few thousand keys.  The span is what one 32-row tile sees, not
  // the union over the canvas (causal windowed rows each see window keys, the canvas window + canvas).
  {
    uint32_t span = 0;
    if (d->causal_rows < d->canvas) span = std::max(span, pl->t_all - std::min(pl->lo_nc, pl->t_all));
    if (d->causal_rows > 0) {
      uint32_t c = d->kv_len + d->causal_rows;
      if (d->window) c = std::min(c, d->window + dg::kBlockN);
      if (d->flags & DG_ATTN_F_CAUSAL_SEES_MASKED) c = pl->t_all;
      span = std::max(span, std::min(c, pl->t_all));
    }
    const uint32_t span_tiles = std::min(ntiles, span / dg::kBlockN + 2u);
    pl->wsplit = !pl->scalar && hd <= 256 && d->n_splits == 0 && !(d->flags & DG_ATTN_F_SPLIT_OVER_WORKGROUPS) &&
                 span_tiles <= kWsplitMaxTiles;
  }
  uint32_t splits = d->n_splits;
  if (pl->scalar || pl->wsplit) {
    splits = 1;
  } else if (splits == 0) {
    // enough workgroups for every CU, but no split shorter than 6 tiles: below that the partial
    // rows a split writes (and the merge reads back) cost more than the idle CUs do (a sliding
    // layer's 40 tiles, step in us: 4 splits 25.7, 5 splits 24.8, 6 and 7 splits 23.7, 8 splits 24.5,
    // 10 splits 33.4)
    const uint32_t base = d->n_kv_heads * pl->n_mtiles;
    splits = std::max(1u, (uint32_t)cus / std::max(1u, base));
    splits = std::min(splits, std::max(1u, ntiles / 6u));
  }
  splits = std::min(std::min(splits, kMaxSplits), ntiles);
  pl->tiles_per_split = (ntiles + splits - 1) / splits;
  pl->n_splits = (ntiles + pl->tiles_per_split - 1) / pl->tiles_per_split;

  // workspace carve-up
  size_t off = 0;
  if (pl->convert_q) {
    pl->off_q = off;
    off += align_up((size_t)d->canvas * d->n_q_heads * hd * 2);
  }
  if (pl->gather_kv) {
    pl->off_kv = off;
    off += align_up((size_t)2 * d->n_kv_heads * pl->t_all * hd * 2);
  }
  // f16 partial rows need |V| <= 65504: an f16 cache guarantees it, for a bf16 cache the caller says so
  pl->part_half = pl->n_splits > 1 && d->out_dtype != DG_F32 && !(d->flags & DG_ATTN_F_F32_PARTIALS) &&
                  (pl->e_dtype == DG_F16 || (d->flags & DG_ATTN_F_F16_PARTIALS));
  if (pl->n_splits > 1) {
    pl->off_part_o = off;
    off += align_up((size_t)pl->n_splits * d->n_kv_heads * pl->rows_pad * hd * (pl->part_half ? 2 : 4));
    pl->off_part_ml = off;
    off += align_up((size_t)pl->n_splits * d->n_kv_heads * pl->rows_pad * 2 * 4);
  }
  pl->total = off;
  return DG_OK;
}

}  // namespace

extern "C" {

uint32_t dg_attn_abi_version(void) { return DG_ATTN_ABI_VERSION; }

const char* dg_attn_strerror(int status) {
  switch (status) {
    case DG_OK: return "ok";
    case DG_ERR_NULL: return "required pointer is null";
    case DG_ERR_SHAPE: return "unsupported canvas / head count / head_dim";
    case DG_ERR_DTYPE: return "unsupported dtype tag or dtype combination";
    case DG_ERR_LAYOUT: return "KV strides or offsets not usable (16-byte alignment, ring mask, range)";
    case DG_ERR_WORKSPACE: return "workspace missing or too small";
    case DG_ERR_MASK: return "inconsistent mask description";
    case DG_ERR_LAUNCH: return "HIP launch failed";
    case DG_ERR_DEVICE: return "no gfx950 device current";
    case DG_ERR_UNSUPPORTED: return "request not implemented";
    case DG_ERR_SCRATCH_LIMIT:
      return "the call needs more scratch than dg_attn_forward_static holds (dg_attn_static_scratch_bytes); "
             "use dg_attn_forward with a workspace";
    default: return "unknown status";
  }
}

void dg_attn_desc_reference_layout(dg_attn_desc* d) {
  const int64_t row = (int64_t)d->n_kv_heads * d->head_dim;
  d->k_tok_stride = 2 * row;
  d->k_head_stride = d->head_dim;
  d->v_base_off = row;
  d->v_tok_stride = 2 * row;
  d->v_head_stride = d->head_dim;
}

void dg_attn_desc_head_major_layout(dg_attn_desc* d, uint64_t t_cap) {
  d->k_tok_stride = d->head_dim;
  d->k_head_stride = (int64_t)t_cap * d->head_dim;
  d->v_base_off = (int64_t)d->n_kv_heads * (int64_t)t_cap * d->head_dim;
  d->v_tok_stride = d->head_dim;
  d->v_head_stride = (int64_t)t_cap * d->head_dim;
}

int dg_attn_workspace_bytes(const dg_attn_desc* d, size_t* out_bytes) {
  if (!d || !out_bytes) return DG_ERR_NULL;
  Plan pl;
  const int rc = make_plan(d, plan_cus(), &pl);
  if (rc != DG_OK) return rc;
  *out_bytes = pl.total;
  return DG_OK;
}

int dg_attn_resolved_splits(const dg_attn_desc* d, uint32_t* out_splits) {
  if (!d || !out_splits) return DG_ERR_NULL;
  Plan pl;
  const int rc = make_plan(d, plan_cus(), &pl);
  if (rc != DG_OK) return rc;
  *out_splits = pl.n_splits;
  return DG_OK;
}

int dg_attn_visible_pairs(const dg_attn_desc* d, uint64_t* pairs, double* flops) {
  if (!d) return DG_ERR_NULL;
  Plan pl;
  const int rc = make_plan(d, plan_cus(), &pl);
  if (rc != DG_OK) return rc;
  uint64_t n = 0;
  for (uint32_t tok = 0; tok < d->canvas; ++tok) {
    const bool causal = tok < d->causal_rows;
    const uint32_t qpos = d->kv_len + tok;
    uint32_t lo, hi, extra;
    if (causal) {
      hi = std::min(pl.t_all, qpos + 1u);
      lo = (d->window && qpos > d->window - 1u) ? qpos - (d->window - 1u) : 0u;
      extra = pl.extra_lo;
    } else {
      hi = pl.t_all;
      lo = pl.lo_nc;
      extra = pl.t_all;
    }
    if (hi > lo) n += hi - lo;
    const uint32_t e = std::max(extra, std::max(hi, lo));
    if (pl.t_all > e) n += pl.t_all - e;
  }
  if (pairs) *pairs = n;
  if (flops) *flops = 4.0 * d->head_dim * d->n_q_heads * (double)n;
  return DG_OK;
}

namespace {
// Fills the kernel parameter block from a validated descriptor; runs the f32 -> f16 conversion
// passes into the workspace when the plan asks for them.
int fill_params(const dg_attn_desc* d, const Plan& pl, const void* q, const void* kv_base, void* out, float* lse,
                char* ws, hipStream_t s, dg::AttnParams* pp) {
  const uint32_t hd = d->head_dim;
  const uint32_t esz_kv = elem_size(d->kv_dtype);
  dg::AttnParams& p = *pp;
  std::memset(&p, 0, sizeof(p));
  const char* region = (const char*)kv_base + d->kv_region_bytes;
  p.q = q;
  p.ring_mask = d->kv_ring_mask;
  p.t_clip_lo = pl.clip_lo;
  p.t_clip_hi = pl.clip_hi;
  if (pl.convert_q) {
    if (dg::launch_convert(q, d->q_dtype, ws + pl.off_q, DG_BF16, (size_t)d->canvas * d->n_q_heads * hd, s) != hipSuccess)
      return DG_ERR_LAUNCH;
    p.q = ws + pl.off_q;
  }
  if (pl.gather_kv) {
    char* kp = ws + pl.off_kv;
    char* vp = kp + (size_t)d->n_kv_heads * pl.t_all * hd * 2;
    if (dg::launch_kv_gather(region, d->kv_dtype, kp, pl.e_dtype, d->n_kv_heads, pl.t_all, hd, d->k_tok_stride,
                             d->k_head_stride, d->kv_ring_mask, s) != hipSuccess)
      return DG_ERR_LAUNCH;
    if (dg::launch_kv_gather(region + d->v_base_off * (int64_t)esz_kv, d->kv_dtype, vp, pl.e_dtype, d->n_kv_heads,
                             pl.t_all, hd, d->v_tok_stride, d->v_head_stride, d->kv_ring_mask, s) != hipSuccess)
      return DG_ERR_LAUNCH;
    p.k = kp;
    p.v = vp;
    p.k_tok_stride = p.v_tok_stride = hd;
    p.k_head_stride = p.v_head_stride = (int64_t)pl.t_all * hd;
    p.ring_mask = 0;
  } else {
    p.k = region;
    p.v = region + d->v_base_off * 2;
    p.k_tok_stride = d->k_tok_stride;
    p.k_head_stride = d->k_head_stride;
    p.v_tok_stride = d->v_tok_stride;
    p.v_head_stride = d->v_head_stride;
  }
  p.out = out;
  p.lse = lse;
  p.dbg = nullptr;
  p.canvas = d->canvas;
  p.hq = d->n_q_heads;
  p.hkv = d->n_kv_heads;
  p.group = pl.group;
  p.kv_len = d->kv_len;
  p.t_all = pl.t_all;
  p.causal_rows = d->causal_rows;
  p.win_m1 = pl.win_m1;
  p.lo_nc = pl.lo_nc;
  p.extra_lo = pl.extra_lo;
  p.rows_total = pl.rows_total;
  p.rows_pad = pl.rows_pad;
  p.n_mtiles = pl.n_mtiles;
  p.n_splits = pl.n_splits;
  p.tile_first = pl.tile_first;
  p.tiles_per_split = pl.tiles_per_split;
  p.tile_end = pl.tile_end;
  p.q_is_bf16 = pl.q_is_bf16 ? 1u : 0u;
  p.out_dtype = d->out_dtype;
  p.out_trunc = (d->flags & DG_ATTN_F_OUT_TRUNCATE) ? 1u : 0u;
  p.part_half = pl.part_half ? 1u : 0u;
  p.lo_explicit = (d->flags & DG_ATTN_F_T_LO_EXPLICIT) ? 1u : 0u;
  p.sees_masked = (d->flags & DG_ATTN_F_CAUSAL_SEES_MASKED) ? 1u : 0u;
  // key/value rows this call streams: more than the 256 MiB memory-side cache holds cannot have
  // stayed there from the previous call, whatever else runs in between (131072 keys: 0.933 -> 0.912 ms)
  const uint64_t kv_streamed = 2ull * d->n_kv_heads * (uint64_t)(pl.tile_end - pl.tile_first) * dg::kBlockN * d->head_dim * 2ull;
  // ... and a cache that other large caches were streamed after since its last use has been displaced
  // (cache_is_cold); DG_ATTN_F_KV_CACHED says the caller knows better
  const bool cold = cache_is_cold(region, kv_streamed) && hd == 512;   // (every call counts towards what was streamed)
  p.touch_ahead = ((d->flags & DG_ATTN_F_KV_FROM_HBM) || kv_streamed > (256ull << 20) ||
                   (cold && !(d->flags & DG_ATTN_F_KV_CACHED))) ? 1u : 0u;
  p.scale_log2 = pl.scale * dg::kLog2e;
  return DG_OK;
}

}  // namespace

namespace {
// One attention call with its plan made: validation of the pointers, parameter block, launches.
int forward_planned(const dg_attn_desc* d, const Plan& pl, const void* q, const void* kv_base, void* out, float* lse,
                    void* workspace, size_t workspace_bytes, void* stream, const uint32_t* step_dev = nullptr) {
  int rc = DG_OK;
  if (pl.total > 0 && (!workspace || workspace_bytes < pl.total)) return DG_ERR_WORKSPACE;
  if (pl.total > 0 && ((uintptr_t)workspace % 16) != 0) return DG_ERR_WORKSPACE;
  if (((uintptr_t)q % 16) != 0 || ((uintptr_t)kv_base % 16) != 0 || ((uintptr_t)out % 16) != 0) return DG_ERR_LAYOUT;
  hipStream_t s = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const uint32_t hd = d->head_dim;

  dg::AttnParams p;
  rc = fill_params(d, pl, q, kv_base, out, lse, ws, s, &p);
  if (rc != DG_OK) return rc;
  if (pl.n_splits > 1) {
    p.part_o = (float*)(ws + pl.off_part_o);
    p.part_ml = (float*)(ws + pl.off_part_ml);
  }
  p.dbg = g_tls_dbg;  // set only while dg_attention_dispatch is on the stack
  p.step_dev = step_dev;
  if (step_dev && (pl.scalar || pl.gather_kv)) return DG_ERR_UNSUPPORTED;   // (the f32 cache copy is made for a host-known length)

  if (pl.scalar) {
    if (dg::launch_attn_scalar(p, hd, pl.e_dtype, s) != hipSuccess) return DG_ERR_LAUNCH;
    return DG_OK;
  }
  const bool prof = g_prof.active && 2 * (size_t)g_prof.used + 1 < g_prof.ev.size();
  if (prof) (void)hipEventRecord(g_prof.ev[2 * g_prof.used], s);
  if ((pl.wsplit ? dg::launch_attn_wsplit(p, hd, pl.e_dtype, s) : dg::launch_attn_mfma(p, hd, pl.e_dtype, s)) != hipSuccess)
    return DG_ERR_LAUNCH;
  if (prof) {
    (void)hipEventRecord(g_prof.ev[2 * g_prof.used + 1], s);
    ++g_prof.used;
  }
  if (pl.n_splits > 1 && dg::launch_attn_merge(p, hd, (d->flags & DG_ATTN_F_STREAMED_MERGE) != 0, s) != hipSuccess) return DG_ERR_LAUNCH;
  return DG_OK;
}
}  // namespace

int dg_attn_forward(const dg_attn_desc* d, const void* q, const void* kv_base, void* out, float* lse,
                    void* workspace, size_t workspace_bytes, void* stream) {
  if (!d || !q || !kv_base || !out) return DG_ERR_NULL;
  DeviceInfo di;
  int rc = device_info(&di);
  if (rc != DG_OK) return rc;
  Plan pl;
  rc = make_plan(d, di.cus, &pl);
  if (rc != DG_OK) return rc;
  return forward_planned(d, pl, q, kv_base, out, lse, workspace, workspace_bytes, stream);
}

int dg_attn_forward_dev(const dg_attn_desc* d, const dg_step_params* step_dev, const void* q, const void* kv_base, void* out,
                        float* lse, void* workspace, size_t workspace_bytes, void* stream) {
  if (!d || !step_dev || !q || !kv_base || !out) return DG_ERR_NULL;
  if (((uintptr_t)step_dev % 4) != 0) return DG_ERR_LAYOUT;
  DeviceInfo di;
  int rc = device_info(&di);
  if (rc != DG_OK) return rc;
  Plan pl;
  rc = make_plan(d, di.cus, &pl);
  if (rc != DG_OK) return rc;
  return forward_planned(d, pl, q, kv_base, out, lse, workspace, workspace_bytes, stream, (const uint32_t*)step_dev);
}

size_t dg_attn_static_scratch_bytes(void) { return kStaticScratchBytes; }

int dg_attn_forward_static(const dg_attn_desc* d, const void* q, const void* kv_base, void* out, float* lse,
                           void* stream) {
  if (!d || !q || !kv_base || !out) return DG_ERR_NULL;
  DeviceInfo di;
  int rc = device_info(&di);
  if (rc != DG_OK) return rc;
  Plan pl;
  rc = make_plan(d, di.cus, &pl);
  if (rc != DG_OK) return rc;
  if (pl.total > kStaticScratchBytes) return DG_ERR_SCRATCH_LIMIT;
  void* ptr = nullptr;
  rc = static_scratch_ptr(&ptr);
  if (rc != DG_OK) return rc;
  // Nothing in the scratch has to start at zero: a launch writes every partial row and every
  // converted element it later reads.
  return forward_planned(d, pl, q, kv_base, out, lse, ptr, kStaticScratchBytes, stream);
}

// ---- key-range partials and their merge --------------------------------------------------------

namespace {
inline size_t state_bytes_of(const dg_attn_desc* d) {
  const size_t rows = (size_t)d->canvas * d->n_q_heads;
  return (dg::state_acc_offset(rows) + rows * d->head_dim) * sizeof(float);
}
// The descriptor of a partial: the caller's, with an fp32 result (the state's accumulators).
inline dg_attn_desc partial_desc(const dg_attn_desc* d) {
  dg_attn_desc pd = *d;
  pd.out_dtype = DG_F32;
  pd.flags &= ~(uint32_t)(DG_ATTN_F_OUT_TRUNCATE | DG_ATTN_F_F16_PARTIALS);
  return pd;
}
}  // namespace

int dg_attn_state_bytes(const dg_attn_desc* d, size_t* out_bytes) {
  if (!d || !out_bytes) return DG_ERR_NULL;
  Plan pl;
  const int rc = make_plan(d, plan_cus(), &pl);
  if (rc != DG_OK) return rc;
  *out_bytes = state_bytes_of(d);
  return DG_OK;
}

int dg_attn_partial_workspace_bytes(const dg_attn_desc* d, uint32_t t_begin, uint32_t t_end, size_t* out_bytes) {
  if (!d || !out_bytes) return DG_ERR_NULL;
  const dg_attn_desc pd = partial_desc(d);
  const uint32_t range[2] = {t_begin, t_end};
  Plan pl;
  const int rc = make_plan(&pd, plan_cus(), &pl, range);
  if (rc != DG_OK) return rc;
  *out_bytes = pl.total;
  return DG_OK;
}

int dg_attn_partial(const dg_attn_desc* d, uint32_t t_begin, uint32_t t_end, const void* q, const void* kv_base,
                    void* state, size_t state_bytes, void* workspace, size_t workspace_bytes, void* stream) {
  if (!d || !q || !kv_base || !state) return DG_ERR_NULL;
  DeviceInfo di;
  int rc = device_info(&di);
  if (rc != DG_OK) return rc;
  const dg_attn_desc pd = partial_desc(d);
  const uint32_t range[2] = {t_begin, t_end};
  Plan pl;
  rc = make_plan(&pd, di.cus, &pl, range);
  if (rc != DG_OK) return rc;
  if (state_bytes < state_bytes_of(d) || ((uintptr_t)state % 16) != 0) return DG_ERR_WORKSPACE;
  // The attention kernels leave the row normalised (acc / l) and its log-sum-exp: the state's normal
  // form is exactly that, (m, l) = (lse, 1), or (-inf, 0) for a row that saw no key of the range.
  const size_t rows = (size_t)d->canvas * d->n_q_heads;
  float* const m_plane = (float*)state;
  float* const acc = m_plane + dg::state_acc_offset(rows);
  rc = forward_planned(&pd, pl, q, kv_base, acc, m_plane, workspace, workspace_bytes, stream);
  if (rc != DG_OK) return rc;
  return dg::launch_state_unit_l(m_plane, m_plane + rows, (uint32_t)rows, (hipStream_t)stream) == hipSuccess
             ? DG_OK
             : DG_ERR_LAUNCH;
}

int dg_attn_merge(const dg_attn_desc* d, const void* const* states, uint32_t n_states, void* out, float* lse,
                  void* state_out, void* stream) {
  if (!d || !states) return DG_ERR_NULL;
  if (!out && !state_out) return DG_ERR_NULL;
  if (n_states == 0 || n_states > dg::kMaxStates) return DG_ERR_SHAPE;
  DeviceInfo di;
  int rc = device_info(&di);
  if (rc != DG_OK) return rc;
  Plan pl;
  rc = make_plan(d, di.cus, &pl);
  if (rc != DG_OK) return rc;
  dg::StateMergeParams p;
  std::memset(&p, 0, sizeof(p));
  for (uint32_t i = 0; i < n_states; ++i) {
    if (!states[i] || ((uintptr_t)states[i] % 16) != 0) return DG_ERR_NULL;
    p.states[i] = (const float*)states[i];
  }
  if ((out && ((uintptr_t)out % 16) != 0) || (state_out && ((uintptr_t)state_out % 16) != 0)) return DG_ERR_LAYOUT;
  p.n = n_states;
  p.rows = d->canvas * d->n_q_heads;
  p.hd = d->head_dim;
  p.hq = d->n_q_heads;
  p.out = out;
  p.lse = lse;
  p.state_out = (float*)state_out;
  p.out_dtype = d->out_dtype;
  p.out_trunc = (d->flags & DG_ATTN_F_OUT_TRUNCATE) ? 1u : 0u;
  p.dbg = g_tls_dbg;
  return dg::launch_state_merge(p, (hipStream_t)stream) == hipSuccess ? DG_OK : DG_ERR_LAUNCH;
}

namespace {
// Top-k sparse attention walks the canvas in row blocks so that the fp32 score plane of a block
// ([Hq][rows][t_pad]) stays within the memory-side cache between the kernel that writes it and
// the one that reads it.
#ifndef DG_TOPK_PLANE_MIB
#define DG_TOPK_PLANE_MIB 144
#endif
constexpr size_t kTopkPlaneBudget = (size_t)DG_TOPK_PLANE_MIB << 20;

struct TopkPlan {
  uint32_t t_pad = 0, block_tok = 0;
  size_t total = 0;
};

int make_topk_plan(const dg_attn_desc* d, const uint32_t* k_cfg, const Plan& pl, TopkPlan* tk) {
  if (!k_cfg) return DG_ERR_NULL;
  if (pl.scalar || d->q_dtype == DG_F32 || d->kv_dtype == DG_F32) return DG_ERR_UNSUPPORTED;
  if (k_cfg[1] == 0u) {
    if (k_cfg[0] > (uint32_t)dg::kTopkMaxK) return DG_ERR_SHAPE;
  } else if (k_cfg[3] > (uint32_t)dg::kTopkMaxK || k_cfg[2] > k_cfg[3]) {
    return DG_ERR_SHAPE;
  }
  tk->t_pad = (pl.t_all + dg::kBlockN - 1) / dg::kBlockN * dg::kBlockN;
  const size_t per_tok = (size_t)d->n_q_heads * tk->t_pad * sizeof(float);
  size_t blk = std::max<size_t>(1, kTopkPlaneBudget / per_tok);
  if (blk >= 16) blk &= ~(size_t)15;
  tk->block_tok = (uint32_t)std::min<size_t>(blk, d->canvas);
  tk->total = align_up((size_t)tk->block_tok * per_tok);
  if (tk->total / sizeof(float) >= (1ull << 32)) return DG_ERR_SHAPE;   // score rows are addressed with 32-bit offsets
  return DG_OK;
}
}  // namespace

int dg_attn_topk_workspace_bytes(const dg_attn_desc* d, const uint32_t* k_cfg, size_t* out_bytes) {
  if (!d || !out_bytes) return DG_ERR_NULL;
  Plan pl;
  int rc = make_plan(d, plan_cus(), &pl);
  if (rc != DG_OK) return rc;
  TopkPlan tk;
  rc = make_topk_plan(d, k_cfg, pl, &tk);
  if (rc != DG_OK) return rc;
  *out_bytes = tk.total;
  return DG_OK;
}

int dg_attn_topk_forward(const dg_attn_desc* d, const uint32_t* k_cfg, const void* q, const void* kv_base,
                         void* out, void* workspace, size_t workspace_bytes, void* stream) {
  if (!d || !q || !kv_base || !out) return DG_ERR_NULL;
  DeviceInfo di;
  int rc = device_info(&di);
  if (rc != DG_OK) return rc;
  Plan pl;
  rc = make_plan(d, plan_cus(), &pl);
  if (rc != DG_OK) return rc;
  TopkPlan tk;
  rc = make_topk_plan(d, k_cfg, pl, &tk);
  if (rc != DG_OK) return rc;
  if (!workspace || workspace_bytes < tk.total || ((uintptr_t)workspace % 16) != 0) return DG_ERR_WORKSPACE;
  if (((uintptr_t)q % 16) != 0 || ((uintptr_t)kv_base % 16) != 0 || ((uintptr_t)out % 16) != 0) return DG_ERR_LAYOUT;
  hipStream_t s = (hipStream_t)stream;

  dg::TopkParams tp;
  std::memset(&tp, 0, sizeof(tp));
  rc = fill_params(d, pl, q, kv_base, out, nullptr, nullptr, s, &tp.a);   // no conversion passes: dtypes checked above
  if (rc != DG_OK) return rc;
  tp.a.dbg = g_tls_dbg;
  tp.s_plane = (float*)workspace;
  tp.t_pad = tk.t_pad;
  tp.tile_first = pl.tile_first;
  tp.tile_end = pl.tile_end;
  for (int i = 0; i < 4; ++i) tp.k_cfg[i] = k_cfg[i];
  tp.scale = pl.scale;
  const uint32_t ntiles = std::max(1u, pl.tile_end - pl.tile_first);
  for (uint32_t tok0 = 0; tok0 < d->canvas; tok0 += tk.block_tok) {
    tp.tok0 = tok0;
    tp.ntok = std::min(tk.block_tok, d->canvas - tok0);
    tp.n_mtiles = (tp.ntok * pl.group + dg::kBlockM - 1) / dg::kBlockM;
    // enough workgroups for every CU, no split shorter than 8 key tiles; splits write disjoint
    // columns of the score plane, so there is nothing to merge
    const uint32_t base = d->n_kv_heads * tp.n_mtiles;
    uint32_t splits = std::max(1u, ((uint32_t)di.cus + base - 1u) / base);
    tp.n_splits = std::max(1u, std::min(splits, ntiles / 8u));
    // (timing aid: one event pair per kernel, scores first)
    const bool prof = g_prof.active && 2 * (size_t)g_prof.used + 3 < g_prof.ev.size();
    if (prof) (void)hipEventRecord(g_prof.ev[2 * g_prof.used], s);
    if (dg::launch_topk_scores(tp, d->head_dim, pl.e_dtype, s) != hipSuccess) return DG_ERR_LAUNCH;
    if (prof) {
      (void)hipEventRecord(g_prof.ev[2 * g_prof.used + 1], s);
      (void)hipEventRecord(g_prof.ev[2 * g_prof.used + 2], s);
    }
    if (dg::launch_topk_select(tp, d->head_dim, pl.e_dtype, s) != hipSuccess) return DG_ERR_LAUNCH;
    if (prof) {
      (void)hipEventRecord(g_prof.ev[2 * g_prof.used + 3], s);
      g_prof.used += 2;
    }
  }
  return DG_OK;
}

static void desc_from_reference(const dg_layer_offsets* L, const dg_attn_dims* dims, uint32_t kv_len,
                                dg_attn_desc* d) {
  std::memset(d, 0, sizeof(*d));
  d->canvas = dims->canvas;
  d->n_q_heads = dims->n_q_heads;
  d->n_kv_heads = L->n_kv_heads;
  d->head_dim = L->head_dim;
  d->kv_len = kv_len;
  d->causal_rows = dims->causal ? dims->canvas : 0u;
  d->window = dims->window;
  d->kv_ring_mask = L->kv_ring_mask;
  d->q_dtype = DG_BF16;
  d->kv_dtype = DG_F16;
  d->out_dtype = DG_BF16;
  d->flags = DG_ATTN_F_OUT_TRUNCATE;
  d->kv_region_bytes = L->kv_region;
  dg_attn_desc_reference_layout(d);
}

int dg_attention_state_bytes(const dg_layer_offsets* L, const dg_attn_dims* dims, uint32_t kv_len,
                             size_t* out_bytes) {
  if (!L || !dims || !out_bytes) return DG_ERR_NULL;
  dg_attn_desc d;
  desc_from_reference(L, dims, kv_len, &d);
  return dg_attn_workspace_bytes(&d, out_bytes);
}

int dg_attention_dispatch(const void* q, const void* kvcache, void* out, const dg_layer_offsets* L,
                          const dg_step_params* P, const dg_attn_dims* dims, dg_debug_status* dbg,
                          void* attn_state, size_t attn_state_bytes, void* stream) {
  if (!L || !P || !dims) return DG_ERR_NULL;
  dg_attn_desc d;
  desc_from_reference(L, dims, P->kv_len, &d);
  g_tls_dbg = (uint32_t*)dbg;
  const int rc = dg_attn_forward(&d, q, kvcache, out, nullptr, attn_state, attn_state_bytes, stream);
  g_tls_dbg = nullptr;
  return rc;
}

int dg_attention_dispatch_dev(const void* q, const void* kvcache, void* out, const dg_layer_offsets* L,
                              const dg_step_params* P_dev, uint32_t kv_len_max, const dg_attn_dims* dims,
                              dg_debug_status* dbg, void* attn_state, size_t attn_state_bytes, void* stream) {
  if (!L || !P_dev || !dims) return DG_ERR_NULL;
  dg_attn_desc d;
  desc_from_reference(L, dims, kv_len_max, &d);
  g_tls_dbg = (uint32_t*)dbg;
  const int rc = dg_attn_forward_dev(&d, P_dev, q, kvcache, out, nullptr, attn_state, attn_state_bytes, stream);
  g_tls_dbg = nullptr;
  return rc;
}

int dg_attention_block_state_bytes(const dg_layer_offsets* L, const dg_attn_dims* dims, uint32_t kv_len,
                                   size_t* out_bytes) {
  if (!L || !dims || !out_bytes) return DG_ERR_NULL;
  dg_attn_desc d;
  desc_from_reference(L, dims, kv_len, &d);
  size_t ws_full = 0;
  int rc = dg_attn_workspace_bytes(&d, &ws_full);
  if (rc != DG_OK) return rc;
  // The partial of a block [a, b) is split over workgroups like a whole call, and the number of splits a
  // range resolves to is not monotone in its length (ceil(n / ceil(n / s)) jumps up and down with n), so a
  // shorter range can take more splits than the whole one.  What bounds every range is the cap the split
  // count is cut to before that rounding; the partial workspace is sized for it, with fp32 partial rows
  // (a partial's result is fp32 accumulators).
  const dg_attn_desc pd = partial_desc(&d);
  Plan pl;
  const int cus = plan_cus();
  rc = make_plan(&pd, cus, &pl);
  if (rc != DG_OK) return rc;
  const uint32_t ntiles_full = std::max(1u, (pl.t_all + dg::kBlockN - 1) / dg::kBlockN);
  const uint32_t base = d.n_kv_heads * pl.n_mtiles;
  const uint32_t cap = std::min(std::min(std::max(1u, (uint32_t)cus / std::max(1u, base)), std::max(1u, ntiles_full / 6u)),
                                kMaxSplits);
  size_t ws_part = 0;
  if (cap > 1)
    ws_part = align_up((size_t)cap * d.n_kv_heads * pl.rows_pad * d.head_dim * 4) +
              align_up((size_t)cap * d.n_kv_heads * pl.rows_pad * 2 * 4);
  *out_bytes = 2 * align_up(state_bytes_of(&d)) + std::max(ws_full, ws_part);
  return DG_OK;
}

int dg_attention_dispatch_block(const void* q, const void* kvcache, void* out, const dg_layer_offsets* L,
                                const dg_step_params* P, const dg_attn_dims* dims, const dg_attn_block_range* blk,
                                dg_debug_status* dbg, void* attn_state, size_t attn_state_bytes, void* stream) {
  if (!L || !P || !dims || !blk) return DG_ERR_NULL;
  if (blk->is_first && blk->is_last)
    return dg_attention_dispatch(q, kvcache, out, L, P, dims, dbg, attn_state, attn_state_bytes, stream);
  if (!attn_state || ((uintptr_t)attn_state % 16) != 0) return DG_ERR_WORKSPACE;
  dg_attn_desc d;
  desc_from_reference(L, dims, P->kv_len, &d);
  const size_t sb = align_up(state_bytes_of(&d));
  if (attn_state_bytes < 2 * sb) return DG_ERR_WORKSPACE;
  char* const carried = (char*)attn_state;        // (m, l, acc) of the blocks so far
  char* const fresh = carried + sb;               // this block's own partial
  char* const ws = carried + 2 * sb;
  const size_t ws_bytes = attn_state_bytes - 2 * sb;
  // A block with no key for some rows (a causal row's range ends before it) leaves l = 0 there, and
  // the merge passes the carried state through, which is what the reference's early return does.
  int rc = dg_attn_partial(&d, blk->t_begin, blk->t_end, q, kvcache, blk->is_first ? carried : fresh, sb, ws, ws_bytes,
                           stream);
  if (rc != DG_OK || blk->is_first) return rc;
  const void* both[2] = {carried, fresh};
  if (!blk->is_last) return dg_attn_merge(&d, both, 2u, nullptr, nullptr, carried, stream);
  if (!out) return DG_ERR_NULL;
  g_tls_dbg = (uint32_t*)dbg;
  rc = dg_attn_merge(&d, both, 2u, out, nullptr, nullptr, stream);
  g_tls_dbg = nullptr;
  return rc;
}

int dg_attention_topk_state_bytes(const dg_layer_offsets* L, const dg_attn_dims* dims, uint32_t kv_len,
                                  const uint32_t* k_cfg, size_t* out_bytes) {
  if (!L || !dims || !out_bytes) return DG_ERR_NULL;
  dg_attn_desc d;
  desc_from_reference(L, dims, kv_len, &d);
  return dg_attn_topk_workspace_bytes(&d, k_cfg, out_bytes);
}

int dg_attention_topk_dispatch(const void* q, const void* kvcache, void* out, const dg_layer_offsets* L,
                               const dg_step_params* P, const dg_attn_dims* dims, const uint32_t* k_cfg,
                               dg_debug_status* dbg, void* scratch, size_t scratch_bytes, void* stream) {
  if (!L || !P || !dims) return DG_ERR_NULL;
  dg_attn_desc d;
  desc_from_reference(L, dims, P->kv_len, &d);
  g_tls_dbg = (uint32_t*)dbg;
  const int rc = dg_attn_topk_forward(&d, k_cfg, q, kvcache, out, scratch, scratch_bytes, stream);
  g_tls_dbg = nullptr;
  return rc;
}

int dg_prof_begin(uint32_t max_launches) {
  if (g_prof.active) return DG_ERR_UNSUPPORTED;
  g_prof.ev.assign(2 * (size_t)max_launches, nullptr);
  for (auto& e : g_prof.ev)
    if (hipEventCreate(&e) != hipSuccess) return DG_ERR_LAUNCH;
  g_prof.used = 0;
  g_prof.active = true;
  return DG_OK;
}

int dg_prof_end_split(double* even_ms_total, double* odd_ms_total, uint32_t* n_pairs) {
  if (!g_prof.active) return DG_ERR_UNSUPPORTED;
  double total[2] = {0.0, 0.0};
  int rc = DG_OK;
  if (g_prof.used > 0 && hipEventSynchronize(g_prof.ev[2 * g_prof.used - 1]) != hipSuccess) rc = DG_ERR_LAUNCH;
  for (uint32_t i = 0; i < g_prof.used && rc == DG_OK; ++i) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, g_prof.ev[2 * i], g_prof.ev[2 * i + 1]) != hipSuccess) rc = DG_ERR_LAUNCH;
    total[i & 1u] += ms;
  }
  for (auto e : g_prof.ev)
    if (e) (void)hipEventDestroy(e);
  if (even_ms_total) *even_ms_total = total[0];
  if (odd_ms_total) *odd_ms_total = total[1];
  if (n_pairs) *n_pairs = g_prof.used;
  g_prof.ev.clear();
  g_prof.used = 0;
  g_prof.active = false;
  return rc;
}

int dg_prof_end(double* main_kernel_ms_total, uint32_t* n_launches) {
  double even = 0.0, odd = 0.0;
  const int rc = dg_prof_end_split(&even, &odd, n_launches);
  if (main_kernel_ms_total) *main_kernel_ms_total = even + odd;
  return rc;
}

int dg_calib_copy(void* dst, const void* src, size_t bytes, void* stream) {
  if (!dst || !src) return DG_ERR_NULL;
  if (bytes % 16 != 0 || ((uintptr_t)dst % 16) != 0 || ((uintptr_t)src % 16) != 0) return DG_ERR_LAYOUT;
  return dg::launch_calib_copy(dst, src, bytes, (hipStream_t)stream) == hipSuccess ? DG_OK : DG_ERR_LAUNCH;
}

int dg_calib_mfma(float* sink, size_t sink_bytes, uint32_t workgroups, uint32_t iters, uint32_t random_operands,
                  uint64_t* flops, void* stream) {
  if (!sink || !flops) return DG_ERR_NULL;
  if (random_operands > 3u) return DG_ERR_UNSUPPORTED;
  if (workgroups == 0 || iters == 0 || sink_bytes < (size_t)workgroups * 256 * sizeof(float)) return DG_ERR_WORKSPACE;
  // per workgroup: 4 waves x iters x 16 MFMAs x (32 x 32 x 16 multiply-adds)
  *flops = (uint64_t)workgroups * 4ull * iters * 16ull * (2ull * 32 * 32 * 16);
  return dg::launch_calib_mfma(sink, workgroups, iters, random_operands, (hipStream_t)stream) == hipSuccess
             ? DG_OK
             : DG_ERR_LAUNCH;
}

uint64_t dg_kv_row_bytes(uint32_t head_dim, uint32_t kv_dtype) { return (uint64_t)head_dim * elem_size(kv_dtype); }

uint64_t dg_kv_region_bytes(uint32_t n_kv_heads, uint32_t head_dim, uint64_t slots, uint32_t kv_dtype) {
  return slots * (uint64_t)n_kv_heads * 2ull * dg_kv_row_bytes(head_dim, kv_dtype);
}

uint64_t dg_kv_slot(uint32_t kv_ring_mask, uint64_t pos) { return kv_ring_mask ? (pos & kv_ring_mask) : pos; }

uint64_t dg_layer_kv_slots(int is_full, uint64_t max_seq, uint64_t ring_slots_cap) {
  if (is_full) return (max_seq + 8 + 7) / 8 * 8;
  uint64_t p2 = 1;
  while (p2 < max_seq) p2 <<= 1;
  return ring_slots_cap ? std::min(p2, ring_slots_cap) : p2;
}

}  // extern "C"
