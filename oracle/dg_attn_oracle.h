/* CPU oracle for diffgemma's denoise-step attention.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a restatement, on the CPU, of the algorithm the reference's own CPU
 * twins implement.  Only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg may load it; nothing in the shipped library links it.
 *
 * Reference files each function follows (paths relative to the reference root):
 *   dgo_attention_f32        src/shaders/attn/cpu.rs:148-197 (recurrence, indexing, no scale)
 *                            src/shaders/attn/attention/attention.metal:49-63 (causal, window)
 *                            src/shaders/attn/attention/attention_mma2.metal:199-211,297 (row mask, guards)
 *                            src/shaders/include/attention_device.metal:27-33 (ring slot map)
 *                            src/shaders/attn/attention_gemm/mod.rs:306-359 (causal rows)
 *   dgo_attention_blocked_f32 src/shaders/attn/attention_flash/mod.rs:20-94 (blocked online softmax)
 *   dgo_attention_bitmap_f32 src/model/attention.rs:354-394,861-934 + src/model/mask.rs:4-27
 *                            + src/shaders/cpu/mod.rs:175-190 (dense scores, MASK_NEG, softmax_rows)
 *   dgo_attention_f64        textbook two-pass softmax(QK^T)V in double (closed form, no reference twin)
 *   dgo_attention_topk_f32   src/shaders/attn/attention_topk/cpu.rs:41-120 (exact top-k by f32 score, ties to the
 *                            lower index, softmax over the kept keys, V summed in selection order);
 *   dgo_topk_row_k           src/shaders/attn/attention_topk/attention_topk.metal:160-182 (fixed or
 *                            context-adaptive k per row), src/flags/accessors.rs:210-221 (k_cfg)
 *   dgo_fnv1a64              src/metal/step_kernel/runtime.rs:127-133 (FNV-1a, 64 bit); the snapshot gather /
 *                            scatter and the live-KV byte walk (src/metal/step_kv/mod.rs:108-151,
 *                            runtime.rs:118-148) are restated in numpy in pyoracle.py (kv_gather_prefix,
 *                            kv_scatter_prefix, kv_live_stream)
 *   dgo_merge_partials_f32   closed form m=max m_i, l=sum l_i e^(m_i-m), O=sum O_i e^(m_i-m)/l; the
 *                            reference's state planes: attention_mma_full.metal:107-118,355-368
 *   rounding helpers         src/shaders/common/bf16.rs:9-41, src/shaders/common/f16.rs:3-60
 *   dgo_rms_norm_no_scale    src/shaders/cpu/mod.rs:24-35 ; dgo_rms_norm_head src/shaders/attn/cpu.rs:67-75
 *   dgo_rope_split_half      src/shaders/attn/cpu.rs:31-45 ; dgo_rope_proportional cpu.rs:48-65
 *   dgo_qk_rope_kv_f32       src/shaders/attn/cpu.rs:78-145 (per-head RMSNorm + RoPE + cache write, V aliasing)
 *                            src/shaders/attn/qk_rope_kv/qk_rope_kv.metal:56-60 (kv_write_end suppression),
 *                            :87,:114 + src/shaders/include/attention_device.metal:28-33 (ring slot of the write)
 *   dgo_fixture_rope_*       src/shaders/attn/qk_rope_kv/mod.rs:80-189
 *   fixture generators       src/shaders/attn/attention/mod.rs:59-184,689-691,
 *                            src/shaders/attn/attention_gemm/mod.rs:364-432,
 *                            src/metal/step_kernel/runtime.rs:183-206 (synthetic_fill_kv)
 *
 * Pinning (what each function is checked against in tests/test_oracle_*.py):
 *   - recurrence == float64 two-pass closed form; brute force on the reference's tiny fixtures
 *   - window / ring / causal / mixed-mask rows == all-valid result on the visible key sub-range
 *   - bitmap path == predicate path for every mask the predicate can express
 *   - blocked(bk) == unblocked for bk in {1,3,8,16,64,4096} (reference's own test, 1e-3)
 *   - special cases: all keys equal -> mean(V), LSE = s + ln n; one dominant key -> that V row
 *   - rounding known answers (bf16.rs:47-55 value 1.234567; f16 clamp / flush-subnormal cases)
 *   - producer (qk_rope_kv): unit RMS of every normed head; pair norms preserved by the rotation;
 *     position 0 is the identity; R(a)R(b) = R(a+b) via the angle closed form theta^(-2d/hd);
 *     one-hot inputs show which elements are paired (split-half vs proportional) and which are
 *     left alone (proportional: only hd/4 of the head rotates); cache rows land at the slot the
 *     attention oracle reads; V = rms_norm_no_scale(raw k) when V aliases k
 *   - top-k: k >= visible keys == the dense oracle; k = 1 == the V row of the arg-max key; numpy
 *     brute force (lexsort by (-score, index), float64 softmax over the kept set) on random small
 *     cases incl. duplicated keys (tie-break) and ragged causal rows (k > visible keys); the
 *     per-row k rule against hand-computed values
 *   - FNV-1a: the published test vectors ("" -> offset basis, "a", "foobar"); the snapshot
 *     restatements: a hand-laid-out two-layer cache, scatter(gather(x)) == x on the live part
 * LSE is not emitted anywhere in the reference; it is the closed form m + ln(l) of the
 * recurrence's own (m, l), cross-checked against a float64 logsumexp of the score row.
 */
#ifndef DG_ATTN_ORACLE_H
#define DG_ATTN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dgo_desc {
  uint32_t canvas;        /* query rows (AttnDims.canvas) */
  uint32_t n_q_heads;     /* AttnDims.n_q_heads */
  uint32_t n_kv_heads;    /* LayerOffsets.n_kv_heads */
  uint32_t head_dim;      /* LayerOffsets.head_dim */
  uint32_t kv_len;        /* StepParams.kv_len: committed prefix length */
  uint32_t causal_rows;   /* rows [0,causal_rows) use the reference's causal=1 rule, the rest causal=0 */
  uint32_t window;        /* 0 = unwindowed */
  uint32_t kv_ring_mask;  /* 0 = linear, else slot = pos & mask */
  uint32_t causal_sees_masked; /* 1: causal rows additionally see canvas keys >= kv_len+causal_rows */
  uint32_t strict_order;  /* 1: sequential fp32 sums exactly in the reference's order (slow) */
  int64_t  t_lo_override; /* >=0: first visible key for non-causal rows instead of the window rule */
  int64_t  k_off, k_tok_stride, k_head_stride;  /* element offsets into kv[] */
  int64_t  v_off, v_tok_stride, v_head_stride;
  float    scale;         /* multiplies every score; the reference uses 1.0 */
} dgo_desc;

/* fills the strides for the reference's slot-major layout [slot][K: Hkv*d | V: Hkv*d] (cpu.rs:173,184) */
void dgo_desc_reference_layout(dgo_desc* d);
/* fills the strides for two planes [Hkv][t_cap][d], K plane first then V plane */
void dgo_desc_head_major_layout(dgo_desc* d, int64_t t_cap);

/* 1 if query row tok may attend absolute key position t */
int dgo_visible(const dgo_desc* d, uint32_t tok, uint32_t t);
/* number of visible (tok,key) pairs for one head */
uint64_t dgo_visible_pairs(const dgo_desc* d);

/* Online-softmax recurrence in fp32.  q/out: [canvas][n_q_heads][head_dim]; lse: [canvas][n_q_heads]
 * (may be NULL).  Only rows tok_list[0..n_tok) are computed when tok_list != NULL.  n_threads<=0: all. */
void dgo_attention_f32(const dgo_desc* d, const float* q, const float* kv, float* out, float* lse,
                       const uint32_t* tok_list, uint32_t n_tok, int n_threads);
/* Top-k sparse attention (attention_topk/cpu.rs:41-120): per (row, head) only the k highest scores among the
 * visible keys are kept (ties: lower index first), softmax is renormalised over them and the V rows are summed
 * in that order.  k_cfg = (fixed_k | chunk grid, dyn_divisor, k_min, k_max) as in attention_topk.metal:160-182:
 * divisor 0 -> k = k_cfg[0]; else k = clamp(t_equiv / divisor, k_min, k_max) with t_equiv the row's visible-key
 * count, rounded up to the grid for causal rows.  sel_idx [canvas][Hq][sel_cap] / sel_count [canvas][Hq] (may
 * be NULL) receive the selected key positions in selection order. */
uint32_t dgo_topk_row_k(const uint32_t k_cfg[4], uint32_t n_valid, int causal_row);
void dgo_attention_topk_f32(const dgo_desc* d, const uint32_t k_cfg[4], const float* q, const float* kv, float* out,
                            uint32_t* sel_idx, uint32_t sel_cap, uint32_t* sel_count, const uint32_t* tok_list,
                            uint32_t n_tok, int n_threads);
/* FNV-1a over bytes, continuing seed_hash (src/metal/step_kernel/runtime.rs:127-133). */
uint64_t dgo_fnv1a64(const uint8_t* bytes, size_t n, uint64_t seed_hash);
/* Same mask semantics, two-pass softmax in double. */
void dgo_attention_f64(const dgo_desc* d, const float* q, const float* kv, double* out, double* lse,
                       const uint32_t* tok_list, uint32_t n_tok, int n_threads);
/* Blocked online softmax with key blocks of bk. */
void dgo_attention_blocked_f32(const dgo_desc* d, const float* q, const float* kv, float* out, float* lse,
                               uint32_t bk, int n_threads);
/* Key-range partial: visits only keys in [t_begin,t_end); returns unnormalised acc plus (m,l) per row.
 * acc: [canvas][n_q_heads][head_dim], m,l: [canvas][n_q_heads]. */
void dgo_attention_partial_f32(const dgo_desc* d, const float* q, const float* kv, uint32_t t_begin,
                               uint32_t t_end, float* acc, float* m, float* l, int n_threads);
/* Merge n_parts partials (arrays of pointers) into out/lse. */
void dgo_merge_partials_f32(uint32_t rows, uint32_t head_dim, uint32_t n_parts, const float* const* acc,
                            const float* const* m, const float* const* l, float* out, float* lse);
/* General boolean-mask attention: k,v [total_kv][n_kv_heads][head_dim], mask [seq][total_kv] bytes. */
void dgo_attention_bitmap_f32(uint32_t seq_len, uint32_t total_kv, uint32_t n_heads, uint32_t n_kv_heads,
                              uint32_t head_dim, const float* q, const float* k, const float* v,
                              const uint8_t* mask, float* out);

/* rounding (bits <-> f32) */
uint16_t dgo_f32_to_bf16_trunc(float v);
uint16_t dgo_f32_to_bf16_rne(float v);
float    dgo_bf16_to_f32(uint16_t b);
uint16_t dgo_f32_to_f16_trunc(float v);   /* reference host conversion: clamp, flush subnormals, truncate */
uint16_t dgo_f32_to_f16_rne(float v);     /* IEEE round-to-nearest-even incl. subnormals */
float    dgo_f16_to_f32(uint16_t b);
/* mode: 0 bf16 trunc, 1 bf16 rne, 2 f16 trunc (reference), 3 f16 rne.  In-place value rounding. */
void dgo_round_array(float* x, size_t n, int mode);
void dgo_to_bits(const float* x, uint16_t* bits, size_t n, int mode);
void dgo_from_bits(const uint16_t* bits, float* x, size_t n, int is_f16);

void dgo_rms_norm_no_scale(float* out, const float* x, size_t n, float eps);
void dgo_rms_norm_head(float* x, const float* weight /*may be NULL*/, size_t n, float eps);

/* ---- the producer of the cache rows attention reads: per-head RMSNorm + RoPE + KV write ---- */
typedef struct dgo_rope_desc {
  uint32_t canvas, n_q_heads, n_kv_heads, head_dim;
  uint32_t kv_len;        /* canvas row tok sits at position kv_len + tok */
  uint32_t kv_write_end;  /* positions >= this are normed/rotated but never written to the cache */
  uint32_t kv_ring_mask;  /* 0 = linear, else the row goes to slot pos & mask; RoPE uses the absolute pos */
  uint32_t is_full;       /* 1: proportional RoPE, theta 1e6, rot = hd/4; 0: split-half, theta 1e4, rot = hd */
  uint32_t v_from_k;      /* 1 (reference v_proj == 0): V is the RAW k projection, normed without weight */
  int64_t  k_off, k_tok_stride, k_head_stride;  /* element offsets into kvcache[] */
  int64_t  v_off, v_tok_stride, v_head_stride;
} dgo_rope_desc;
void dgo_rope_split_half(float* x, uint32_t rot, uint32_t head_dim, float theta, uint32_t pos);
void dgo_rope_proportional(float* x, uint32_t rotary_dim, uint32_t head_dim, float theta, uint32_t pos);
/* q [canvas][Hq][hd] and k [canvas][Hkv][hd] are updated in place (k only when V does not alias it);
 * v [canvas][Hkv][hd] is read when v_from_k == 0.  No storage rounding happens here. */
void dgo_qk_rope_kv_f32(const dgo_rope_desc* d, float* q, float* k, const float* v, float* kvcache,
                        const float* q_norm_w, const float* k_norm_w);
/* the reference's producer fixtures (qk_rope_kv/mod.rs:80-189): which = 0 tiny, 1 full_layer,
 * 2 full_hd512_v_alias; buffers sized by the caller from the fixture's dims */
void dgo_fixture_rope(int which, float* q, float* k, float* v, float* q_norm_w, float* k_norm_w);

/* reference fixture generators; kv in the reference slot-major layout, sizes as the reference computes them */
void dgo_fixture_tiny(float* q /*2*4*32*/, float* kv /*4*2*32*2*/);
void dgo_fixture_wide(float* q /*4*8*64*/, float* kv /*8*2*64*2*/);
void dgo_fixture_model_attn(uint32_t canvas, uint32_t n_q_heads, uint32_t n_kv, uint32_t hd, uint32_t kv_len,
                            float* q, float* kv);
void dgo_fixture_model_full(uint32_t canvas, uint32_t n_q_heads, uint32_t n_kv, uint32_t hd, uint32_t kv_len,
                            float* q, float* kv);
/* xorshift64* filler writing f16 bit patterns in +-[0.125,0.25) */
void dgo_synthetic_fill_kv(uint16_t* bits, size_t n, uint64_t seed);

int dgo_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
