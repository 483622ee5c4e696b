/* C-ABI of the MI355X (gfx950) denoise-step attention library, libdg_attn_hip.so.
 *
 * Every entry point takes plain pointers and sizes: device pointers are caller-owned HIP
 * allocations, `stream` is a hipStream_t passed as void* (NULL = the default stream).
 * Calls enqueue work in order on that stream, never synchronise the host, never allocate,
 * and never unwind across the boundary; 0 means success, a negative value is a dg_status
 * (dg_attn_strerror gives the text).  One thread drives one stream, as in the reference
 * ("one thread owns the GPU + KV", reference ARCHITECTURE.md:553).
 *
 * Reference interfaces replaced (paths relative to the reference root):
 *   dg_attention_dispatch    StepEnc::encode_layer_attention_dispatch,
 *                            src/metal/step_kernel/enc.rs:2102-2296 (buffers 0..8 it binds)
 *   dg_attn_forward          the kernels behind it: attention, attention_mma2, attention_mma_full
 *                            (src/shaders/attn/attention/ *.metal files) and their harnesses
 *                            attention::gpu / gpu_mma2 / gpu_mma_full (attention/mod.rs:377-686)
 *   dg_layer_offsets         LayerOffsets, src/metal/step_kernel/mod.rs:132-167
 *   dg_step_params           StepParams,   src/metal/step_kernel/mod.rs:189-213
 *   dg_attn_dims             AttnDims,     src/shaders/attn/qk_rope_kv/mod.rs:15-38
 *   dg_attn_block_range      AttnBlockRange, src/shaders/include/attention_device.metal:160-165
 *   dg_debug_status          DebugStatus,  src/metal/debug_status.rs:11-43
 *   dg_kv_*                  kv_row_bytes / kv_region_bytes / kv_slot / layer_kv_slots,
 *                            src/metal/step_kv/mod.rs:65-100, src/metal/step_kernel/mod.rs:511-527
 */
#ifndef DG_ATTN_H
#define DG_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DG_ATTN_ABI_VERSION 1u

typedef enum dg_status {
  DG_OK = 0,
  DG_ERR_NULL = -1,        /* a required pointer is NULL */
  DG_ERR_SHAPE = -2,       /* canvas/head counts/head_dim not supported */
  DG_ERR_DTYPE = -3,       /* dtype tag or dtype combination not supported */
  DG_ERR_LAYOUT = -4,      /* strides / offsets not 16-byte aligned, ring mask not 2^k-1, ... */
  DG_ERR_WORKSPACE = -5,   /* workspace missing or too small */
  DG_ERR_MASK = -6,        /* causal_rows > canvas, window/t_lo inconsistent */
  DG_ERR_LAUNCH = -7,      /* the HIP runtime refused a launch (sticky error text kept) */
  DG_ERR_DEVICE = -8,      /* not a gfx950 device, or no device */
  DG_ERR_UNSUPPORTED = -9, /* valid request the library does not implement (e.g. q8 KV) */
  DG_ERR_SCRATCH_LIMIT = -10 /* dg_attn_forward_static: the call needs more scratch than the library holds */
} dg_status;

struct dg_step_params;   /* below */

typedef enum dg_dtype { DG_BF16 = 0, DG_F16 = 1, DG_F32 = 2 } dg_dtype;

typedef enum dg_kernel_sel {
  DG_KERNEL_AUTO = 0,   /* MFMA kernel, split count chosen by the library */
  DG_KERNEL_SCALAR = 1, /* one wave per (row, head): the slow on-GPU cross-check, like the
                           reference's scalar `attention` kernel next to its MMA kernels */
  DG_KERNEL_MFMA = 2
} dg_kernel_sel;

/* desc.flags */
#define DG_ATTN_F_OUT_TRUNCATE 0x1u        /* bf16/f16 store by truncation (reference arena_store,
                                              src/shaders/include/common.metal:16-18); default RNE */
#define DG_ATTN_F_CAUSAL_SEES_MASKED 0x2u  /* causal rows also see canvas keys >= kv_len+causal_rows */
#define DG_ATTN_F_T_LO_EXPLICIT 0x4u       /* non-causal rows start at desc.t_lo instead of the
                                              window rule kv_len-(window-1) */
#define DG_ATTN_F_F32_PARTIALS 0x8u        /* keep split partial rows in fp32 (always the case with an
                                              f32 output) */
#define DG_ATTN_F_F16_PARTIALS 0x10u       /* bf16 cache, 16-bit output: let split partial rows travel
                                              between the attention and the merge kernel as f16 after
                                              division by the split's row sum (a weighted mean of V
                                              rows).  The caller asserts |V| <= 65504 and accepts that
                                              partial-row values below 2^-14 lose precision; true of
                                              every cache the producer below writes (V rows are
                                              RMS-normalised, |v| <= sqrt(head_dim)).  Values beyond
                                              the range saturate.  This is the default for an f16
                                              cache, which guarantees the range; the rounding is 1/8 of
                                              a bf16 output's. */
#define DG_ATTN_F_KV_FROM_HBM 0x40u        /* hint: the cache rows this call reads will not be in the
                                              memory-side cache (256 MB on MI355X) when it runs, as in a loop
                                              over many layers whose caches add up to more than that.  The
                                              head_dim 512 kernel then touches key/value tiles into the L2
                                              six tiles before it loads them: 5 % faster when the rows do come
                                              from HBM, 2 % slower when they were cached after all.  Results
                                              are the same bits either way.  A call that streams more than
                                              256 MiB of keys and values does this without being told. */
#define DG_ATTN_F_KV_CACHED 0x100u         /* hint, the opposite: the rows WILL be in the memory-side cache.  Without either
                                              hint the library guesses from what the calling thread's recent calls
                                              streamed: a cache is taken to be displaced when other caches of more than
                                              200 MiB in total were read since its last use (a loop over a model's
                                              layers), or on its first use when it is 32 MiB or more. */
#define DG_ATTN_F_STREAMED_MERGE 0x20u     /* merge the split partial rows with the streaming kernel (weights
                                              first, then only the rows of splits that count) even where the
                                              library would pick the one that fetches every partial row up
                                              front (at most 8 splits, f16 partial rows, workspace below
                                              32 MiB).  Both give the same bits; the flag is there to compare them. */

#define DG_ATTN_F_SPLIT_OVER_WORKGROUPS 0x80u /* head_dim <= 256 and a short key range (a sliding-window layer): the
                                              library runs one launch in which the waves of a workgroup split the
                                              keys and merge in LDS.  This flag asks for the general kernel instead
                                              (keys split over workgroups, partial rows in the workspace, a merge
                                              launch), as does an explicit n_splits.  Results agree to the rounding
                                              of the probabilities; the flag is there to compare the two. */

typedef struct dg_attn_desc {
  uint32_t canvas;        /* query rows; the reference passes active_canvas (256/128/64) */
  uint32_t n_q_heads;
  uint32_t n_kv_heads;
  uint32_t head_dim;      /* 32, 64, 128, 256 or 512 */
  uint32_t kv_len;        /* committed prefix length; canvas keys live at [kv_len, kv_len+canvas) */
  uint32_t causal_rows;   /* 0 = denoise (reference causal=0); canvas = reference causal=1;
                             in between = rows below it causal, rows from it on bidirectional */
  uint32_t window;        /* 0 = global layer; else reference rule: non-causal rows see keys
                             >= kv_len-(window-1), causal row at qpos sees >= qpos-(window-1) */
  uint32_t kv_ring_mask;  /* 0 = linear; else slot = pos & mask (mask+1 a power of two) */
  uint32_t q_dtype;       /* dg_dtype: DG_BF16 or DG_F32 */
  uint32_t kv_dtype;      /* dg_dtype: DG_BF16, DG_F16 or DG_F32 */
  uint32_t out_dtype;     /* dg_dtype: DG_BF16 or DG_F32 */
  uint32_t flags;
  uint32_t t_lo;          /* used with DG_ATTN_F_T_LO_EXPLICIT */
  uint32_t n_splits;      /* key-range splits; 0 = library chooses */
  uint32_t kernel;        /* dg_kernel_sel */
  float    softmax_scale; /* multiplies q.k; 0 means 1.0 (the reference applies no scale) */
  uint64_t kv_region_bytes; /* byte offset of this layer's region inside kv_base */
  /* element strides/offsets inside the region (elements of kv_dtype), head_dim contiguous */
  int64_t  k_tok_stride, k_head_stride;
  int64_t  v_base_off, v_tok_stride, v_head_stride;
} dg_attn_desc;

/* Strides of the reference's slot-major cache [slot][K: Hkv*d | V: Hkv*d]
 * (src/metal/step_kv/mod.rs:8-22). */
void dg_attn_desc_reference_layout(dg_attn_desc* d);
/* Strides of two planes [Hkv][t_cap][d] (K plane, then V plane at Hkv*t_cap*d). */
void dg_attn_desc_head_major_layout(dg_attn_desc* d, uint64_t t_cap);

/* Bytes of device scratch dg_attn_forward needs for this descriptor (0 is possible). */
int dg_attn_workspace_bytes(const dg_attn_desc* d, size_t* out_bytes);

/* Splits the library would use for this descriptor (n_splits==0 resolved). */
int dg_attn_resolved_splits(const dg_attn_desc* d, uint32_t* out_splits);

/* q, out: [canvas][n_q_heads][head_dim]; lse: [canvas][n_q_heads] fp32 natural-log
 * log-sum-exp of the scaled scores (NULL to skip; a row with no visible key gets -inf and
 * an all-zero output row).  Accuracy of lse: the row sum is taken over the probabilities as
 * rounded to the MFMA operand type (the numbers P.V multiplies, so that out is an exact
 * weighted mean): bf16 keeps 8 significant bits, so each is within 2^-8 of its value (2^-11 with an f16
 * cache), and on a row with one dominant key nothing averages out: ln(sum) moves by at most 2^-8 = 3.9e-3
 * absolute: |lse - exact| <= max(1e-3 |exact|, 2^-8). */
int dg_attn_forward(const dg_attn_desc* d, const void* q, const void* kv_base, void* out, float* lse,
                    void* workspace, size_t workspace_bytes, void* stream);

/* dg_attn_forward with the prefix length read on the device when the kernels run, the way the reference binds
 * StepParams as a device buffer (src/metal/step_kernel/enc.rs:2177-2220, buffer 4: its kernels read kv_len at
 * execution time, so one encoded step serves every committed prefix).  step_dev is a DEVICE dg_step_params (only
 * kv_len is read); d->kv_len is the largest prefix the call has to cover: grid, split count and workspace are planned
 * for it (dg_attn_workspace_bytes with the same descriptor), and a device value above it is clamped to it.  A HIP
 * graph recorded with this entry stays valid while the caller advances kv_len in device memory after every committed
 * block (src/metal/step_generate/turn.rs:575-660) instead of recording again.  For every device value the result is
 * that of dg_attn_forward with kv_len set to it, bit for bit when both resolve to the same split count.  Not for the
 * scalar cross-check kernel or an f32 cache (DG_ERR_UNSUPPORTED). */
int dg_attn_forward_dev(const dg_attn_desc* d, const struct dg_step_params* step_dev, const void* q, const void* kv_base,
                        void* out, float* lse, void* workspace, size_t workspace_bytes, void* stream);

/* dg_attn_forward for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no workspace argument.  It has no
 * counterpart in the reference.  The scratch dg_attn_forward takes from its workspace (split
 * partial rows, converted copies of f32 inputs) lives in DG_ATTN_STATIC_SCRATCH_BYTES of device
 * memory inside the library, held on every GPU the library runs on until the process ends; a call
 * whose dg_attn_workspace_bytes() exceeds that returns DG_ERR_SCRATCH_LIMIT and enqueues nothing.
 * 40 MiB covers the model's layers with f16 partial rows (global layer at any prefix: 32.3 MiB;
 * a 1024-row prefill super-chunk: 32.3 MiB), not a global layer with fp32 partial rows (64.3 MiB).
 * Same kernels, same results as dg_attn_forward, bit for bit.  The call allocates and frees
 * nothing; its first call on a device looks the scratch address up (do that once outside a graph
 * capture).  All calls on one GPU share the one scratch: calls that overlap on a GPU (two
 * streams, two threads) race; calls on one stream are ordered and safe. */
#define DG_ATTN_STATIC_SCRATCH_BYTES (40u << 20)
int dg_attn_forward_static(const dg_attn_desc* d, const void* q, const void* kv_base, void* out, float* lse,
                           void* stream);
size_t dg_attn_static_scratch_bytes(void);

/* ---- key-range partials and their merge ----
 *
 * The reference's attention_mma_full can be dispatched once per block of keys, in order, with the
 * softmax state (m, l, unnormalised O) carried in attn_state between the dispatches
 * (src/shaders/attn/attention/attention_mma_full.metal:107-118 state planes, 151-186 resume,
 * 355-368 persist; host loop src/metal/step_kernel/enc.rs:2261-2291).  The same split is the
 * key-length sharding of this path over devices: each holder of a key range produces a state,
 * one exchange later any of them merges.  Two calls expose it:
 *
 * dg_attn_partial attends only the keys t_begin <= t < t_end (positions in the mask's numbering:
 * prefix keys 0 .. kv_len-1, canvas keys kv_len ..; the range may be empty, may end past the last
 * key and need not be aligned) under the descriptor's mask, and writes a state.
 * dg_attn_merge combines 1 .. 16 states of the same descriptor into the output rows (out, in the
 * descriptor's out_dtype and rounding, with lse if not NULL) and/or into a state again (state_out,
 * which may be one of the inputs).  Merging the partials of ranges that tile [0, kv_len + canvas)
 * gives dg_attn_forward's result up to fp32 rounding, whatever the cuts.
 *
 * A state is device memory of dg_attn_state_bytes(): with rows = canvas * n_q_heads and
 * row = canvas_row * n_q_heads + head: float m[rows], float l[rows], then from the next 16-byte
 * boundary float acc[rows][head_dim]; output row = acc / l, log-sum-exp = m + ln l (natural log),
 * l = 0 for a row that saw no key.  (The reference keeps the same three quantities head-major;
 * nothing outside the kernels reads its planes.)  dg_attn_partial leaves states in the normal
 * form l = 1, acc = the normalised row.  The workspace of a partial is sized by
 * dg_attn_partial_workspace_bytes for the same range. */
int dg_attn_state_bytes(const dg_attn_desc* d, size_t* out_bytes);
int dg_attn_partial_workspace_bytes(const dg_attn_desc* d, uint32_t t_begin, uint32_t t_end, size_t* out_bytes);
int dg_attn_partial(const dg_attn_desc* d, uint32_t t_begin, uint32_t t_end, const void* q, const void* kv_base,
                    void* state, size_t state_bytes, void* workspace, size_t workspace_bytes, void* stream);
int dg_attn_merge(const dg_attn_desc* d, const void* const* states, uint32_t n_states, void* out, float* lse,
                  void* state_out, void* stream);

const char* dg_attn_strerror(int status);
uint32_t dg_attn_abi_version(void);
/* Visible (row,key) pairs per head and the FLOP count 4*head_dim*n_q_heads*pairs
 * (reference convention, src/commands/bench.rs:535-536). */
int dg_attn_visible_pairs(const dg_attn_desc* d, uint64_t* pairs, double* flops);

/* ---- the reference's own argument block, for a drop-in call site ---- */

typedef struct dg_layer_offsets {
  uint64_t input_ln, q_proj, q_norm, k_proj, k_norm, v_proj, o_proj, post_attn_ln;
  uint64_t pre_ff_ln, mlp_gate, mlp_up, mlp_down, post_ff_ln_1;
  uint64_t router_scale, router_proj, per_expert_scale, pre_ff_ln_2;
  uint64_t experts_gate_up, experts_down, post_ff_ln_2, post_ff_ln, layer_scalar;
  uint64_t kv_region;
  uint32_t head_dim, n_kv_heads, is_full, kv_ring_mask;
} dg_layer_offsets;

typedef struct dg_step_params {
  uint32_t kv_len, max_steps;
  float entropy_bound, t_min, t_max, conf_threshold;
  uint32_t stability_threshold, min_early_stop_steps, accept_plateau_threshold;
  float plateau_prefix_mean_max;
  uint32_t eos_token_id, kv_write_end;
} dg_step_params;

typedef struct dg_attn_dims {
  uint32_t canvas, n_q_heads, causal, window;
} dg_attn_dims;

typedef struct dg_attn_block_range {
  uint32_t t_begin, t_end, is_first, is_last;
} dg_attn_block_range;

typedef struct dg_debug_status {
  uint32_t code, kernel_id, tg_id, value;
} dg_debug_status;

/* The record a kernel leaves in *dbg is the reference's own, so that the host-side decoder it already has
 * (check_status, src/metal/debug_status.rs:33-75) names the right error in the right kernel: error codes
 * DbgErrorCode (src/shaders/include/debug_status.metal:8-19), kernel ids DbgKernelId
 * (src/shaders/include/dgq_kernels.metal:33-34).  First writer wins (debug_status.metal:38-52).
 *   code 3, kernel 26: a row's softmax denominator was not > 0; value = (canvas row << 16) | query head
 *                      (attention.metal:123, attention_mma2.metal:283, attention_mma_full.metal:371)
 *   code 4, kernel 26: an output element was NaN or infinite; value = its index in the head (of the first
 *                      element of the group a lane stores; attention.metal:129, attention_mma_full.metal:384-389)
 *   code 4, kernel 25: the producer found a head whose 1/rms was not finite; value = canvas row
 *                      (qk_rope_kv.metal:77)
 * tg_id is (canvas row << 16) | head of the row at fault in all three (the reference's call sites leave 0).
 * Code 8 (DbgErrBadDim, qk_rope_kv.metal:48) is never written: head_dim is validated on the host and a bad
 * one is DG_ERR_SHAPE before anything is enqueued.  The top-k entry points take dbg and write nothing: the
 * reference's top-k kernels assert nothing either (attention_topk.metal has no debug_set_error). */
#define DG_DBG_ERR_SOFTMAX_NORM_ZERO 3u
#define DG_DBG_ERR_NONFINITE 4u
#define DG_DBG_ERR_BAD_DIM 8u
#define DG_DBG_KERNEL_QK_ROPE_KV 25u
#define DG_DBG_KERNEL_ATTENTION 26u

/* One layer's attention with exactly the buffers encode_layer_attention_dispatch binds:
 * q = arena+attnq_off (bf16 [canvas][16][hd]), kvcache = whole KV buffer (f16, the kernel adds
 * L->kv_region), out = arena+attno_off, L/P/dims are HOST structs (the reference binds L and P
 * as device buffers; a host copy is what its encoder holds when it encodes the dispatch).
 * dbg: device dg_debug_status (first-writer-wins) or NULL.  attn_state: device scratch of at
 * least dg_attention_state_bytes() bytes (the reference's attn_state buffer, enc.rs:2214-2216).
 * Output is stored with the reference's truncating bf16 store. */
int dg_attention_dispatch(const void* q, const void* kvcache, void* out, const dg_layer_offsets* L,
                          const dg_step_params* P, const dg_attn_dims* dims, dg_debug_status* dbg,
                          void* attn_state, size_t attn_state_bytes, void* stream);
int dg_attention_state_bytes(const dg_layer_offsets* L, const dg_attn_dims* dims, uint32_t kv_len,
                             size_t* out_bytes);

/* dg_attention_dispatch with P bound as the reference binds it: a DEVICE dg_step_params whose kv_len is read when the
 * kernels run.  kv_len_max (host) is the largest prefix the session can reach; attn_state is sized with it
 * (dg_attention_state_bytes(L, dims, kv_len_max)). */
int dg_attention_dispatch_dev(const void* q, const void* kvcache, void* out, const dg_layer_offsets* L,
                              const dg_step_params* P_dev, uint32_t kv_len_max, const dg_attn_dims* dims,
                              dg_debug_status* dbg, void* attn_state, size_t attn_state_bytes, void* stream);

/* dg_attention_dispatch for one block of keys, the way the reference's host loop dispatches
 * attention_mma_full (enc.rs:2261-2291: blocks in order, blk = {t_begin, t_end, is_first, is_last}
 * bound at index 7): the first block starts the state in attn_state, a middle block folds its keys
 * into it, the last block also writes `out`.  A block that is both first and last is
 * dg_attention_dispatch.  attn_state must hold dg_attention_block_state_bytes() and keep its
 * contents between the calls of one sequence.  The result equals the single dispatch up to fp32
 * rounding of the merges (the reference's blocks are bit-identical to its monolithic pass; here
 * each block is itself split over workgroups, so the sums associate differently). */
int dg_attention_dispatch_block(const void* q, const void* kvcache, void* out, const dg_layer_offsets* L,
                                const dg_step_params* P, const dg_attn_dims* dims, const dg_attn_block_range* blk,
                                dg_debug_status* dbg, void* attn_state, size_t attn_state_bytes, void* stream);
int dg_attention_block_state_bytes(const dg_layer_offsets* L, const dg_attn_dims* dims, uint32_t kv_len,
                                   size_t* out_bytes);

/* ---- top-k sparse attention (full-attention layers; the reference's default for them at depth) ----
 *
 * Replaces the three Metal kernels attn_gemm_qk (with the u16 key plane) + attn_topk_softmax +
 * attn_topk_pv (src/shaders/attn/attention_topk/attention_topk.metal; encoded by
 * StepEnc::encode_attn_decomp, src/metal/step_kernel/enc.rs:1820-2100) and their CPU twin
 * (attention_topk/cpu.rs:41-120).  Per (query row, head): scores over the visible keys, the k
 * highest kept (exact by fp32 score; equal scores: lower key position first, the CPU twin's
 * rule), softmax over the kept keys only, their V rows summed.  Same descriptor, tensors, masks
 * and layouts as dg_attn_forward; Q and the cache must be bf16 or f16 (no f32 inputs), LSE is
 * not produced.
 *
 * k_cfg = the reference's (fixed_k | chunk grid, dyn_divisor, k_min, k_max)
 * (src/flags/accessors.rs:210-221, attention_topk.metal:160-182): divisor 0 keeps k_cfg[0] keys
 * (at least 1); otherwise a row keeps clamp(t_equiv / divisor, k_min, k_max) keys, t_equiv being
 * its number of visible keys, rounded up to the grid for causal rows.  Never more than the row
 * sees, never more than 1024. */
int dg_attn_topk_workspace_bytes(const dg_attn_desc* d, const uint32_t* k_cfg, size_t* out_bytes);
int dg_attn_topk_forward(const dg_attn_desc* d, const uint32_t* k_cfg, const void* q, const void* kv_base,
                         void* out, void* workspace, size_t workspace_bytes, void* stream);

/* The same with the reference's argument block (bf16 Q/out with the truncating store, f16 cache at
 * L->kv_region); `scratch` stands for the S / P / Idx / pattern planes the reference allocates
 * (attention_topk/mod.rs:121-128), sized by dg_attention_topk_state_bytes. */
int dg_attention_topk_state_bytes(const dg_layer_offsets* L, const dg_attn_dims* dims, uint32_t kv_len,
                                  const uint32_t* k_cfg, size_t* out_bytes);
int dg_attention_topk_dispatch(const void* q, const void* kvcache, void* out, const dg_layer_offsets* L,
                               const dg_step_params* P, const dg_attn_dims* dims, const uint32_t* k_cfg,
                               dg_debug_status* dbg, void* scratch, size_t scratch_bytes, void* stream);

/* ---- the producer of the rows attention reads: per-head RMSNorm + RoPE + KV-cache write ----
 * Replaces the reference's qk_rope_kv kernel (src/shaders/attn/qk_rope_kv/qk_rope_kv.metal:29-149,
 * encoded by StepEnc::encode_layer_qk_rope_kv, src/metal/step_kernel/enc.rs:1739-1804; CPU twin
 * src/shaders/attn/cpu.rs:78-145).  For canvas row tok at position pos = kv_len + tok:
 *   Q head:  q <- rope(rms_norm(q) * q_norm_w, pos), in place
 *   K head:  x  = rope(rms_norm(k) * k_norm_w, pos); cache K row at slot(pos) <- x;
 *            k <- x in place unless V aliases the raw k projection (v_from_k)
 *   V head:  cache V row at slot(pos) <- rms_norm(v_from_k ? raw k : v), no weight
 * is_full selects proportional RoPE (pairs (d, hd/2+d), d < hd/8, theta 1e6), otherwise
 * split-half over the whole head (pairs (d, hd/2+d), theta 1e4).  RoPE uses the absolute
 * position; only the storage slot is ring-mapped.  Positions >= kv_write_end are not written
 * to the cache (prefill pad rows, qk_rope_kv.metal:56-60). */
#define DG_ROPE_F_QK_TRUNCATE 0x1u  /* store q/k with the reference's truncating bf16 store; default RNE */

typedef struct dg_rope_desc {
  uint32_t canvas, n_q_heads, n_kv_heads;
  uint32_t head_dim;        /* 32, 64, 128, 256 or 512 */
  uint32_t kv_len;          /* StepParams.kv_len */
  uint32_t kv_write_end;    /* StepParams.kv_write_end; 0xffffffff = write every row */
  uint32_t kv_ring_mask;    /* LayerOffsets.kv_ring_mask */
  uint32_t is_full;         /* LayerOffsets.is_full */
  uint32_t v_from_k;        /* LayerOffsets.v_proj == 0 */
  uint32_t kv_dtype;        /* DG_F16 or DG_BF16: element type of the cache */
  uint32_t flags;
  uint32_t reserved;
  uint64_t kv_region_bytes; /* byte offset of this layer's region inside kv_base */
  /* element strides/offsets inside the region, as in dg_attn_desc */
  int64_t  k_tok_stride, k_head_stride;
  int64_t  v_base_off, v_tok_stride, v_head_stride;
} dg_rope_desc;

/* q [canvas][n_q_heads][hd], k and v [canvas][n_kv_heads][hd]: bf16, device.  q_norm_w, k_norm_w:
 * [hd] bf16, device.  v may be NULL when v_from_k.  Enqueues one kernel on `stream`. */
int dg_qk_rope_kv(const dg_rope_desc* d, void* q, void* k, const void* v, void* kv_base, const void* q_norm_w,
                  const void* k_norm_w, dg_debug_status* dbg, void* stream);

/* dg_qk_rope_kv with kv_len and kv_write_end read from a DEVICE dg_step_params when the kernel runs (the reference
 * binds StepParams as a device buffer, qk_rope_kv.metal:30-38); d->kv_len and d->kv_write_end are ignored.  Pairs
 * with dg_attn_forward_dev: a recorded producer + attention sequence follows the committed prefix without being
 * recorded again.  The cache must have room for the largest prefix + canvas the caller will set. */
int dg_qk_rope_kv_dev(const dg_rope_desc* d, const struct dg_step_params* step_dev, void* q, void* k, const void* v,
                      void* kv_base, const void* q_norm_w, const void* k_norm_w, dg_debug_status* dbg, void* stream);

/* The same with exactly the buffers the reference kernel binds (qk_rope_kv.metal:30-38): q, k, v
 * in the arena, the whole f16 KV buffer (the kernel adds L->kv_region), the weight blob (norm
 * weights at L->q_norm / L->k_norm, bf16), host copies of L / P / dims.  q and k are stored with
 * the reference's truncating bf16 store, the cache as f16 (kv_store). */
int dg_qk_rope_kv_dispatch(void* q, void* k, void* v, void* kvcache, const void* blob, const dg_layer_offsets* L,
                           const dg_step_params* P, const dg_attn_dims* dims, dg_debug_status* dbg, void* stream);
/* ... with P bound as a device buffer, as the reference binds it */
int dg_qk_rope_kv_dispatch_dev(void* q, void* k, void* v, void* kvcache, const void* blob, const dg_layer_offsets* L,
                               const dg_step_params* P_dev, const dg_attn_dims* dims, dg_debug_status* dbg, void* stream);

/* ---- KV-cache layout arithmetic (host) ---- */
uint64_t dg_kv_row_bytes(uint32_t head_dim, uint32_t kv_dtype);
uint64_t dg_kv_region_bytes(uint32_t n_kv_heads, uint32_t head_dim, uint64_t slots, uint32_t kv_dtype);
uint64_t dg_kv_slot(uint32_t kv_ring_mask, uint64_t pos);
uint64_t dg_layer_kv_slots(int is_full, uint64_t max_seq, uint64_t ring_slots_cap);

/* ---- KV-cache snapshots: the live part of every layer's region <-> a compact blob ----
 *
 * Replaces gather_kv_prefix / scatter_kv_prefix (src/metal/step_kv/mod.rs:108-151) and the byte
 * walk of StepRuntime::live_kv_fnv (src/metal/step_kernel/runtime.rs:118-148), which in the
 * reference are host loops over unified memory.  The blob keeps the reference's format whatever
 * layout the cache uses: layers concatenated; per layer, position after position, a row of
 * [K: Hkv x head_dim | V: Hkv x head_dim] elements.  A snapshot takes the first
 * min(kv_len, slots) physical slots of a layer as they lie (ring layers too); the live stream is
 * what the fingerprint hashes: linear layers their positions [0, kv_len), ring layers their last
 * min(kv_len, window) positions in position order.  All pointers are device pointers; the calls
 * enqueue one kernel per 32 layers on `stream` and return. */
typedef struct dg_kv_layer {
  uint64_t kv_region_bytes;  /* byte offset of the layer's region inside kv_base (LayerOffsets.kv_region) */
  uint32_t n_kv_heads, head_dim;
  uint32_t slots;            /* capacity of the region in positions (layer_kv_slots) */
  uint32_t kv_ring_mask;     /* 0 = linear */
  uint32_t kv_dtype;         /* DG_F16 / DG_BF16 / DG_F32 */
  uint32_t reserved;
  /* element strides/offsets inside the region, as in dg_attn_desc */
  int64_t  k_tok_stride, k_head_stride;
  int64_t  v_base_off, v_tok_stride, v_head_stride;
} dg_kv_layer;
void dg_kv_layer_reference_layout(dg_kv_layer* l);   /* [slot][K heads | V heads] */
void dg_kv_layer_head_major_layout(dg_kv_layer* l);  /* K plane [Hkv][slots][hd], then V plane */

/* layer_offsets (n_layers entries, may be NULL) receives each layer's byte offset in the blob */
int dg_kv_snapshot_bytes(const dg_kv_layer* layers, uint32_t n_layers, uint64_t kv_len, uint64_t* total_bytes,
                         uint64_t* layer_offsets);
int dg_kv_snapshot_gather(const void* kv_base, const dg_kv_layer* layers, uint32_t n_layers, uint64_t kv_len,
                          void* blob, size_t blob_bytes, void* stream);
int dg_kv_snapshot_scatter(void* kv_base, const dg_kv_layer* layers, uint32_t n_layers, uint64_t kv_len,
                           const void* blob, size_t blob_bytes, void* stream);
int dg_kv_live_bytes(const dg_kv_layer* layers, uint32_t n_layers, uint64_t kv_len, uint32_t window,
                     uint64_t* total_bytes);
int dg_kv_live_gather(const void* kv_base, const dg_kv_layer* layers, uint32_t n_layers, uint64_t kv_len,
                      uint32_t window, void* stream_bytes, size_t capacity, void* stream);
/* FNV-1a over host bytes, continuing seed_hash (runtime.rs:127-133); the hash is a serial
 * recurrence, so the fingerprint is dg_kv_live_gather + a copy to the host + this. */
uint64_t dg_fnv1a64(const void* bytes, size_t n, uint64_t seed_hash);

#ifdef __cplusplus
}
#endif
#endif
