/* Measurement aids of libdg_attn_hip.so: kernel timing with HIP events and two calibration
 * kernels.  None of this is part of the drop-in boundary (include/dg_attn.h) and none of it has a
 * counterpart in the reference; bench.py is the only caller. */
#ifndef DG_ATTN_BENCH_H
#define DG_ATTN_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- optional kernel timing (measurement aid; no counterpart in the reference, whose
 * harness times whole command buffers: src/shaders/attn/harness.rs:149-170) ----
 * Between dg_prof_begin and dg_prof_end every dg_attn_forward issued by the calling thread
 * records one HIP event pair on its stream around the main attention kernel only (the
 * merge and conversion kernels stay outside the pair).  dg_prof_end waits for the last
 * recorded event, returns the summed kernel time and releases the events. */
int dg_prof_begin(uint32_t max_launches);
int dg_prof_end(double* main_kernel_ms_total, uint32_t* n_launches);
/* dg_attn_topk_forward records two pairs per block of canvas rows instead: one around the score
 * kernel, then one around the select kernel.  dg_prof_end_split ends the session like dg_prof_end
 * and returns the time of the even-numbered pairs (0, 2, ...: the score kernels of a top-k
 * session) and of the odd-numbered ones (the select kernels) separately. */
int dg_prof_end_split(double* even_ms_total, double* odd_ms_total, uint32_t* n_pairs);

/* Plain device-to-device copy of `bytes` (multiple of 16) with a kernel of this library: a
 * launch of known HBM traffic (bytes read + bytes written) that the FETCH_SIZE / WRITE_SIZE
 * profiler counters are scaled by.  Measurement aid, no counterpart in the reference. */
int dg_calib_copy(void* dst, const void* src, size_t bytes, void* stream);

/* Launch of nothing but bf16 32x32x16 MFMAs (`workgroups` x 4 waves x `iters` x 16) writing
 * `*flops` = the floating-point operations it performs; the caller times it.  `sink` (at
 * least workgroups*256 floats, device memory) is never written in practice.  What this
 * sustains is the MFMA ceiling of the machine at hand, next to which the attention kernel's
 * rate is read.  `random_operands` = 0: near-constant operands (the multipliers draw little
 * power and the clock stays high); 1: operands of random sign, exponent and mantissa, which
 * is what attention feeds the matrix cores (the clock the chip then holds is lower); 2, 3: as
 * 1 with three quarters / 95 % of one operand's elements zero.
 * Measurement aid, no counterpart in the reference. */
int dg_calib_mfma(float* sink, size_t sink_bytes, uint32_t workgroups, uint32_t iters, uint32_t random_operands,
                  uint64_t* flops, void* stream);

#ifdef __cplusplus
}
#endif
#endif
