/* hip_decode_debug.h -- verification and diagnostic entry points of libhipdecode.so.
 *
 * Not part of the drop-in boundary (include/hip_decode.h): nothing here has a counterpart in
 * crates/metal-decode/src/lib.rs.  The parity tests use these calls to look inside the library (stored
 * weights, the draw kernels on crafted inputs, the restated C-library functions), the profiling front
 * end uses the time-stamp builds of the persistent kernels, and the benchmark uses the calibration
 * copy.  Same conventions as hip_decode.h: extern "C", plain pointers and sizes, status codes. */
#ifndef HIP_DECODE_DEBUG_H
#define HIP_DECODE_DEBUG_H

#include "hip_decode.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Debug/verification: copy one stored weight matrix back as fp32 after de-quantisation, in
 * out-major [rows][k] order.  which: 0 wqkv (rows q_dim+2*kv_dim, k dim), 1 wo (dim, q_dim),
 * 2 w13 (2*hidden interleaved gate/up rows, dim), 3 w2 (dim, hidden), 4 embed (vocab, dim). */
int hipdec_export_weight(hipdec_model *m, size_t layer_idx, uint32_t which, float *out, size_t cap);

/* Diagnostic: runs one greedy step with the persistent step kernel and returns the wall-clock stamps
 * (100 MHz ticks) workgroup 0 took at its phase boundaries: (nlayers + 1) * 32 slots, unused ones 0. */
int hipdec_debug_step_profile(hipdec_model *m, uint32_t token, uint64_t *out, size_t cap, size_t *out_count);

/* Diagnostic: one step of the open batch (tokens[n_rows], as hipdec_decode_token_argmax_from_ids_batch without
 * the tokens) with the build of the one-launch layer kernel that takes time stamps: 16 slots per layer of
 * workgroup 0's wall clock (100 MHz ticks) at its phase boundaries, (nlayers + 1) * 16 values, unused ones 0.
 * HIPDEC_ERR_UNSUPPORTED when hipdec_batch_layers_in_one_launch says 0. */
int hipdec_debug_batch_step_profile(hipdec_model *m, const uint32_t *tokens, uint64_t *out, size_t cap, size_t *out_count);

/* Diagnostic: `reps` launches of a plain device-to-device copy kernel (k_calib_copy) of `bytes` bytes,
 * the known-size yardstick that hardware memory-traffic counters are scaled by. */
int hipdec_debug_calibration_copy(size_t bytes, int reps);

/* Verification: the draw kernels of the sampled runs on caller-supplied inputs (one row).  top-k: the
 * per-block candidate lists vals/idxs[blocks * top_k] as hipdec_decode_token_topk_from_id returns them
 * (engine/src/decode.rs:218-253 merge, engine/src/inference.rs:823-849 draw); full vocabulary: raw
 * logits[vocab] with their block statistics maxes/sums[ceil(vocab / 256)] (inference.rs:851-921).
 * *rng_state in and out, *out_token = the drawn token. */
int hipdec_debug_sample_topk(const float *vals, const uint32_t *idxs, size_t blocks, uint32_t top_k, float temperature,
                             float softcap, uint64_t *rng_state, uint32_t *out_token);
int hipdec_debug_sample_fullvocab(const float *logits, size_t vocab, const float *maxes, const float *sums,
                                  float temperature, float softcap, uint64_t *rng_state, uint32_t *out_token);
/* 1 when this host's C library computes expf and tanhf as the on-device sampler reproduces them
 * (the probe the sampled runs consult), else 0. */
int hipdec_debug_hostmath_probe(void);
/* Verification of the two host C library functions the on-device sampler restates (fn 0: expf,
 * fn 1: tanhf): evaluate the restatement for n inputs on the host (on_device = 0) or on the GPU; */
int hipdec_debug_hostmath_eval(int fn, const float *in, float *out, size_t n, int on_device);
/* an order-independent checksum of its results over `count` consecutive float bit patterns starting
 * at first_bits, computed on the host (with host_threads threads) or on the GPU: equal checksums
 * mean equal results; */
int hipdec_debug_hostmath_checksum(int fn, uint32_t first_bits, uint64_t count, int on_device, int host_threads,
                                   uint64_t *out);
/* and the number of those inputs for which the host evaluation differs from the C library's function. */
int hipdec_debug_hostmath_count_mismatch(int fn, uint32_t first_bits, uint64_t count, int host_threads,
                                         uint64_t *out_mismatches);

/* Which form the single-row token step of this model takes: 0 one kernel per product, 1 the persistent
 * kernel (hipdec_mega.h), 2 its short-phase form for bf16 models whose reduction lengths are multiples of
 * 512 (hipdec_lean.h).  Environment HIPDEC_NO_LEAN=1 / HIPDEC_NO_MEGA=1 at creation select the earlier forms. */
int hipdec_debug_step_kernel(const hipdec_model *m, int *out);

/* The launch of one product P[splits][rows][n] = A[rows][k] x W[n][k]^T of the prompt prefill and the
 * multi-row step on a device of num_cu compute units, worked out on the host (no GPU needed): out[0] the
 * kernel (0 tiled, 1 tiled with its operands loaded straight into LDS, 2 few-row, 3 few-row for 4-bit
 * weights, 4 few-row for e4m3 weights), out[1] the K splits (planes written), out[2] the reduction steps per
 * split (32 elements each in the few-row kernels, 64 in the tiled ones), out[3..5] the grid, out[6] the
 * threads per workgroup, out[7] the dynamic LDS bytes.  It is the plan the library's own launches follow;
 * tests check it against what the kernels assume (whole scale groups per split, the staged rows within the
 * LDS budget, no empty split).  HIPDEC_ERR_ARG for shapes the library never launches (k not a multiple of
 * 32, of 128 for 4-bit weights; fp32 weights with more than 32 rows). */
int hipdec_debug_gemm_plan(uint32_t weight_dtype, int rows, int n, int k, int num_cu, uint64_t out[8]);

/* Test hook for the bounded waits of the persistent kernels (every wait on another workgroup gives up
 * after a number of polls, raises the model's abort flag and every workgroup leaves; the host call then
 * returns HIPDEC_ERR_HIP and later steps take the one-kernel-per-product path).  check_mask: a waiting
 * thread looks at its poll count when (count & check_mask) == 0; limit: the count it gives up at.
 * (0, 0) makes the first stale poll of any thread give up -- every kernel still exits normally --;
 * (127, 1 << 22) are the defaults.  Process-wide, current device; takes effect for launches enqueued
 * after the call. */
int hipdec_debug_set_spin_limit(uint32_t check_mask, uint32_t limit);

#ifdef __cplusplus
}
#endif
#endif /* HIP_DECODE_DEBUG_H */
