/*
 * hip_decode.h -- C ABI of the MI355X (gfx950) decode backend for rustane.
 *
 * This is the boundary a `hip-decode` FFI crate binds: one entry point per public item of the
 * reference's `metal_decode::Model` (crates/metal-decode/src/lib.rs), plus the few additions a
 * backend without an Apple Neural Engine needs (prompt prefill, full logits, multi-token runs).
 * Plain pointers and sizes only; every call returns a status code and never aborts the process
 * (the reference panics where this returns HIPDEC_ERR_*).
 *
 * Threading: one model owns one HIP stream.  Calls on one model are synchronous and not
 * re-entrant; distinct models may be used from distinct threads.
 */
#ifndef HIP_DECODE_H
#define HIP_DECODE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Constants that are part of the interface (crates/metal-decode/src/lib.rs:14-15, :156, :201). */
#define HIPDEC_MAX_GPU_TOPK 32u   /* MAX_GPU_TOPK, lib.rs:15 */
#define HIPDEC_HEAD_BLOCK 256u    /* vocab rows per head block, lib.rs:156 (argmax_threads) */
#define HIPDEC_RMS_EPS 1e-5f      /* RMS_EPS, lib.rs:14 */

typedef enum {
    HIPDEC_OK = 0,
    HIPDEC_ERR_ARG = 1,      /* bad argument: null pointer, short buffer, token >= vocab, k out of range */
    HIPDEC_ERR_FULL = 2,     /* len >= cfg.seq: the KV window is full (lib.rs:242-245 panics here) */
    HIPDEC_ERR_HIP = 3,      /* a HIP runtime call failed; see hipdec_last_error */
    HIPDEC_ERR_UNSUPPORTED = 4 /* shape or option this build has no kernel for */
} hipdec_status;

typedef enum {
    HIPDEC_W_F32 = 0,        /* weights streamed as fp32 (the reference's precision) */
    HIPDEC_W_BF16 = 1,       /* round-to-nearest-even bf16 */
    HIPDEC_W_FP8_E4M3 = 2,   /* OCP e4m3fn, per-output-channel fp32 scale amax/448; embed stays bf16 */
    HIPDEC_W_INT4_G128 = 3   /* symmetric 4-bit, groups of 128 along the reduction axis, bf16 scale
                                amax/7; embed stays bf16 */
} hipdec_weight_dtype;

typedef enum {
    HIPDEC_KV_F32 = 0,
    HIPDEC_KV_BF16 = 1
} hipdec_kv_dtype;

/* metal_decode::Config, lib.rs:22-35 (same fields, same meaning). */
typedef struct {
    uint32_t dim, hidden, heads, kv_heads, hd, seq, nlayers, vocab, q_dim, kv_dim, gqa_ratio;
} hipdec_config;

/* metal_decode::LayerInit, lib.rs:37-47.  Row-major fp32, borrowed for the call only:
 * wq[dim*q_dim], wk/wv[dim*kv_dim], wo[q_dim*dim], w1/w3[dim*hidden] with row = input channel;
 * w2[dim*hidden] with row = output channel; gamma1/gamma2[dim]. */
typedef struct {
    const float *wq, *wk, *wv, *wo, *w1, *w3, *w2, *gamma1, *gamma2;
} hipdec_layer_f32;

/* metal_decode::FinalHeadInit, lib.rs:49-52: gamma_final[dim], embed[vocab*dim] (tied LM head). */
typedef struct {
    const float *gamma_final, *embed;
} hipdec_head_f32;

typedef struct {
    uint32_t weight_dtype;   /* hipdec_weight_dtype */
    uint32_t kv_dtype;       /* hipdec_kv_dtype */
    int32_t device;          /* HIP device ordinal */
    uint32_t ffn_activation; /* 0 = SwiGLU, 1 = leaky_relu(x, 0.5)^2  (engine/src/model.rs:3-7) */
    uint32_t flags;          /* HIPDEC_FLAG_* */
    uint32_t max_rows;       /* rows of the batched decode entry points (0 or 1 = single row) */
} hipdec_options;

#define HIPDEC_FLAG_NO_GRAPH 1u   /* launch kernels eagerly instead of replaying a captured hipGraph */
#define HIPDEC_FLAG_NO_MEGA 2u    /* one kernel per matrix product instead of the persistent per-token kernel */
#define HIPDEC_FLAG_PREFILL_STEPS 4u /* hipdec_prefill runs one token step per prompt row instead of the
                                        chunked matrix-core path (which bf16 and e4m3 weights use by default) */
#define HIPDEC_FLAG_PREFILL_BF16_ACT 8u /* the chunked prefill's GEMMs multiply the weights by the activations rounded
                                        to one bf16 number instead of the (hi, lo) pair that keeps 16 mantissa bits:
                                        half the matrix-core work, prompt logits within ~1e-2 of the token path
                                        (meant for 8-bit / 4-bit weights, whose own rounding is coarser) */
#define HIPDEC_FLAG_PREFILL_F16_ACT 16u /* the same with the activations rounded to one fp16 number (11 mantissa bits,
                                        saturating at +-65504; the weights are widened to fp16 exactly): half the
                                        matrix-core work, the precision of the reference's own fp16 prefill;
                                        the default of 8-bit / 4-bit models with a bf16 cache */
#define HIPDEC_FLAG_PREFILL_PAIR_ACT 32u /* the (hi, lo) bf16 pair, 16 mantissa bits (the default of every other
                                        model), also for those */

typedef struct hipdec_model hipdec_model;

/* Model::new, lib.rs:147-207.  Copies (and converts) the weights to device memory; the caller
 * keeps ownership of every pointer.  n_layers must equal cfg->nlayers (lib.rs:186-188). */
int hipdec_create(const hipdec_config *cfg, const hipdec_layer_f32 *layers, size_t n_layers,
                  const hipdec_head_f32 *head, const hipdec_options *opts, hipdec_model **out);
void hipdec_destroy(hipdec_model *m);

/* A second model on the weights `base` already holds on its device: same configuration and weight
 * format, KV caches, step state and workspaces of its own, no upload.  The weights stay alive until the
 * last model using them is destroyed (in any order).  (No counterpart in the reference, where every
 * Model::new uploads its own copy, lib.rs:147-207; a server that keeps several prompts' sessions resident
 * pays the weights once with this.) */
int hipdec_create_shared(const hipdec_model *base, uint32_t kv_dtype, uint32_t flags, hipdec_model **out);

/* Text of the last error on this model (or of the last failed hipdec_create when m is NULL). */
const char *hipdec_last_error(const hipdec_model *m);

/* Model::len / Model::set_len, lib.rs:209-215 (set_len clamps to cfg.seq). */
size_t hipdec_len(const hipdec_model *m);
int hipdec_set_len(hipdec_model *m, size_t len);

/* How hipdec_prefill carries activations into its GEMMs from now on: 0 the (hi, lo) bf16 pair
 * (HIPDEC_FLAG_PREFILL_PAIR_ACT), 1 one bf16 number (_BF16_ACT), 2 one fp16 number (_F16_ACT).
 * (No counterpart in the reference, whose prefill precision is fixed by the ANE's fp16; the other flags
 * are fixed at hipdec_create.) */
int hipdec_set_prefill_activations(hipdec_model *m, int mode);

/* Model::seed_layer_cache_from_channel_first, lib.rs:217-237:
 * cache[pos*kv_dim + d] = k_rope_cf[d*seq + pos] for pos < live_len, the rest zero. */
int hipdec_seed_layer_cache_from_channel_first(hipdec_model *m, size_t layer_idx, size_t live_len,
                                               const float *k_rope_cf, const float *v_cf);

/* Model::decode_token, lib.rs:239-269: x_in[dim] -> layers -> x_out[dim]; len += 1. */
int hipdec_decode_token(hipdec_model *m, const float *x_in, float *x_out);
/* Model::decode_token_from_id, lib.rs:271-304. */
int hipdec_decode_token_from_id(hipdec_model *m, uint32_t token, float *x_out);
/* Model::decode_token_argmax, lib.rs:306-338. */
int hipdec_decode_token_argmax(hipdec_model *m, const float *x_in, uint32_t *out_token);
/* Model::decode_token_argmax_from_id, lib.rs:340-375: final norm, tied LM head, argmax with ties
 * to the lower index (lib.rs:1553, :1749); no softcap (monotone). */
int hipdec_decode_token_argmax_from_id(hipdec_model *m, uint32_t token, uint32_t *out_token);
/* Model::decode_token_topk_from_id, lib.rs:377-434: per 256-row block, the top_k largest raw
 * logits (value desc, index asc), padded with (-inf, 0xffffffff).  Writes blocks*top_k pairs;
 * cap = capacity of both output arrays in elements; *out_count = blocks*top_k. */
int hipdec_decode_token_topk_from_id(hipdec_model *m, uint32_t token, uint32_t top_k,
                                     float *out_vals, uint32_t *out_idxs, size_t cap,
                                     size_t *out_count);
/* Model::decode_token_block_stats_from_id, lib.rs:436-487: z = softcap(logit) * inv_temperature;
 * per block max z and sum exp(z - max).  *out_count = blocks. */
int hipdec_decode_token_block_stats_from_id(hipdec_model *m, uint32_t token, float inv_temperature,
                                            float softcap, float *out_maxes, float *out_sums,
                                            size_t cap, size_t *out_count);
/* Model::materialize_current_logits_block, lib.rs:489-511: softcapped (not temperature-scaled)
 * logits of one block of the step that ran last; does not advance len.
 * *out_valid = min(256, vocab - 256*block_idx). */
int hipdec_materialize_current_logits_block(hipdec_model *m, size_t block_idx, float softcap,
                                            float *out_logits, size_t cap, size_t *out_valid);

/* ---- additions with no counterpart in metal_decode::Model ---- */

/* The work of DecodeContext::decode_next_logits (engine/src/decode.rs:91-127) done on the GPU:
 * layers, final RMSNorm, tied LM head, optional softcap; out_logits[vocab]. */
int hipdec_decode_logits_from_id(hipdec_model *m, uint32_t token, float softcap, float *out_logits);

/* Prompt prefill (the reference prefills on the ANE, engine/src/inference.rs:136-144): runs
 * positions len .. len+n-1 with causal attention, fills the KV cache, len += n.  last_logits
 * (nullable, [vocab]) receives the softcapped logits of the last position. */
int hipdec_prefill(hipdec_model *m, const uint32_t *ids, size_t n, float softcap, float *last_logits);

/* ---- multi-sample decode: n_rows continuations of one shared prefix, stepped together ----
 *
 * The reference draws its `samples` one after the other, re-seeding the KV cache from the shared
 * prompt caches for each (engine/src/inference.rs:247-262, :561).  Here the rows share cache
 * positions [0, len) as they are when hipdec_batch_begin is called and each row appends to a
 * suffix cache of its own, so every weight matrix is streamed once per step for all rows.  Row r of
 * every batched call returns what the single-row call of the same name would return for a model
 * that had decoded row r's tokens alone.  Between begin and end only the *_batch calls may be
 * used; hipdec_batch_end leaves len and the shared positions as they were.  1 <= n_rows <= 32;
 * needs model dimensions that are multiples of 32 (128 with 4-bit weights);
 * HIPDEC_ERR_UNSUPPORTED otherwise. */
int hipdec_batch_begin(hipdec_model *m, size_t n_rows);
int hipdec_batch_end(hipdec_model *m);
/* steps taken since hipdec_batch_begin (each row is at position len + steps) */
int hipdec_batch_steps(const hipdec_model *m, size_t *out_steps);
/* Diagnostic, no counterpart in the reference: *out = 1 when the open batch runs the layers of a step as
 * one persistent launch (bf16 weights, at most 8 rows, dimensions that are multiples of 256 within the
 * kernel's register budget), 0 when it runs one kernel per product. */
int hipdec_batch_layers_in_one_launch(const hipdec_model *m, int *out);
/* tokens[n_rows]; out_logits[n_rows][vocab]  (hipdec_decode_logits_from_id per row) */
int hipdec_decode_logits_from_ids_batch(hipdec_model *m, const uint32_t *tokens, float softcap, float *out_logits);
/* tokens[n_rows] -> out_tokens[n_rows]  (Model::decode_token_argmax_from_id per row, lib.rs:340-375) */
int hipdec_decode_token_argmax_from_ids_batch(hipdec_model *m, const uint32_t *tokens, uint32_t *out_tokens);
/* out_vals/out_idxs[n_rows][blocks*top_k], cap = capacity of each array in elements, *out_count =
 * blocks*top_k per row  (Model::decode_token_topk_from_id per row, lib.rs:377-434) */
int hipdec_decode_token_topk_from_ids_batch(hipdec_model *m, const uint32_t *tokens, uint32_t top_k,
                                            float *out_vals, uint32_t *out_idxs, size_t cap, size_t *out_count);
/* out_maxes/out_sums[n_rows][blocks], *out_count = blocks per row
 * (Model::decode_token_block_stats_from_id per row, lib.rs:436-487) */
int hipdec_decode_token_block_stats_from_ids_batch(hipdec_model *m, const uint32_t *tokens, float inv_temperature,
                                                   float softcap, float *out_maxes, float *out_sums, size_t cap,
                                                   size_t *out_count);
/* Model::materialize_current_logits_block for one row of the last batched step (lib.rs:489-511) */
int hipdec_materialize_current_logits_block_batch(hipdec_model *m, size_t row, size_t block_idx, float softcap,
                                                  float *out_logits, size_t cap, size_t *out_valid);

/* Greedy run without a host round trip per token (the loop of engine/src/inference.rs:576-585):
 * starting from `token`, performs n_steps argmax steps, each feeding its result to the next;
 * out_tokens[n_steps].  Equivalent to n_steps calls of hipdec_decode_token_argmax_from_id. */
int hipdec_decode_greedy_run(hipdec_model *m, uint32_t token, size_t n_steps, uint32_t *out_tokens);

/* Sampled runs without a host round trip per token.  The reference finishes every sampled step on
 * the CPU: it merges the per-block candidates and draws among them (engine/src/inference.rs:586-599,
 * engine/src/decode.rs:218-253, inference.rs:823-849), or draws a block from the block statistics
 * and then a token from that block's logits (inference.rs:600-625, :851-921).  These calls do the
 * same merge and the same draws on the GPU, in the host's operation order and with the host C
 * library's expf reproduced bit for bit, feed each drawn token to the next step on the device and
 * return n_steps tokens at once; *rng_state is the sampler's 64-bit LCG state (inference.rs:759-768),
 * read at entry and advanced exactly as the host loop would advance it.  Equivalent to n_steps
 * rounds of hipdec_decode_token_topk_from_id + host merge + host draw (resp.
 * hipdec_decode_token_block_stats_from_id + block draw + hipdec_materialize_current_logits_block +
 * token draw); with softcap > 0 the top-k form applies cap * tanhf(v / cap) to the merged candidates
 * as the host does (decode.rs:155-159), the host C library's tanhf reproduced bit for bit as well.
 * Needs vocab <= 262144, and a host C library whose expf and tanhf are the ones reproduced (probed
 * once per process on 2^21 inputs); HIPDEC_ERR_UNSUPPORTED otherwise, and nothing has run. */
int hipdec_decode_topk_sampled_run(hipdec_model *m, uint32_t token, uint32_t top_k, float temperature, float softcap,
                                   uint64_t *rng_state, size_t n_steps, uint32_t *out_tokens);
int hipdec_decode_fullvocab_sampled_run(hipdec_model *m, uint32_t token, float temperature, float softcap,
                                        uint64_t *rng_state, size_t n_steps, uint32_t *out_tokens);
/* The same for every row of an open batch: tokens[n_rows], rng_states[n_rows] (row r draws from its
 * own state, the reference's seed + r, inference.rs:256), out_tokens[n_steps][n_rows]. */
int hipdec_decode_topk_sampled_run_batch(hipdec_model *m, const uint32_t *tokens, uint32_t top_k, float temperature,
                                         float softcap, uint64_t *rng_states, size_t n_steps, uint32_t *out_tokens);
int hipdec_decode_fullvocab_sampled_run_batch(hipdec_model *m, const uint32_t *tokens, float temperature, float softcap,
                                              uint64_t *rng_states, size_t n_steps, uint32_t *out_tokens);

/* Device time of the last call that ran a step (a single decode step, a multi-row step,
 * hipdec_decode_greedy_run, hipdec_prefill), measured with HIP events on the model's stream: total
 * milliseconds of that call's kernels. */
int hipdec_last_device_ms(const hipdec_model *m, float *out_ms);

/* Bytes of device memory the model streams per decoded token at the given live KV length
 * (weights + scales + norms + one embedding row + KV read/write): the algorithmic traffic the
 * bandwidth roofline is computed from. */
int hipdec_bytes_per_token(const hipdec_model *m, size_t kv_len, uint64_t *out_bytes);

/* Offline conversion.  The reference's loader reads fp32 RSTK files (engine/src/checkpoint.rs:25-242) and the
 * model converts them when it is created (lib.rs:159-202 uploads fp32; here also bf16 / e4m3 / 4-bit).  These
 * entry points, which have no counterpart in the reference, let a caller do that conversion once: copy the
 * stored weights of a model out (exactly the bytes the kernels read: fused q/k/v rows, interleaved gate/up
 * rows, every matrix [rows][k] in the weight format, then its scales), keep them in a file, and create later
 * models from them with plain copies -- an eighth of the fp32 bytes for 4-bit weights, and no staging.
 * hipdec_packed_sizes_of needs no GPU; sizes are bytes per layer array and for the embedding. */
typedef struct hipdec_packed_sizes {
    uint64_t wqkv, wo, w13, w2, s_qkv, s_wo, s_w13, s_w2, gamma, embed;
} hipdec_packed_sizes;
typedef struct hipdec_packed_layer {
    const void *wqkv, *wo, *w13, *w2;          /* hipdec_packed_sizes bytes each */
    const void *s_qkv, *s_wo, *s_w13, *s_w2;   /* scales; unused (size 0) for fp32 and bf16 weights */
    const float *gamma1, *gamma2;
} hipdec_packed_layer;
typedef struct hipdec_packed_head {
    const float *gamma_final;
    const void *embed;                         /* fp32 with fp32 weights, bf16 otherwise */
} hipdec_packed_head;
int hipdec_packed_sizes_of(const hipdec_config *cfg, uint32_t weight_dtype, hipdec_packed_sizes *out);
int hipdec_export_packed_layer(hipdec_model *m, size_t layer_idx, void *wqkv, void *wo, void *w13, void *w2, void *s_qkv,
                               void *s_wo, void *s_w13, void *s_w2, float *gamma1, float *gamma2);
int hipdec_export_packed_head(hipdec_model *m, float *gamma_final, void *embed);
/* As hipdec_create, from stored weights in the format opts->weight_dtype names. */
int hipdec_create_packed(const hipdec_config *cfg, const hipdec_packed_layer *layers, size_t n_layers,
                         const hipdec_packed_head *head, const hipdec_options *opts, hipdec_model **out);

/* The full-vocabulary draw for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * Same draw as hipdec_debug_sample_fullvocab (block from the statistics, then the token inside the
 * block; engine/src/inference.rs:851-921 on the device), but every buffer is DEVICE memory of the
 * current device -- d_logits[vocab] raw logits, d_maxes/d_sums[ceil(vocab / 256)], *d_rng_state in and
 * out, *d_out_token out -- and the two kernels are enqueued on `stream` (a hipStream_t, NULL = the
 * default stream) without waiting for them.  Calls no hipMalloc / hipFree: the kernels' run state lives
 * in a 256-byte array the library holds on every GPU it runs on, reset by the call itself.  Every call
 * on a GPU shares that array, so calls that overlap on one GPU (two streams, two threads) race.
 * The library looks the array's address up once per GPU (not a capturable operation): in hipdec_create*,
 * else in the first call of this entry point on that GPU -- which must then be made outside stream capture.
 * vocab <= 262144 (1024 blocks), else HIPDEC_ERR_ARG; errors are reported through hipdec_last_error(NULL). */
int hipdec_sample_fullvocab_noalloc(const float *d_logits, size_t vocab, const float *d_maxes, const float *d_sums,
                                    float temperature, float softcap, uint64_t *d_rng_state, uint32_t *d_out_token,
                                    void *stream);
#ifdef __cplusplus
}
#endif
#endif /* HIP_DECODE_H */
