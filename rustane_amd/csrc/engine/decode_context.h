// DecodeContext: the adapter between the session layer and the GPU decode backend
// (crates/engine/src/decode.rs:14-253), here over the C ABI of include/hip_decode.h instead of
// metal_decode::Model.
#pragma once
#include <stdint.h>

#include <string>
#include <vector>

#include "hip_decode.h"
#include "model.h"

namespace rustane {

constexpr size_t MAX_GPU_TOPK = HIPDEC_MAX_GPU_TOPK;   // decode.rs:12

// decode.rs:218-253: keeps the top_k best (value desc, index asc) of the per-block candidates,
// skipping exhausted slots (idx == u32::MAX) and non-finite values; returns how many are valid.
size_t merge_topk_candidates(const float *vals, const uint32_t *idxs, size_t count, size_t top_k, float *out_vals,
                             uint32_t *out_idxs);

struct ForwardCaches {     // per layer channel-first [kv_dim][seq] (layer.rs:52-67 k_rope / v)
    std::vector<std::vector<float>> k_rope, v;
};

class DecodeContext {
public:
    // decode.rs:34-71 (throws std::runtime_error where the reference `expect`s)
    DecodeContext(const ModelConfig &cfg, const ModelWeights &weights, WeightDtype wdt = WeightDtype::F32,
                  KvDtype kvdt = KvDtype::F32, int device = 0, uint32_t flags = 0);
    // a context on the device weights another context already holds (hipdec_create_shared): no upload,
    // KV caches and step state of its own; the weights live as long as any context that uses them
    DecodeContext(const ModelConfig &cfg, const DecodeContext &weights_of, KvDtype kvdt, uint32_t flags);
    ~DecodeContext();
    // the weights as this context's model stores them on the device (for a checkpoint converted ahead of time)
    void export_packed(const ModelConfig &cfg, WeightDtype wdt, PackedWeights *out) const;
    DecodeContext(const DecodeContext &) = delete;
    DecodeContext &operator=(const DecodeContext &) = delete;

    size_t len() const;
    void set_len(size_t len);
    // decode.rs:73-89
    void seed_from_forward_caches(const ModelConfig &cfg, const ForwardCaches &caches, size_t live_len);
    // decode.rs:91-127 (final norm, LM head and softcap run on the GPU here)
    const std::vector<float> &decode_next_logits(uint32_t token, float softcap);
    // decode.rs:129-131
    uint32_t decode_next_greedy_token(uint32_t token);
    // decode.rs:133-165: merged candidates, softcap applied to the survivors
    void decode_next_topk_candidates(uint32_t token, size_t top_k, float softcap, const uint32_t **idxs,
                                     const float **logits, size_t *n);
    // decode.rs:167-183
    void decode_next_fullvocab_block_stats(uint32_t token, float temperature, float softcap, const float **maxes,
                                           const float **sums, size_t *n);
    // decode.rs:185-197
    void materialize_current_logits_block(size_t block_idx, float softcap, const float **logits, size_t *n);

    // not in the reference: prompt prefill on the GPU and greedy runs without per-token host round trips
    const std::vector<float> &prefill(const uint32_t *ids, size_t n, float softcap);
    void decode_greedy_run(uint32_t token, size_t n_steps, uint32_t *out);
    // The sampled loops of inference.rs:586-625 run on the device for n_steps tokens: candidates merged
    // and drawn (top_k in 1..=MAX_GPU_TOPK), or block then token drawn from the block statistics.
    // *rng advances as the host loop would advance it.  false: the backend does not serve this
    // request on the device (nothing has run; use the per-step calls).
    bool sample_topk_run(uint32_t token, size_t top_k, float temperature, float softcap, uint64_t *rng, size_t n_steps,
                         uint32_t *out);
    bool sample_fullvocab_run(uint32_t token, float temperature, float softcap, uint64_t *rng, size_t n_steps, uint32_t *out);
    // the same for every row of an open batch; out[n_steps][rows]
    bool sample_topk_run_batch(const uint32_t *tokens, size_t top_k, float temperature, float softcap, uint64_t *rngs,
                               size_t n_steps, uint32_t *out);
    bool sample_fullvocab_run_batch(const uint32_t *tokens, float temperature, float softcap, uint64_t *rngs,
                                    size_t n_steps, uint32_t *out);
    // not in the reference: `rows` continuations of the current cache contents stepped together
    // (the reference runs its samples one after the other, inference.rs:247-262).  batch_begin
    // returns false when the backend has no multi-row path for this model.
    bool batch_begin(size_t rows);
    void batch_end();
    size_t batch_rows() const { return batch_rows_; }
    // tokens[rows] -> out[rows]
    void decode_next_greedy_tokens(const uint32_t *tokens, uint32_t *out);
    // row r's merged, softcapped candidates are at idxs + r * MAX_GPU_TOPK / logits + r * MAX_GPU_TOPK, n[r] of them
    void decode_next_topk_candidates_batch(const uint32_t *tokens, size_t top_k, float softcap, const uint32_t **idxs,
                                           const float **logits, const size_t **n);
    // row r's block statistics are at maxes + r * blocks / sums + r * blocks
    void decode_next_fullvocab_block_stats_batch(const uint32_t *tokens, float temperature, float softcap,
                                                 const float **maxes, const float **sums, size_t *blocks);
    void materialize_current_logits_block_batch(size_t row, size_t block_idx, float softcap, const float **logits,
                                                size_t *n);
    // row r's logits are at result + r * vocab
    const float *decode_next_logits_batch(const uint32_t *tokens, float softcap);
    float last_device_ms() const;
    uint64_t bytes_per_token(size_t kv_len) const;
    hipdec_model *raw() { return m_; }

private:
    void check(int rc, const char *what) const;
    void init_buffers(const ModelConfig &cfg);
    hipdec_model *m_ = nullptr;
    size_t vocab_ = 0, blocks_ = 0;
    // decode.rs:19-31 DecodeWorkspace
    std::vector<float> logits_, block_maxes_, block_sums_, block_logits_, topk_vals_, merged_vals_;
    std::vector<uint32_t> topk_idxs_, merged_idxs_;
    // multi-row workspace
    size_t batch_rows_ = 0;
    std::vector<float> b_logits_, b_vals_, b_merged_vals_, b_maxes_, b_sums_;
    std::vector<uint32_t> b_idxs_, b_merged_idxs_;
    std::vector<size_t> b_counts_;
};

}  // namespace rustane
