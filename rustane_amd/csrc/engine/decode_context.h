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
    ~DecodeContext();
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
    float last_device_ms() const;
    uint64_t bytes_per_token(size_t kv_len) const;
    hipdec_model *raw() { return m_; }

private:
    void check(int rc, const char *what) const;
    hipdec_model *m_ = nullptr;
    size_t vocab_ = 0, blocks_ = 0;
    // decode.rs:19-31 DecodeWorkspace
    std::vector<float> logits_, block_maxes_, block_sums_, block_logits_, topk_vals_, merged_vals_;
    std::vector<uint32_t> topk_idxs_, merged_idxs_;
};

}  // namespace rustane
