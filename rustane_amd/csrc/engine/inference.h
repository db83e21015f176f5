// Session API for generation (crates/engine/src/inference.rs): backend selection, the naive and
// the KV-cached token loops, the CPU-side samplers and their LCG.  The `hip` backend takes the
// place the reference gives `metal`; `naive` re-runs the whole window on the GPU per token.
#pragma once
#include <stdint.h>

#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "decode_context.h"
#include "model.h"

namespace rustane {

constexpr size_t AUTO_KV_PARAM_THRESHOLD = 20000000;   // inference.rs:9 AUTO_METAL_PARAM_THRESHOLD

// inference.rs:11-35, with Hip beside Auto / Naive.  "metal" stays the name of the reference's Apple-GPU
// backend: this build has none, so parse() refuses it and decode_backend_error() says so by name
// instead of treating it as another spelling of "hip".
enum class DecodeBackendRequest { Auto, Naive, Hip };
bool parse_decode_backend(const std::string &raw, DecodeBackendRequest *out);
// The message for a value parse_decode_backend() refused; `what` names the flag or field.
std::string decode_backend_error(const std::string &what, const std::string &raw);
const char *decode_backend_str(DecodeBackendRequest r);

// inference.rs:37-52
enum class DecodeMode { PrefillOnly, NaiveFullContext, KvCacheHip };
const char *decode_mode_str(DecodeMode m);

// inference.rs:54-59
struct DecodeSelection {
    DecodeMode mode = DecodeMode::PrefillOnly;
    const char *fallback_reason = nullptr;
    const char *auto_reason = nullptr;
};

// inference.rs:61-82
struct GenerationRequest {
    DecodeBackendRequest decode_backend = DecodeBackendRequest::Auto;
    size_t steps = 32;
    float temperature = 0.0f;
    size_t top_k = 0;
    size_t samples = 1;
    uint64_t seed = 1;
};

// inference.rs:84-90 (durations in seconds)
struct SampleResult {
    uint64_t seed = 0;
    std::vector<uint32_t> generated, sampled;
    double decode_elapsed = 0.0;
};

// inference.rs:92-103
struct GenerationBatch {
    DecodeSelection decode_selection;
    double base_prefill_elapsed = 0.0, request_prefill_elapsed = 0.0, prefill_elapsed = 0.0;
    double total_decode_elapsed = 0.0, avg_decode_elapsed = 0.0, total_elapsed = 0.0;
    std::vector<SampleResult> results;
};

// inference.rs:105: (token, sampled so far, whole sequence) -> empty string to continue, else the error
using StreamCallback = std::function<std::string(uint32_t, const std::vector<uint32_t> &, const std::vector<uint32_t> &)>;

bool auto_prefers_kv_cache(const ModelConfig &cfg);                                     // inference.rs:454-456
DecodeSelection select_decode_mode(const ModelConfig &cfg, DecodeBackendRequest requested,
                                   size_t effective_context_len, size_t steps);         // inference.rs:458-528

// RNG and samplers, inference.rs:759-921
uint64_t next_u64(uint64_t *state);
float next_f32(uint64_t *state);
uint32_t sample_next(const float *logits, size_t n, float temperature, size_t top_k, uint64_t *rng,
                     std::vector<size_t> *scratch);
uint32_t sample_topk_candidates(const uint32_t *idxs, const float *logits, size_t n, float temperature, uint64_t *rng);
size_t sample_block_from_stats(const float *maxes, const float *sums, size_t n, uint64_t *rng);
size_t sample_softmax_index(const float *logits, size_t n, float temperature, uint64_t *rng);
uint32_t sample_block_logits(uint32_t base, const float *logits, size_t n, float temperature, uint64_t *rng);
// inference.rs:736-757
std::string validate_token_ids(const uint32_t *ids, size_t n, size_t vocab, const char *source);
size_t fill_input_window(const std::vector<uint32_t> &generated, size_t seq, std::vector<uint32_t> *input);

struct SessionOptions {
    WeightDtype weight_dtype = WeightDtype::F32;
    KvDtype kv_dtype = KvDtype::F32;
    int device = 0;
    uint32_t flags = 0;
    // samples > 1 on the KV-cache path advance together, one weight pass per step for all of them
    // (the reference runs them one after the other, inference.rs:247-262; results per sample are
    // the same).  false restores the sequential loop.
    bool batch_samples = true;
    // sampled requests without a per-token consumer draw their tokens on the device and run without a
    // host round trip per token; false restores the reference's loop (candidates or block statistics
    // read back and drawn on the host each step, inference.rs:586-625).  Tokens are the same.
    bool device_sampling = true;
};

// inference.rs:107-452.  Errors the reference returns as Err(String) come back through `err`
// (empty on success); construction failure leaves ok() false.
class InferenceSession {
public:
    // share_weights_with: a live session of the same model whose device weights this one uses instead of
    // uploading its own (the session cache keeps several prompts resident on one copy of the weights)
    InferenceSession(const ModelConfig &cfg, const ModelWeights &weights, const std::vector<uint32_t> &prompt_ids,
                     float softcap, const SessionOptions &opts, std::string *err,
                     InferenceSession *share_weights_with = nullptr);
    bool ok() const { return ctx_ != nullptr; }
    const std::vector<uint32_t> &prompt_ids() const { return prompt_ids_; }
    size_t prompt_len() const { return prompt_len_; }
    double prefill_elapsed() const { return prefill_elapsed_; }
    float softcap() const { return softcap_; }
    const std::vector<float> &prompt_logits() const { return prompt_logits_; }
    DecodeContext *context() { return ctx_.get(); }
    // device time (HIP events) summed over the steps of the last request whose samples advanced together
    double batch_device_ms() const { return batch_device_ms_; }

    bool generate(const GenerationRequest &req, GenerationBatch *out, std::string *err);
    bool generate_with_suffix(const GenerationRequest &req, const std::vector<uint32_t> &suffix, GenerationBatch *out,
                              std::string *err);
    bool generate_stream_with_suffix(const GenerationRequest &req, const std::vector<uint32_t> &suffix,
                                     const StreamCallback &on_token, GenerationBatch *out, std::string *err);

private:
    bool run_request(const GenerationRequest &req, const std::vector<uint32_t> &suffix, const StreamCallback *cb,
                     GenerationBatch *out, std::string *err);
    bool run_cached_sample(const std::vector<uint32_t> &prompt, const std::vector<float> &prompt_logits,
                           const std::vector<uint32_t> &suffix, const GenerationRequest &req, uint64_t seed,
                           const StreamCallback *cb, SampleResult *out, std::string *err);
    bool run_naive_sample(const std::vector<uint32_t> &prompt, const std::vector<float> &prompt_logits,
                          const GenerationRequest &req, uint64_t seed, const StreamCallback *cb, SampleResult *out,
                          std::string *err);
    // all samples of a request at once; *done = false when the backend has no multi-row path
    bool run_cached_batch(const std::vector<uint32_t> &prompt, const std::vector<float> &prompt_logits,
                          const std::vector<uint32_t> &suffix, const GenerationRequest &req,
                          std::vector<SampleResult> *out, bool *done, std::string *err);
    std::vector<float> window_logits(const std::vector<uint32_t> &ids);   // naive: whole window from position 0
    void restore_prompt_cache();                                          // device KV holds the base prompt again

    ModelConfig cfg_;
    std::unique_ptr<DecodeContext> ctx_;
    std::vector<uint32_t> prompt_ids_, input_;
    size_t prompt_len_ = 0;
    float softcap_ = 0.0f;
    bool device_sampling_ = true;
    double prefill_elapsed_ = 0.0;
    std::vector<float> prompt_logits_;
    std::vector<size_t> sampler_scratch_;
    bool prompt_cache_valid_ = false;
    bool batch_samples_ = true;
    double batch_device_ms_ = 0.0;
};

}  // namespace rustane
