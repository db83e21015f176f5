// The session cache of the reference's server (crates/engine/src/bin/serve.rs:225-471), without the
// HTTP front end around it: a small LRU set of InferenceSessions keyed by their (window-normalised)
// prompt.  A request whose prompt is cached reuses that session; one that extends a cached prompt
// prefills only the remainder on top of the deepest matching entry (generate_with_suffix) and then
// gets an entry of its own; anything else starts a new session.  With the HIP backend the prompt of
// every entry stays in that entry's device cache, so a hit costs no prefill at all.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "inference.h"

namespace rustane {

// serve.rs:241-246
struct CacheGeneration {
    GenerationBatch batch;
    size_t effective_prompt_tokens = 0;
    bool prompt_truncated = false;
    size_t cache_prefix_tokens = 0;      // prompt tokens that were already in a cached session
};

class SessionCache {
public:
    // serve.rs:254-271 (max_entries is at least 1).  cfg and weights must outlive the cache.
    SessionCache(const ModelConfig &cfg, const ModelWeights &weights, float softcap, size_t max_entries,
                 const SessionOptions &opts);

    // serve.rs:275-328
    bool generate(const std::vector<uint32_t> &prompt_ids, const GenerationRequest &req, CacheGeneration *out, std::string *err);
    // serve.rs:330-393
    bool stream_generate(const std::vector<uint32_t> &prompt_ids, const GenerationRequest &req, const StreamCallback &cb,
                         CacheGeneration *out, std::string *err);

    // serve.rs:452-457: prompts longer than the window keep their last cfg.seq tokens
    std::vector<uint32_t> normalize_prompt_ids(const std::vector<uint32_t> &prompt_ids) const;
    // serve.rs:437-450: index of the entry with this prompt / of the longest entry that is a prefix of it, or -1
    long find_exact(const std::vector<uint32_t> &prompt_ids) const;
    long find_longest_prefix(const std::vector<uint32_t> &prompt_ids) const;
    // serve.rs:402-423: a new session for this prompt (evicting the least recently used entry when full); -1 on error
    long insert(const std::vector<uint32_t> &prompt_ids, std::string *err);

    size_t len() const { return entries_.size(); }                  // serve.rs:459-461
    size_t max_entries() const { return max_entries_; }             // serve.rs:463-465
    const std::vector<uint32_t> &entry_prompt(size_t i) const { return entries_[i].window_prompt_ids; }

private:
    struct Entry {                                                  // serve.rs:235-239
        std::vector<uint32_t> window_prompt_ids;
        std::unique_ptr<InferenceSession> session;
        uint64_t last_used_tick = 0;
    };
    bool run(const std::vector<uint32_t> &prompt_ids, const GenerationRequest &req, const StreamCallback *cb,
             CacheGeneration *out, std::string *err);
    bool maybe_insert(const std::vector<uint32_t> &prompt_ids, std::string *err);   // serve.rs:395-400
    void evict_lru();                                                               // serve.rs:425-435
    uint64_t bump_tick() { return ++tick_; }                                        // serve.rs:467-470

    const ModelConfig &cfg_;
    const ModelWeights &weights_;
    float softcap_;
    size_t max_entries_;
    SessionOptions opts_;
    uint64_t tick_ = 0;
    std::vector<Entry> entries_;
};

}  // namespace rustane
