#include "session_cache.h"

#include <algorithm>

namespace rustane {

SessionCache::SessionCache(const ModelConfig &cfg, const ModelWeights &weights, float softcap, size_t max_entries,
                           const SessionOptions &opts)
    : cfg_(cfg), weights_(weights), softcap_(softcap), max_entries_(std::max<size_t>(max_entries, 1)), opts_(opts) {}

std::vector<uint32_t> SessionCache::normalize_prompt_ids(const std::vector<uint32_t> &p) const {
    if (p.size() <= cfg_.seq) return p;
    return std::vector<uint32_t>(p.end() - (ptrdiff_t)cfg_.seq, p.end());
}

long SessionCache::find_exact(const std::vector<uint32_t> &p) const {
    for (size_t i = 0; i < entries_.size(); ++i)
        if (entries_[i].window_prompt_ids == p) return (long)i;
    return -1;
}

// Iterator::max_by_key keeps the LAST of equally long matches; two entries never hold the same prompt
// (insert is only reached when find_exact failed), so lengths of matching prefixes are distinct.
long SessionCache::find_longest_prefix(const std::vector<uint32_t> &p) const {
    long best = -1;
    for (size_t i = 0; i < entries_.size(); ++i) {
        const std::vector<uint32_t> &e = entries_[i].window_prompt_ids;
        if (e.size() <= p.size() && std::equal(e.begin(), e.end(), p.begin()) &&
            (best < 0 || e.size() >= entries_[(size_t)best].window_prompt_ids.size()))
            best = (long)i;
    }
    return best;
}

void SessionCache::evict_lru() {
    if (entries_.empty()) return;
    size_t idx = 0;
    for (size_t i = 1; i < entries_.size(); ++i)
        if (entries_[i].last_used_tick < entries_[idx].last_used_tick) idx = i;     // min_by_key: the first minimum
    std::swap(entries_[idx], entries_.back());                                      // Vec::swap_remove
    entries_.pop_back();
}

long SessionCache::insert(const std::vector<uint32_t> &p, std::string *err) {
    // every entry after the first runs on the device weights of an entry that is already there
    InferenceSession *donor = entries_.empty() ? nullptr : entries_.front().session.get();
    std::unique_ptr<InferenceSession> s(new InferenceSession(cfg_, weights_, p, softcap_, opts_, err, donor));
    if (!s->ok()) return -1;
    if (entries_.size() >= max_entries_) evict_lru();
    Entry e;
    e.window_prompt_ids = p;
    e.session = std::move(s);
    e.last_used_tick = bump_tick();
    entries_.push_back(std::move(e));
    return (long)entries_.size() - 1;
}

bool SessionCache::maybe_insert(const std::vector<uint32_t> &p, std::string *err) {
    if (find_exact(p) >= 0) return true;
    return insert(p, err) >= 0;
}

bool SessionCache::run(const std::vector<uint32_t> &prompt_ids, const GenerationRequest &req, const StreamCallback *cb,
                       CacheGeneration *out, std::string *err) {
    const std::vector<uint32_t> window = normalize_prompt_ids(prompt_ids);
    out->prompt_truncated = window.size() != prompt_ids.size();
    out->effective_prompt_tokens = window.size();
    const std::vector<uint32_t> none;
    auto gen = [&](Entry &e, const std::vector<uint32_t> &suffix) {
        e.last_used_tick = bump_tick();
        return cb ? e.session->generate_stream_with_suffix(req, suffix, *cb, &out->batch, err)
                  : e.session->generate_with_suffix(req, suffix, &out->batch, err);
    };
    long idx = find_exact(window);
    if (idx >= 0) {
        if (!gen(entries_[(size_t)idx], none)) return false;
        out->cache_prefix_tokens = window.size();
        return true;
    }
    idx = find_longest_prefix(window);
    if (idx >= 0) {
        const size_t prefix_len = entries_[(size_t)idx].window_prompt_ids.size();
        const std::vector<uint32_t> suffix(window.begin() + (ptrdiff_t)prefix_len, window.end());
        if (!gen(entries_[(size_t)idx], suffix)) return false;
        if (!maybe_insert(window, err)) return false;
        out->cache_prefix_tokens = prefix_len;
        return true;
    }
    idx = insert(window, err);
    if (idx < 0) return false;
    if (!gen(entries_[(size_t)idx], none)) return false;
    out->cache_prefix_tokens = 0;
    return true;
}

bool SessionCache::generate(const std::vector<uint32_t> &prompt_ids, const GenerationRequest &req, CacheGeneration *out,
                            std::string *err) {
    return run(prompt_ids, req, nullptr, out, err);
}

bool SessionCache::stream_generate(const std::vector<uint32_t> &prompt_ids, const GenerationRequest &req,
                                   const StreamCallback &cb, CacheGeneration *out, std::string *err) {
    return run(prompt_ids, req, &cb, out, err);
}

}  // namespace rustane
