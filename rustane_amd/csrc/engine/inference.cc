#include "inference.h"

#include <math.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <limits>

namespace rustane {

namespace {
double now_s() {
    return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
// f32::total_cmp as an integer key
int32_t total_key(float f) {
    int32_t b;
    memcpy(&b, &f, 4);
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}
// Iterator::max_by(total_cmp): the LAST maximal element (inference.rs:778-783)
size_t argmax_last(const float *x, size_t n) {
    if (n == 0) return 0;
    size_t bi = 0;
    int32_t best = total_key(x[0]);
    for (size_t i = 1; i < n; ++i) {
        int32_t k = total_key(x[i]);
        if (k >= best) { best = k; bi = i; }
    }
    return bi;
}
}  // namespace

bool parse_decode_backend(const std::string &raw, DecodeBackendRequest *out) {
    if (raw == "auto") *out = DecodeBackendRequest::Auto;
    else if (raw == "naive") *out = DecodeBackendRequest::Naive;
    else if (raw == "hip") *out = DecodeBackendRequest::Hip;
    else return false;
    return true;
}
std::string decode_backend_error(const std::string &what, const std::string &raw) {
    if (raw == "metal")
        return what + " metal is the Apple-GPU backend, which this build does not have: use hip for the KV-cache path on the AMD GPU";
    return what + " must be one of: auto, naive, hip; got " + raw;
}
const char *decode_backend_str(DecodeBackendRequest r) {
    switch (r) {
        case DecodeBackendRequest::Auto: return "auto";
        case DecodeBackendRequest::Naive: return "naive";
        default: return "hip";
    }
}
const char *decode_mode_str(DecodeMode m) {
    switch (m) {
        case DecodeMode::PrefillOnly: return "prefill_only";
        case DecodeMode::NaiveFullContext: return "naive_full_context";
        default: return "kv_cache_hip";
    }
}

bool auto_prefers_kv_cache(const ModelConfig &cfg) { return cfg.param_count() >= AUTO_KV_PARAM_THRESHOLD; }

DecodeSelection select_decode_mode(const ModelConfig &cfg, DecodeBackendRequest requested, size_t ctx_len, size_t steps) {
    DecodeSelection s;
    if (steps == 0) { s.mode = DecodeMode::PrefillOnly; return s; }
    const bool window_ok = steps > 1 && ctx_len + steps <= cfg.seq;               // inference.rs:472
    switch (requested) {
        case DecodeBackendRequest::Naive:
            s.mode = DecodeMode::NaiveFullContext;
            break;
        case DecodeBackendRequest::Hip:
            if (window_ok) s.mode = DecodeMode::KvCacheHip;
            else {
                s.mode = DecodeMode::NaiveFullContext;
                s.fallback_reason = steps <= 1 ? "single_step_prefers_naive" : "requested_length_exceeds_cfg_seq";
            }
            break;
        case DecodeBackendRequest::Auto:
            if (!window_ok) {
                s.mode = DecodeMode::NaiveFullContext;
                if (ctx_len + steps > cfg.seq && steps > 1) s.fallback_reason = "requested_length_exceeds_cfg_seq";
                s.auto_reason = steps <= 1 ? "single_step_prefers_naive" : "window_not_metal_eligible";
            } else if (auto_prefers_kv_cache(cfg)) {
                s.mode = DecodeMode::KvCacheHip;
                s.auto_reason = "model_param_count_ge_threshold";
            } else {
                s.mode = DecodeMode::NaiveFullContext;
                s.auto_reason = "model_param_count_lt_threshold";
            }
            break;
    }
    return s;
}

uint64_t next_u64(uint64_t *state) {
    *state = *state * 6364136223846793005ull + 1442695040888963407ull;
    return *state;
}
float next_f32(uint64_t *state) { return (float)(next_u64(state) >> 40) / (float)(1ull << 24); }

size_t sample_softmax_index(const float *logits, size_t n, float temperature, uint64_t *rng) {
    float mx = -std::numeric_limits<float>::infinity();
    for (size_t i = 0; i < n; ++i) mx = fmaxf(mx, logits[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) sum += expf((logits[i] - mx) / temperature);
    if (!std::isfinite(sum) || sum <= 0.0f) return argmax_last(logits, n);
    float draw = next_f32(rng) * sum;
    for (size_t i = 0; i < n; ++i) {
        draw -= expf((logits[i] - mx) / temperature);
        if (draw <= 0.0f) return i;
    }
    return n ? n - 1 : 0;
}

uint32_t sample_next(const float *logits, size_t n, float temperature, size_t top_k, uint64_t *rng,
                     std::vector<size_t> *scratch) {
    if (temperature <= 0.0f || top_k == 1) return (uint32_t)argmax_last(logits, n);
    if (top_k == 0 || top_k >= n) return (uint32_t)sample_softmax_index(logits, n, temperature, rng);
    std::vector<size_t> local;
    std::vector<size_t> &ix = scratch ? *scratch : local;
    ix.resize(n);
    for (size_t i = 0; i < n; ++i) ix[i] = i;
    // descending by total_cmp; the reference's sort is unstable, equal values are ordered by index here.
    // Only the first top_k places survive the truncate (inference.rs:795-797), so only they are sorted.
    std::partial_sort(ix.begin(), ix.begin() + (ptrdiff_t)top_k, ix.end(), [&](size_t a, size_t b) {
        int32_t ka = total_key(logits[a]), kb = total_key(logits[b]);
        return ka != kb ? ka > kb : a < b;
    });
    ix.resize(top_k);
    float mx = -std::numeric_limits<float>::infinity();
    for (size_t i : ix) mx = fmaxf(mx, logits[i]);
    float sum = 0.0f;
    for (size_t i : ix) sum += expf((logits[i] - mx) / temperature);
    if (!std::isfinite(sum) || sum <= 0.0f) return (uint32_t)ix[0];
    float draw = next_f32(rng) * sum;
    for (size_t i : ix) {
        draw -= expf((logits[i] - mx) / temperature);
        if (draw <= 0.0f) return (uint32_t)i;
    }
    return (uint32_t)ix.back();
}

uint32_t sample_topk_candidates(const uint32_t *idxs, const float *logits, size_t n, float temperature, uint64_t *rng) {
    if (n == 0) return 0;
    if (temperature <= 0.0f || n == 1) return idxs[0];
    float mx = -std::numeric_limits<float>::infinity();
    for (size_t i = 0; i < n; ++i) mx = fmaxf(mx, logits[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) sum += expf((logits[i] - mx) / temperature);
    if (!std::isfinite(sum) || sum <= 0.0f) return idxs[0];
    float draw = next_f32(rng) * sum;
    for (size_t i = 0; i < n; ++i) {
        draw -= expf((logits[i] - mx) / temperature);
        if (draw <= 0.0f) return idxs[i];
    }
    return idxs[n - 1];
}

size_t sample_block_from_stats(const float *maxes, const float *sums, size_t n, uint64_t *rng) {
    if (n == 0) return 0;
    float g = -std::numeric_limits<float>::infinity();
    for (size_t b = 0; b < n; ++b)
        if (std::isfinite(maxes[b])) g = fmaxf(g, maxes[b]);
    if (!std::isfinite(g)) return 0;
    auto weight = [&](size_t b) {
        return (std::isfinite(maxes[b]) && std::isfinite(sums[b]) && sums[b] > 0.0f) ? expf(maxes[b] - g) * sums[b] : 0.0f;
    };
    float total = 0.0f;
    for (size_t b = 0; b < n; ++b) total += weight(b);
    if (!std::isfinite(total) || total <= 0.0f) return 0;
    float draw = next_f32(rng) * total;
    for (size_t b = 0; b < n; ++b) {
        draw -= weight(b);
        if (draw <= 0.0f) return b;
    }
    return n - 1;
}

uint32_t sample_block_logits(uint32_t base, const float *logits, size_t n, float temperature, uint64_t *rng) {
    return base + (uint32_t)sample_softmax_index(logits, n, temperature, rng);
}

std::string validate_token_ids(const uint32_t *ids, size_t n, size_t vocab, const char *source) {
    for (size_t pos = 0; pos < n; ++pos)
        if (ids[pos] >= vocab)
            return std::string(source) + " token id " + std::to_string(ids[pos]) + " at position " + std::to_string(pos) +
                   " exceeds model vocab " + std::to_string(vocab);
    return std::string();
}

size_t fill_input_window(const std::vector<uint32_t> &generated, size_t seq, std::vector<uint32_t> *input) {
    input->assign(seq, 0);
    const size_t start = generated.size() > seq ? generated.size() - seq : 0;
    const size_t cnt = generated.size() - start;
    std::copy(generated.begin() + start, generated.end(), input->begin());
    return cnt;
}

// ------------------------------------------------------------------ session

InferenceSession::InferenceSession(const ModelConfig &cfg, const ModelWeights &weights,
                                   const std::vector<uint32_t> &prompt_ids, float softcap, const SessionOptions &opts,
                                   std::string *err, InferenceSession *share_weights_with)
    : cfg_(cfg), prompt_ids_(prompt_ids), softcap_(softcap), device_sampling_(opts.device_sampling),
      batch_samples_(opts.batch_samples) {
    err->clear();
    if (prompt_ids.empty()) { *err = "prompt must contain at least one token"; return; }           // inference.rs:131-133
    *err = validate_token_ids(prompt_ids.data(), prompt_ids.size(), cfg.vocab, "prompt");
    if (!err->empty()) return;
    try {
        if (share_weights_with && share_weights_with->ctx_)
            ctx_.reset(new DecodeContext(cfg, *share_weights_with->ctx_, opts.kv_dtype, opts.flags));
        else
            ctx_.reset(new DecodeContext(cfg, weights, opts.weight_dtype, opts.kv_dtype, opts.device, opts.flags));
        prompt_len_ = fill_input_window(prompt_ids, cfg.seq, &input_);
        const double t0 = now_s();
        prompt_logits_ = ctx_->prefill(input_.data(), prompt_len_, softcap);                         // :139-144
        prefill_elapsed_ = now_s() - t0;
        prompt_cache_valid_ = true;
    } catch (const std::exception &e) {
        *err = e.what();
        ctx_.reset();
    }
}

std::vector<float> InferenceSession::window_logits(const std::vector<uint32_t> &ids) {
    const size_t n = fill_input_window(ids, cfg_.seq, &input_);
    ctx_->set_len(0);
    prompt_cache_valid_ = false;
    return ctx_->prefill(input_.data(), n, softcap_);
}

void InferenceSession::restore_prompt_cache() {
    if (!prompt_cache_valid_) {
        fill_input_window(prompt_ids_, cfg_.seq, &input_);
        ctx_->set_len(0);
        ctx_->prefill(input_.data(), prompt_len_, softcap_);
        prompt_cache_valid_ = true;
    }
    ctx_->set_len(prompt_len_);       // the role of seed_from_forward_caches, inference.rs:561
}

bool InferenceSession::generate(const GenerationRequest &req, GenerationBatch *out, std::string *err) {
    return generate_with_suffix(req, {}, out, err);
}

bool InferenceSession::generate_with_suffix(const GenerationRequest &req, const std::vector<uint32_t> &suffix,
                                            GenerationBatch *out, std::string *err) {
    if (req.samples == 0) { *err = "samples must be >= 1"; return false; }                         // :188-190
    return run_request(req, suffix, nullptr, out, err);
}

bool InferenceSession::generate_stream_with_suffix(const GenerationRequest &req, const std::vector<uint32_t> &suffix,
                                                   const StreamCallback &on_token, GenerationBatch *out,
                                                   std::string *err) {
    if (req.samples != 1) { *err = "streaming only supports samples=1"; return false; }             // :330-332
    return run_request(req, suffix, &on_token, out, err);
}

bool InferenceSession::run_request(const GenerationRequest &req, const std::vector<uint32_t> &suffix,
                                   const StreamCallback *cb, GenerationBatch *out, std::string *err) {
    err->clear();
    if (!ctx_) { *err = "session was not initialised"; return false; }
    *err = validate_token_ids(suffix.data(), suffix.size(), cfg_.vocab, "prompt suffix");
    if (!err->empty()) return false;
    try {
        const size_t eff_len = std::min(prompt_len_ + suffix.size(), cfg_.seq);
        const DecodeSelection sel = select_decode_mode(cfg_, req.decode_backend, eff_len, req.steps);
        const bool use_kv = sel.mode == DecodeMode::KvCacheHip;
        std::vector<uint32_t> eff_ids = prompt_ids_;
        eff_ids.insert(eff_ids.end(), suffix.begin(), suffix.end());
        double request_prefill = 0.0;
        std::vector<float> prompt_logits;
        if (suffix.empty()) {
            prompt_logits = prompt_logits_;
        } else if (use_kv) {                                   // prefill_prompt_suffix_cached, :650-670
            const double t0 = now_s();
            restore_prompt_cache();
            for (uint32_t tok : suffix) prompt_logits = ctx_->decode_next_logits(tok, softcap_);
            request_prefill = now_s() - t0;
        } else {                                               // prefill_prompt_suffix_naive, :672-685
            const double t0 = now_s();
            prompt_logits = window_logits(eff_ids);
            request_prefill = now_s() - t0;
        }
        out->results.clear();
        bool batched = false;
        if (use_kv && !cb && req.samples > 1 && req.steps > 1 && batch_samples_) {
            if (!run_cached_batch(eff_ids, prompt_logits, suffix, req, &out->results, &batched, err)) return false;
        }
        for (size_t i = 0; !batched && i < req.samples; ++i) {
            const uint64_t seed = cb ? req.seed : req.seed + (uint64_t)i;                          // :256, :414
            SampleResult r;
            const bool ok = use_kv ? run_cached_sample(eff_ids, prompt_logits, suffix, req, seed, cb, &r, err)
                                   : run_naive_sample(eff_ids, prompt_logits, req, seed, cb, &r, err);
            if (!ok) return false;
            out->results.push_back(std::move(r));
        }
        out->decode_selection = sel;
        out->total_decode_elapsed = 0.0;
        for (const SampleResult &r : out->results) out->total_decode_elapsed += r.decode_elapsed;
        out->avg_decode_elapsed = out->total_decode_elapsed / (double)req.samples;
        out->base_prefill_elapsed = prefill_elapsed_;
        out->request_prefill_elapsed = request_prefill;
        out->prefill_elapsed = prefill_elapsed_ + request_prefill;
        out->total_elapsed = out->prefill_elapsed + out->total_decode_elapsed;
        return true;
    } catch (const std::exception &e) {
        *err = e.what();
        return false;
    }
}

bool InferenceSession::run_cached_sample(const std::vector<uint32_t> &prompt, const std::vector<float> &prompt_logits,
                                         const std::vector<uint32_t> &suffix, const GenerationRequest &req,
                                         uint64_t seed, const StreamCallback *cb, SampleResult *out, std::string *err) {
    out->seed = seed;
    out->generated = prompt;
    out->sampled.clear();
    out->sampled.reserve(req.steps);
    uint64_t rng = seed;
    auto emit = [&](uint32_t tok) -> bool {
        out->generated.push_back(tok);
        out->sampled.push_back(tok);
        if (cb) {
            std::string e = (*cb)(tok, out->sampled, out->generated);
            if (!e.empty()) { *err = e; return false; }
        }
        return true;
    };
    restore_prompt_cache();
    const double t0 = now_s();                                                     // :562
    for (uint32_t tok : suffix) ctx_->decode_next_logits(tok, softcap_);          // :563-565
    if (req.steps > 0) {
        const uint32_t first = sample_next(prompt_logits.data(), prompt_logits.size(), req.temperature, req.top_k, &rng,
                                           &sampler_scratch_);
        if (!emit(first)) return false;
        uint32_t cur = first;
        if (req.temperature <= 0.0f || req.top_k == 1) {                           // :576-585
            if (!cb && req.steps > 1) {
                // no per-token consumer: the whole greedy run stays on the device
                std::vector<uint32_t> run(req.steps - 1);
                ctx_->decode_greedy_run(cur, run.size(), run.data());
                for (uint32_t tok : run) emit(tok);
            } else {
                for (size_t i = 1; i < req.steps; ++i) {
                    cur = ctx_->decode_next_greedy_token(cur);
                    if (!emit(cur)) return false;
                }
            }
        } else if (req.top_k > 0 && req.top_k <= MAX_GPU_TOPK) {                   // :586-599
            // no per-token consumer: merge and draw on the device, the run returns all tokens at once
            std::vector<uint32_t> run(req.steps - 1);
            if (!cb && device_sampling_ && req.steps > 1 &&
                ctx_->sample_topk_run(cur, req.top_k, req.temperature, softcap_, &rng, run.size(), run.data())) {
                for (uint32_t tok : run) emit(tok);
            } else {
                for (size_t i = 1; i < req.steps; ++i) {
                    const uint32_t *idxs; const float *lg; size_t n;
                    ctx_->decode_next_topk_candidates(cur, req.top_k, softcap_, &idxs, &lg, &n);
                    cur = sample_topk_candidates(idxs, lg, n, req.temperature, &rng);
                    if (!emit(cur)) return false;
                }
            }
        } else if (req.top_k == 0) {                                               // :600-625
            std::vector<uint32_t> run(req.steps - 1);
            if (!cb && device_sampling_ && req.steps > 1 &&
                ctx_->sample_fullvocab_run(cur, req.temperature, softcap_, &rng, run.size(), run.data())) {
                for (uint32_t tok : run) emit(tok);
            } else {
                for (size_t i = 1; i < req.steps; ++i) {
                    const float *mx, *sm; size_t nb;
                    ctx_->decode_next_fullvocab_block_stats(cur, req.temperature, softcap_, &mx, &sm, &nb);
                    const size_t blk = sample_block_from_stats(mx, sm, nb, &rng);
                    const float *bl; size_t nv;
                    ctx_->materialize_current_logits_block(blk, softcap_, &bl, &nv);
                    cur = sample_block_logits((uint32_t)(blk * 256), bl, nv, req.temperature, &rng);   // :613
                    if (!emit(cur)) return false;
                }
            }
        } else {                                                                   // :626-638
            for (size_t i = 1; i < req.steps; ++i) {
                const std::vector<float> &lg = ctx_->decode_next_logits(cur, softcap_);
                cur = sample_next(lg.data(), lg.size(), req.temperature, req.top_k, &rng, &sampler_scratch_);
                if (!emit(cur)) return false;
            }
        }
    }
    out->decode_elapsed = now_s() - t0;
    return true;
}

// The loop of run_cached_sample for every sample of the request at once: sample i keeps its own
// RNG (seed + i, inference.rs:256) and its own token stream; one device step serves all of them.
bool InferenceSession::run_cached_batch(const std::vector<uint32_t> &prompt, const std::vector<float> &prompt_logits,
                                        const std::vector<uint32_t> &suffix, const GenerationRequest &req,
                                        std::vector<SampleResult> *out, bool *done, std::string *err) {
    (void)err;
    *done = false;
    const size_t R = req.samples;
    if (R > 32) return true;                                                       // backend limit: fall back
    restore_prompt_cache();
    const double t0 = now_s();                                                     // :562
    for (uint32_t tok : suffix) ctx_->decode_next_logits(tok, softcap_);          // :563-565
    if (!ctx_->batch_begin(R)) return true;
    std::vector<SampleResult> res(R);
    std::vector<uint64_t> rng(R);
    std::vector<uint32_t> cur(R), nxt(R);
    for (size_t r = 0; r < R; ++r) {
        res[r].seed = req.seed + (uint64_t)r;
        res[r].generated = prompt;
        res[r].sampled.reserve(req.steps);
        rng[r] = res[r].seed;
        cur[r] = sample_next(prompt_logits.data(), prompt_logits.size(), req.temperature, req.top_k, &rng[r],
                             &sampler_scratch_);
        res[r].generated.push_back(cur[r]);
        res[r].sampled.push_back(cur[r]);
    }
    batch_device_ms_ = 0.0;
    size_t first_host_step = 1;
    if (device_sampling_ && req.steps > 1 && req.temperature > 0.0f && req.top_k != 1 && req.top_k <= MAX_GPU_TOPK) {
        // every remaining step of every row on the device (the draws of :586-625 included)
        const size_t n = req.steps - 1;
        std::vector<uint32_t> run(n * R);
        const bool ran = req.top_k > 0
            ? ctx_->sample_topk_run_batch(cur.data(), req.top_k, req.temperature, softcap_, rng.data(), n, run.data())
            : ctx_->sample_fullvocab_run_batch(cur.data(), req.temperature, softcap_, rng.data(), n, run.data());
        if (ran) {
            batch_device_ms_ += ctx_->last_device_ms();
            for (size_t i = 0; i < n; ++i)
                for (size_t r = 0; r < R; ++r) {
                    res[r].generated.push_back(run[i * R + r]);
                    res[r].sampled.push_back(run[i * R + r]);
                }
            first_host_step = req.steps;
        }
    }
    for (size_t i = first_host_step; i < req.steps; ++i) {
        if (req.temperature <= 0.0f || req.top_k == 1) {                           // :576-585
            ctx_->decode_next_greedy_tokens(cur.data(), nxt.data());
            batch_device_ms_ += ctx_->last_device_ms();
        } else if (req.top_k > 0 && req.top_k <= MAX_GPU_TOPK) {                   // :586-599
            const uint32_t *idxs; const float *lg; const size_t *n;
            ctx_->decode_next_topk_candidates_batch(cur.data(), req.top_k, softcap_, &idxs, &lg, &n);
            batch_device_ms_ += ctx_->last_device_ms();
            for (size_t r = 0; r < R; ++r)
                nxt[r] = sample_topk_candidates(idxs + r * MAX_GPU_TOPK, lg + r * MAX_GPU_TOPK, n[r], req.temperature, &rng[r]);
        } else if (req.top_k == 0) {                                               // :600-625
            const float *mx, *sm; size_t nb;
            ctx_->decode_next_fullvocab_block_stats_batch(cur.data(), req.temperature, softcap_, &mx, &sm, &nb);
            batch_device_ms_ += ctx_->last_device_ms();
            for (size_t r = 0; r < R; ++r) {
                const size_t blk = sample_block_from_stats(mx + r * nb, sm + r * nb, nb, &rng[r]);
                const float *bl; size_t nv;
                ctx_->materialize_current_logits_block_batch(r, blk, softcap_, &bl, &nv);
                nxt[r] = sample_block_logits((uint32_t)(blk * 256), bl, nv, req.temperature, &rng[r]);   // :613
            }
        } else {                                                                   // :626-638
            const float *lg = ctx_->decode_next_logits_batch(cur.data(), softcap_);
            batch_device_ms_ += ctx_->last_device_ms();
            for (size_t r = 0; r < R; ++r)
                nxt[r] = sample_next(lg + r * cfg_.vocab, cfg_.vocab, req.temperature, req.top_k, &rng[r], &sampler_scratch_);
        }
        for (size_t r = 0; r < R; ++r) {
            cur[r] = nxt[r];
            res[r].generated.push_back(cur[r]);
            res[r].sampled.push_back(cur[r]);
        }
    }
    ctx_->batch_end();
    const double elapsed = now_s() - t0;
    for (size_t r = 0; r < R; ++r) res[r].decode_elapsed = elapsed / (double)R;   // the samples shared every step
    *out = std::move(res);
    *done = true;
    return true;
}

bool InferenceSession::run_naive_sample(const std::vector<uint32_t> &prompt, const std::vector<float> &prompt_logits,
                                        const GenerationRequest &req, uint64_t seed, const StreamCallback *cb,
                                        SampleResult *out, std::string *err) {
    out->seed = seed;
    out->generated = prompt;
    out->sampled.clear();
    uint64_t rng = seed;
    auto emit = [&](uint32_t tok) -> bool {
        out->generated.push_back(tok);
        out->sampled.push_back(tok);
        if (cb) {
            std::string e = (*cb)(tok, out->sampled, out->generated);
            if (!e.empty()) { *err = e; return false; }
        }
        return true;
    };
    if (req.steps > 0) {
        const uint32_t first = sample_next(prompt_logits.data(), prompt_logits.size(), req.temperature, req.top_k, &rng,
                                           &sampler_scratch_);
        if (!emit(first)) return false;
    }
    const double t0 = now_s();                                                     // :714
    for (size_t i = 1; i < req.steps; ++i) {
        const std::vector<float> lg = window_logits(out->generated);               // :716-719
        const uint32_t next = sample_next(lg.data(), lg.size(), req.temperature, req.top_k, &rng, &sampler_scratch_);
        if (!emit(next)) return false;
    }
    out->decode_elapsed = now_s() - t0;
    return true;
}

}  // namespace rustane
