#include "decode_context.h"

#include <math.h>

#include <limits>
#include <stdexcept>

#include "synth.h"

namespace rustane {

ModelWeights ModelWeights::synthetic(const ModelConfig &c, uint64_t seed, float std, bool round_bf16) {
    ModelWeights w;
    auto gen = [&](uint64_t tensor, size_t n) {
        std::vector<float> v(n);
        rs_synth_normal(seed, tensor, n, std, round_bf16 ? 1 : 0, v.data());
        return v;
    };
    w.embed = gen(RS_TENSOR_EMBED, c.vocab * c.dim);
    w.gamma_final.assign(c.dim, 1.0f);
    w.layers.resize(c.nlayers);
    for (size_t l = 0; l < c.nlayers; ++l) {
        LayerWeights &L = w.layers[l];
        L.wq = gen(RS_TENSOR_LAYER(l, 0), c.dim * c.q_dim);
        L.wk = gen(RS_TENSOR_LAYER(l, 1), c.dim * c.kv_dim);
        L.wv = gen(RS_TENSOR_LAYER(l, 2), c.dim * c.kv_dim);
        L.wo = gen(RS_TENSOR_LAYER(l, 3), c.q_dim * c.dim);
        L.w1 = gen(RS_TENSOR_LAYER(l, 4), c.dim * c.hidden);
        L.w3 = gen(RS_TENSOR_LAYER(l, 5), c.dim * c.hidden);
        L.w2 = gen(RS_TENSOR_LAYER(l, 6), c.dim * c.hidden);
        L.gamma1.assign(c.dim, 1.0f);
        L.gamma2.assign(c.dim, 1.0f);
    }
    return w;
}

size_t merge_topk_candidates(const float *vals, const uint32_t *idxs, size_t count, size_t top_k, float *out_vals,
                             uint32_t *out_idxs) {
    const float ninf = -std::numeric_limits<float>::infinity();
    for (size_t i = 0; i < top_k; ++i) { out_vals[i] = ninf; out_idxs[i] = UINT32_MAX; }
    for (size_t c = 0; c < count; ++c) {
        const float val = vals[c];
        const uint32_t idx = idxs[c];
        if (idx == UINT32_MAX || !std::isfinite(val)) continue;                     // decode.rs:229-231
        size_t at = top_k;
        for (size_t s = 0; s < top_k; ++s)
            if (val > out_vals[s] || (val == out_vals[s] && idx < out_idxs[s])) { at = s; break; }   // :234
        if (at < top_k) {
            for (size_t i = top_k - 1; i > at; --i) { out_vals[i] = out_vals[i - 1]; out_idxs[i] = out_idxs[i - 1]; }
            out_vals[at] = val;
            out_idxs[at] = idx;
        }
    }
    for (size_t i = 0; i < top_k; ++i)
        if (out_idxs[i] == UINT32_MAX) return i;                                    // :249-252
    return top_k;
}

void DecodeContext::check(int rc, const char *what) const {
    if (rc != HIPDEC_OK) throw std::runtime_error(std::string(what) + ": " + hipdec_last_error(m_));
}

DecodeContext::DecodeContext(const ModelConfig &cfg, const ModelWeights &weights, WeightDtype wdt, KvDtype kvdt,
                             int device, uint32_t flags) {
    hipdec_config c{};
    c.dim = (uint32_t)cfg.dim; c.hidden = (uint32_t)cfg.hidden; c.heads = (uint32_t)cfg.heads;
    c.kv_heads = (uint32_t)cfg.kv_heads; c.hd = (uint32_t)cfg.hd; c.seq = (uint32_t)cfg.seq;
    c.nlayers = (uint32_t)cfg.nlayers; c.vocab = (uint32_t)cfg.vocab; c.q_dim = (uint32_t)cfg.q_dim;
    c.kv_dim = (uint32_t)cfg.kv_dim; c.gqa_ratio = (uint32_t)cfg.gqa_ratio;
    hipdec_options o{};
    o.weight_dtype = (uint32_t)wdt; o.kv_dtype = (uint32_t)kvdt; o.device = device;
    o.ffn_activation = (uint32_t)cfg.ffn_activation; o.flags = flags;
    if (weights.packed) {
        // a checkpoint converted ahead of time: the stored bytes go to the device as they are
        const PackedWeights &p = *weights.packed;
        if (p.dtype != wdt) throw std::runtime_error("failed to initialize hip decode: the checkpoint holds converted weights of another format than the one asked for");
        std::vector<hipdec_packed_layer> pl(p.layers.size());
        for (size_t l = 0; l < pl.size(); ++l) {
            const PackedLayer &L = p.layers[l];
            pl[l] = hipdec_packed_layer{L.wqkv.data(), L.wo.data(), L.w13.data(), L.w2.data(), L.s_qkv.data(), L.s_wo.data(),
                                        L.s_w13.data(), L.s_w2.data(), L.gamma1.data(), L.gamma2.data()};
        }
        hipdec_packed_head ph{p.gamma_final.data(), p.embed.data()};
        int prc = hipdec_create_packed(&c, pl.data(), pl.size(), &ph, &o, &m_);
        if (prc != HIPDEC_OK)
            throw std::runtime_error(std::string("failed to initialize hip decode: ") + hipdec_last_error(nullptr));
        init_buffers(cfg);
        return;
    }
    std::vector<hipdec_layer_f32> layers(weights.layers.size());
    for (size_t l = 0; l < layers.size(); ++l) {
        const LayerWeights &L = weights.layers[l];
        layers[l] = hipdec_layer_f32{L.wq.data(), L.wk.data(), L.wv.data(), L.wo.data(), L.w1.data(),
                                     L.w3.data(), L.w2.data(), L.gamma1.data(), L.gamma2.data()};
    }
    hipdec_head_f32 head{weights.gamma_final.data(), weights.embed.data()};
    int rc = hipdec_create(&c, layers.data(), layers.size(), &head, &o, &m_);
    if (rc != HIPDEC_OK)
        throw std::runtime_error(std::string("failed to initialize hip decode: ") + hipdec_last_error(nullptr));
    init_buffers(cfg);
}

DecodeContext::DecodeContext(const ModelConfig &cfg, const DecodeContext &weights_of, KvDtype kvdt, uint32_t flags) {
    int rc = hipdec_create_shared(weights_of.m_, (uint32_t)kvdt, flags, &m_);
    if (rc != HIPDEC_OK)
        throw std::runtime_error(std::string("failed to initialize hip decode: ") + hipdec_last_error(nullptr));
    init_buffers(cfg);
}

void DecodeContext::export_packed(const ModelConfig &cfg, WeightDtype wdt, PackedWeights *out) const {
    hipdec_config c{};
    c.dim = (uint32_t)cfg.dim; c.hidden = (uint32_t)cfg.hidden; c.heads = (uint32_t)cfg.heads;
    c.kv_heads = (uint32_t)cfg.kv_heads; c.hd = (uint32_t)cfg.hd; c.seq = (uint32_t)cfg.seq;
    c.nlayers = (uint32_t)cfg.nlayers; c.vocab = (uint32_t)cfg.vocab; c.q_dim = (uint32_t)cfg.q_dim;
    c.kv_dim = (uint32_t)cfg.kv_dim; c.gqa_ratio = (uint32_t)cfg.gqa_ratio;
    hipdec_packed_sizes z;
    check(hipdec_packed_sizes_of(&c, (uint32_t)wdt, &z), "packed sizes");
    out->dtype = wdt;
    out->layers.resize(cfg.nlayers);
    for (size_t l = 0; l < cfg.nlayers; ++l) {
        PackedLayer &L = out->layers[l];
        L.wqkv.resize(z.wqkv); L.wo.resize(z.wo); L.w13.resize(z.w13); L.w2.resize(z.w2);
        L.s_qkv.resize(z.s_qkv); L.s_wo.resize(z.s_wo); L.s_w13.resize(z.s_w13); L.s_w2.resize(z.s_w2);
        L.gamma1.resize(z.gamma / 4); L.gamma2.resize(z.gamma / 4);
        check(hipdec_export_packed_layer(m_, l, L.wqkv.data(), L.wo.data(), L.w13.data(), L.w2.data(), L.s_qkv.data(),
                                         L.s_wo.data(), L.s_w13.data(), L.s_w2.data(), L.gamma1.data(), L.gamma2.data()),
              "export layer");
    }
    out->gamma_final.resize(z.gamma / 4);
    out->embed.resize(z.embed);
    check(hipdec_export_packed_head(m_, out->gamma_final.data(), out->embed.data()), "export head");
}

void DecodeContext::init_buffers(const ModelConfig &cfg) {
    vocab_ = cfg.vocab;
    blocks_ = (cfg.vocab + HIPDEC_HEAD_BLOCK - 1) / HIPDEC_HEAD_BLOCK;
    // decode.rs:200-216
    logits_.assign(cfg.vocab, 0.0f);
    block_maxes_.assign(blocks_, 0.0f);
    block_sums_.assign(blocks_, 0.0f);
    block_logits_.assign(HIPDEC_HEAD_BLOCK, 0.0f);
    topk_vals_.assign(blocks_ * MAX_GPU_TOPK, 0.0f);
    topk_idxs_.assign(blocks_ * MAX_GPU_TOPK, UINT32_MAX);
    merged_vals_.assign(MAX_GPU_TOPK, -std::numeric_limits<float>::infinity());
    merged_idxs_.assign(MAX_GPU_TOPK, UINT32_MAX);
}

DecodeContext::~DecodeContext() { hipdec_destroy(m_); }

size_t DecodeContext::len() const { return hipdec_len(m_); }
void DecodeContext::set_len(size_t len) { check(hipdec_set_len(m_, len), "set_len"); }

void DecodeContext::seed_from_forward_caches(const ModelConfig &cfg, const ForwardCaches &caches, size_t live_len) {
    if (live_len > cfg.seq) live_len = cfg.seq;
    set_len(live_len);
    for (size_t l = 0; l < caches.k_rope.size(); ++l)
        check(hipdec_seed_layer_cache_from_channel_first(m_, l, live_len, caches.k_rope[l].data(), caches.v[l].data()),
              "seed_layer_cache_from_channel_first");
}

const std::vector<float> &DecodeContext::decode_next_logits(uint32_t token, float softcap) {
    check(hipdec_decode_logits_from_id(m_, token, softcap, logits_.data()), "decode_next_logits");
    return logits_;
}

uint32_t DecodeContext::decode_next_greedy_token(uint32_t token) {
    uint32_t out = 0;
    check(hipdec_decode_token_argmax_from_id(m_, token, &out), "decode_next_greedy_token");
    return out;
}

void DecodeContext::decode_next_topk_candidates(uint32_t token, size_t top_k, float softcap, const uint32_t **idxs,
                                                const float **logits, size_t *n) {
    if (top_k > MAX_GPU_TOPK) top_k = MAX_GPU_TOPK;            // decode.rs:140
    if (top_k > vocab_) top_k = vocab_;
    size_t count = 0;
    check(hipdec_decode_token_topk_from_id(m_, token, (uint32_t)top_k, topk_vals_.data(), topk_idxs_.data(),
                                           topk_vals_.size(), &count),
          "decode_next_topk_candidates");
    size_t merged = merge_topk_candidates(topk_vals_.data(), topk_idxs_.data(), count, top_k, merged_vals_.data(),
                                          merged_idxs_.data());
    if (softcap > 0.0f)                                        // decode.rs:155-159
        for (size_t i = 0; i < merged; ++i) merged_vals_[i] = softcap * tanhf(merged_vals_[i] / softcap);
    *idxs = merged_idxs_.data();
    *logits = merged_vals_.data();
    *n = merged;
}

void DecodeContext::decode_next_fullvocab_block_stats(uint32_t token, float temperature, float softcap,
                                                      const float **maxes, const float **sums, size_t *n) {
    const float t = temperature > std::numeric_limits<float>::min() ? temperature : std::numeric_limits<float>::min();
    const float inv_temperature = 1.0f / t;                    // decode.rs:174
    size_t count = 0;
    check(hipdec_decode_token_block_stats_from_id(m_, token, inv_temperature, softcap, block_maxes_.data(),
                                                  block_sums_.data(), block_maxes_.size(), &count),
          "decode_next_fullvocab_block_stats");
    *maxes = block_maxes_.data();
    *sums = block_sums_.data();
    *n = count;
}

void DecodeContext::materialize_current_logits_block(size_t block_idx, float softcap, const float **logits, size_t *n) {
    size_t valid = 0;
    check(hipdec_materialize_current_logits_block(m_, block_idx, softcap, block_logits_.data(), block_logits_.size(),
                                                  &valid),
          "materialize_current_logits_block");
    *logits = block_logits_.data();
    *n = valid;
}

const std::vector<float> &DecodeContext::prefill(const uint32_t *ids, size_t n, float softcap) {
    check(hipdec_prefill(m_, ids, n, softcap, logits_.data()), "prefill");
    return logits_;
}

void DecodeContext::decode_greedy_run(uint32_t token, size_t n_steps, uint32_t *out) {
    check(hipdec_decode_greedy_run(m_, token, n_steps, out), "decode_greedy_run");
}

bool DecodeContext::sample_topk_run(uint32_t token, size_t top_k, float temperature, float softcap, uint64_t *rng,
                                    size_t n_steps, uint32_t *out) {
    if (top_k > MAX_GPU_TOPK) top_k = MAX_GPU_TOPK;            // decode.rs:140
    if (top_k > vocab_) top_k = vocab_;
    const int rc = hipdec_decode_topk_sampled_run(m_, token, (uint32_t)top_k, temperature, softcap, rng, n_steps, out);
    if (rc == HIPDEC_ERR_UNSUPPORTED) return false;
    check(rc, "sample_topk_run");
    return true;
}

bool DecodeContext::sample_fullvocab_run(uint32_t token, float temperature, float softcap, uint64_t *rng, size_t n_steps,
                                         uint32_t *out) {
    const int rc = hipdec_decode_fullvocab_sampled_run(m_, token, temperature, softcap, rng, n_steps, out);
    if (rc == HIPDEC_ERR_UNSUPPORTED) return false;
    check(rc, "sample_fullvocab_run");
    return true;
}

bool DecodeContext::sample_topk_run_batch(const uint32_t *tokens, size_t top_k, float temperature, float softcap,
                                          uint64_t *rngs, size_t n_steps, uint32_t *out) {
    if (top_k > MAX_GPU_TOPK) top_k = MAX_GPU_TOPK;            // decode.rs:140
    if (top_k > vocab_) top_k = vocab_;
    const int rc = hipdec_decode_topk_sampled_run_batch(m_, tokens, (uint32_t)top_k, temperature, softcap, rngs, n_steps, out);
    if (rc == HIPDEC_ERR_UNSUPPORTED) return false;
    check(rc, "sample_topk_run_batch");
    return true;
}

bool DecodeContext::sample_fullvocab_run_batch(const uint32_t *tokens, float temperature, float softcap, uint64_t *rngs,
                                               size_t n_steps, uint32_t *out) {
    const int rc = hipdec_decode_fullvocab_sampled_run_batch(m_, tokens, temperature, softcap, rngs, n_steps, out);
    if (rc == HIPDEC_ERR_UNSUPPORTED) return false;
    check(rc, "sample_fullvocab_run_batch");
    return true;
}

bool DecodeContext::batch_begin(size_t rows) {
    const int rc = hipdec_batch_begin(m_, rows);
    if (rc == HIPDEC_ERR_UNSUPPORTED) return false;
    check(rc, "batch_begin");
    batch_rows_ = rows;
    b_vals_.assign(rows * blocks_ * MAX_GPU_TOPK, 0.0f);
    b_idxs_.assign(rows * blocks_ * MAX_GPU_TOPK, UINT32_MAX);
    b_merged_vals_.assign(rows * MAX_GPU_TOPK, 0.0f);
    b_merged_idxs_.assign(rows * MAX_GPU_TOPK, UINT32_MAX);
    b_counts_.assign(rows, 0);
    b_maxes_.assign(rows * blocks_, 0.0f);
    b_sums_.assign(rows * blocks_, 0.0f);
    return true;
}

void DecodeContext::batch_end() {
    check(hipdec_batch_end(m_), "batch_end");
    batch_rows_ = 0;
}

void DecodeContext::decode_next_greedy_tokens(const uint32_t *tokens, uint32_t *out) {
    check(hipdec_decode_token_argmax_from_ids_batch(m_, tokens, out), "decode_next_greedy_tokens");
}

void DecodeContext::decode_next_topk_candidates_batch(const uint32_t *tokens, size_t top_k, float softcap,
                                                      const uint32_t **idxs, const float **logits, const size_t **n) {
    if (top_k > MAX_GPU_TOPK) top_k = MAX_GPU_TOPK;            // decode.rs:140
    if (top_k > vocab_) top_k = vocab_;
    size_t per_row = 0;
    check(hipdec_decode_token_topk_from_ids_batch(m_, tokens, (uint32_t)top_k, b_vals_.data(), b_idxs_.data(),
                                                  b_vals_.size(), &per_row),
          "decode_next_topk_candidates_batch");
    for (size_t r = 0; r < batch_rows_; ++r) {
        float *mv = b_merged_vals_.data() + r * MAX_GPU_TOPK;
        const size_t merged = merge_topk_candidates(b_vals_.data() + r * per_row, b_idxs_.data() + r * per_row, per_row,
                                                    top_k, mv, b_merged_idxs_.data() + r * MAX_GPU_TOPK);
        if (softcap > 0.0f)                                    // decode.rs:155-159
            for (size_t i = 0; i < merged; ++i) mv[i] = softcap * tanhf(mv[i] / softcap);
        b_counts_[r] = merged;
    }
    *idxs = b_merged_idxs_.data();
    *logits = b_merged_vals_.data();
    *n = b_counts_.data();
}

void DecodeContext::decode_next_fullvocab_block_stats_batch(const uint32_t *tokens, float temperature, float softcap,
                                                            const float **maxes, const float **sums, size_t *blocks) {
    const float t = temperature > std::numeric_limits<float>::min() ? temperature : std::numeric_limits<float>::min();
    size_t count = 0;
    check(hipdec_decode_token_block_stats_from_ids_batch(m_, tokens, 1.0f / t, softcap, b_maxes_.data(), b_sums_.data(),
                                                         b_maxes_.size(), &count),
          "decode_next_fullvocab_block_stats_batch");
    *maxes = b_maxes_.data();
    *sums = b_sums_.data();
    *blocks = count;
}

void DecodeContext::materialize_current_logits_block_batch(size_t row, size_t block_idx, float softcap,
                                                           const float **logits, size_t *n) {
    size_t valid = 0;
    check(hipdec_materialize_current_logits_block_batch(m_, row, block_idx, softcap, block_logits_.data(),
                                                        block_logits_.size(), &valid),
          "materialize_current_logits_block_batch");
    *logits = block_logits_.data();
    *n = valid;
}

const float *DecodeContext::decode_next_logits_batch(const uint32_t *tokens, float softcap) {
    b_logits_.resize(batch_rows_ * vocab_);
    check(hipdec_decode_logits_from_ids_batch(m_, tokens, softcap, b_logits_.data()), "decode_next_logits_batch");
    return b_logits_.data();
}

float DecodeContext::last_device_ms() const {
    float ms = 0.0f;
    hipdec_last_device_ms(m_, &ms);
    return ms;
}

uint64_t DecodeContext::bytes_per_token(size_t kv_len) const {
    uint64_t b = 0;
    hipdec_bytes_per_token(m_, kv_len, &b);
    return b;
}

}  // namespace rustane
