// Plain-C view of the host engine for ctypes (tests, benchmark).  Thin: every function forwards
// to the C++ classes of model.h / decode_context.h / inference.h.
#include <stdint.h>
#include <string.h>

#include <memory>
#include <string>
#include <vector>

#include "checkpoint.h"
#include "http_server.h"
#include "inference.h"
#include "jsonl_session.h"
#include "session_cache.h"

using namespace rustane;

extern "C" {

struct rs_config {
    uint64_t dim, hidden, heads, kv_heads, hd, seq, nlayers, vocab;
    uint32_t ffn_activation;
};
struct rs_request {
    uint32_t backend;            // 0 auto, 1 naive, 2 hip
    uint64_t steps;
    float temperature;
    uint64_t top_k, samples, seed;
};
struct rs_batch_info {
    uint32_t mode;               // 0 prefill_only, 1 naive_full_context, 2 kv_cache_hip
    const char *fallback_reason, *auto_reason;
    double base_prefill_s, request_prefill_s, prefill_s, total_decode_s, avg_decode_s, total_s;
    uint64_t n_results;
};
struct rs_weights { ModelWeights w; };
struct rs_session {
    std::unique_ptr<InferenceSession> s;
    GenerationBatch last;
    size_t stream_count = 0;
};

static ModelConfig to_cfg(const rs_config *c) {
    return ModelConfig::make(c->dim, c->hidden, c->heads, c->kv_heads, c->hd, c->seq, c->nlayers, c->vocab,
                             (FfnActivation)c->ffn_activation);
}
static void put_err(char *buf, size_t cap, const std::string &e) {
    if (buf && cap) { strncpy(buf, e.c_str(), cap - 1); buf[cap - 1] = 0; }
}

uint64_t rs_param_count(const rs_config *c) { return to_cfg(c).param_count(); }

rs_weights *rs_weights_synthetic(const rs_config *c, uint64_t seed, float std, int round_bf16) {
    rs_weights *w = new rs_weights();
    w->w = ModelWeights::synthetic(to_cfg(c), seed, std, round_bf16 != 0);
    return w;
}
// layer_ptrs: nlayers * 9 pointers in the order wq wk wv wo w1 w3 w2 gamma1 gamma2 (copied)
rs_weights *rs_weights_from_arrays(const rs_config *c, const float *const *layer_ptrs, const float *gamma_final,
                                   const float *embed) {
    ModelConfig cfg = to_cfg(c);
    rs_weights *w = new rs_weights();
    const size_t D = cfg.dim, Q = cfg.q_dim, KV = cfg.kv_dim, H = cfg.hidden;
    const size_t sizes[9] = {D * Q, D * KV, D * KV, Q * D, D * H, D * H, D * H, D, D};
    w->w.embed.assign(embed, embed + cfg.vocab * D);
    w->w.gamma_final.assign(gamma_final, gamma_final + D);
    w->w.layers.resize(cfg.nlayers);
    for (size_t l = 0; l < cfg.nlayers; ++l) {
        LayerWeights &L = w->w.layers[l];
        std::vector<float> *dst[9] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.w1, &L.w3, &L.w2, &L.gamma1, &L.gamma2};
        for (int k = 0; k < 9; ++k) dst[k]->assign(layer_ptrs[l * 9 + k], layer_ptrs[l * 9 + k] + sizes[k]);
    }
    return w;
}
void rs_weights_free(rs_weights *w) { delete w; }

// ---- RSTK checkpoints (crates/engine/src/checkpoint.rs)
static void from_cfg(const ModelConfig &c, rs_config *o) {
    o->dim = c.dim; o->hidden = c.hidden; o->heads = c.heads; o->kv_heads = c.kv_heads; o->hd = c.hd; o->seq = c.seq;
    o->nlayers = c.nlayers; o->vocab = c.vocab; o->ffn_activation = (uint32_t)c.ffn_activation;
}
static rs_weights *take_checkpoint(Checkpoint &ck, rs_config *cfg_out, uint32_t *step) {
    rs_weights *w = new rs_weights();
    w->w = std::move(ck.weights);
    if (cfg_out) from_cfg(ck.cfg, cfg_out);
    if (step) *step = ck.step;
    return w;
}
rs_weights *rs_checkpoint_parse(const uint8_t *bytes, size_t n, rs_config *cfg_out, uint32_t *step, char *err, size_t errcap) {
    Checkpoint ck;
    std::string e;
    if (!parse_checkpoint(bytes, n, &ck, &e)) { put_err(err, errcap, e); return nullptr; }
    return take_checkpoint(ck, cfg_out, step);
}
rs_weights *rs_checkpoint_load(const char *path, rs_config *cfg_out, uint32_t *step, char *err, size_t errcap) {
    Checkpoint ck;
    std::string e;
    if (!load_checkpoint(path, &ck, &e)) { put_err(err, errcap, e); return nullptr; }
    return take_checkpoint(ck, cfg_out, step);
}
// A converted checkpoint's header and size check (no device needed): 0 = ok; cfg, step and the weight format
// (0 fp32, 1 bf16, 2 e4m3, 3 4-bit) filled; 1 = rejected with the loader's message.
int rs_packed_checkpoint_parse(const uint8_t *bytes, size_t n, rs_config *cfg_out, uint32_t *step, uint32_t *dtype, char *err,
                               size_t errcap) {
    Checkpoint ck;
    std::string e;
    if (!parse_packed_checkpoint(bytes, n, &ck, &e)) { put_err(err, errcap, e); return 1; }
    from_cfg(ck.cfg, cfg_out);
    *step = ck.step;
    *dtype = (uint32_t)ck.weights.packed->dtype;
    return 0;
}
int rs_checkpoint_write(const char *path, const rs_config *c, const rs_weights *w, uint32_t step, char *err, size_t errcap) {
    std::string e;
    if (!write_checkpoint(path, to_cfg(c), w->w, step, &e)) { put_err(err, errcap, e); return 1; }
    return 0;
}
// tensor `which` of layer `layer` in the order wq wk wv wo w1 w3 w2 gamma1 gamma2; layer < 0: 0 embed, 1 gamma_final
int rs_weights_tensor(const rs_weights *w, int64_t layer, int which, const float **ptr, uint64_t *n) {
    const std::vector<float> *v = nullptr;
    if (layer < 0) v = which == 0 ? &w->w.embed : which == 1 ? &w->w.gamma_final : nullptr;
    else if ((size_t)layer < w->w.layers.size() && which >= 0 && which < 9) {
        const LayerWeights &L = w->w.layers[(size_t)layer];
        const std::vector<float> *t[9] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.w1, &L.w3, &L.w2, &L.gamma1, &L.gamma2};
        v = t[which];
    }
    if (!v) return 1;
    *ptr = v->data(); *n = v->size();
    return 0;
}

rs_session *rs_session_new(const rs_config *c, const rs_weights *w, const uint32_t *prompt, size_t n, float softcap,
                           uint32_t weight_dtype, uint32_t kv_dtype, uint32_t flags, char *err, size_t errcap) {
    SessionOptions o;
    o.weight_dtype = (WeightDtype)weight_dtype;
    o.kv_dtype = (KvDtype)kv_dtype;
    o.flags = flags & 0xffu;                  // HIPDEC_FLAG_* for the backend
    o.batch_samples = !(flags & 0x100u);      // 0x100: run the samples of a request one after the other
    o.device_sampling = !(flags & 0x200u);    // 0x200: draw every sampled token on the host, as the reference does
    std::string e;
    std::unique_ptr<rs_session> s(new rs_session());
    s->s.reset(new InferenceSession(to_cfg(c), w->w, std::vector<uint32_t>(prompt, prompt + n), softcap, o, &e));
    if (!s->s->ok()) { put_err(err, errcap, e); return nullptr; }
    return s.release();
}
void rs_session_free(rs_session *s) { delete s; }

uint64_t rs_session_prompt_len(const rs_session *s) { return s->s->prompt_len(); }
double rs_session_prefill_s(const rs_session *s) { return s->s->prefill_elapsed(); }
void rs_session_prompt_logits(const rs_session *s, float *out) {
    memcpy(out, s->s->prompt_logits().data(), s->s->prompt_logits().size() * sizeof(float));
}

// stream: 0 = generate_with_suffix; 1 = generate_stream_with_suffix whose callback returns an error
// once it has been handed `abort_after` tokens (0 = never)
int rs_session_generate(rs_session *s, const rs_request *r, const uint32_t *suffix, size_t n_suffix, int stream,
                        uint64_t abort_after, rs_batch_info *info, char *err, size_t errcap) {
    GenerationRequest req;
    req.decode_backend = r->backend == 1 ? DecodeBackendRequest::Naive
                         : r->backend == 2 ? DecodeBackendRequest::Hip : DecodeBackendRequest::Auto;
    req.steps = r->steps; req.temperature = r->temperature; req.top_k = r->top_k; req.samples = r->samples;
    req.seed = r->seed;
    std::vector<uint32_t> suf(suffix, suffix + n_suffix);
    std::string e;
    bool ok;
    s->stream_count = 0;
    if (stream) {
        StreamCallback cb = [&](uint32_t, const std::vector<uint32_t> &sampled, const std::vector<uint32_t> &) {
            s->stream_count = sampled.size();
            if (abort_after && sampled.size() >= abort_after) return std::string("callback asked to stop");
            return std::string();
        };
        ok = s->s->generate_stream_with_suffix(req, suf, cb, &s->last, &e);
    } else {
        ok = s->s->generate_with_suffix(req, suf, &s->last, &e);
    }
    if (!ok) { put_err(err, errcap, e); return 1; }
    const GenerationBatch &b = s->last;
    info->mode = (uint32_t)b.decode_selection.mode;
    info->fallback_reason = b.decode_selection.fallback_reason;
    info->auto_reason = b.decode_selection.auto_reason;
    info->base_prefill_s = b.base_prefill_elapsed; info->request_prefill_s = b.request_prefill_elapsed;
    info->prefill_s = b.prefill_elapsed; info->total_decode_s = b.total_decode_elapsed;
    info->avg_decode_s = b.avg_decode_elapsed; info->total_s = b.total_elapsed;
    info->n_results = b.results.size();
    return 0;
}
double rs_session_batch_device_ms(const rs_session *s) { return s->s->batch_device_ms(); }
uint64_t rs_session_bytes_per_token(rs_session *s, size_t kv_len) { return s->s->context()->bytes_per_token(kv_len); }
uint64_t rs_session_stream_count(const rs_session *s) { return s->stream_count; }
uint64_t rs_session_result_len(const rs_session *s, size_t i, int which) {
    const SampleResult &r = s->last.results[i];
    return which ? r.generated.size() : r.sampled.size();
}
void rs_session_result_copy(const rs_session *s, size_t i, int which, uint32_t *out) {
    const SampleResult &r = s->last.results[i];
    const std::vector<uint32_t> &v = which ? r.generated : r.sampled;
    memcpy(out, v.data(), v.size() * sizeof(uint32_t));
}
double rs_session_result_decode_s(const rs_session *s, size_t i) { return s->last.results[i].decode_elapsed; }
uint64_t rs_session_result_seed(const rs_session *s, size_t i) { return s->last.results[i].seed; }

// ---- the server's session cache (bin/serve.rs:225-471)
struct rs_session_cache {
    ModelConfig cfg;
    std::unique_ptr<SessionCache> c;
    CacheGeneration last;
};
rs_session_cache *rs_session_cache_new(const rs_config *c, const rs_weights *w, float softcap, size_t max_entries,
                                       uint32_t weight_dtype, uint32_t kv_dtype, uint32_t flags) {
    SessionOptions o;
    o.weight_dtype = (WeightDtype)weight_dtype;
    o.kv_dtype = (KvDtype)kv_dtype;
    o.flags = flags & 0xffu;
    o.batch_samples = !(flags & 0x100u);
    o.device_sampling = !(flags & 0x200u);
    rs_session_cache *sc = new rs_session_cache();
    sc->cfg = to_cfg(c);
    sc->c.reset(new SessionCache(sc->cfg, w->w, softcap, max_entries, o));     // w must outlive the cache
    return sc;
}
void rs_session_cache_free(rs_session_cache *sc) { delete sc; }
uint64_t rs_session_cache_len(const rs_session_cache *sc) { return sc->c->len(); }
uint64_t rs_session_cache_max_entries(const rs_session_cache *sc) { return sc->c->max_entries(); }
uint64_t rs_session_cache_entry_prompt(const rs_session_cache *sc, size_t i, uint32_t *out, size_t cap) {
    const std::vector<uint32_t> &p = sc->c->entry_prompt(i);
    if (out && cap >= p.size()) memcpy(out, p.data(), p.size() * sizeof(uint32_t));
    return p.size();
}
uint64_t rs_session_cache_normalize(const rs_session_cache *sc, const uint32_t *prompt, size_t n, uint32_t *out, size_t cap) {
    const std::vector<uint32_t> p = sc->c->normalize_prompt_ids(std::vector<uint32_t>(prompt, prompt + n));
    if (out && cap >= p.size()) memcpy(out, p.data(), p.size() * sizeof(uint32_t));
    return p.size();
}
int64_t rs_session_cache_find(const rs_session_cache *sc, const uint32_t *prompt, size_t n, int longest_prefix) {
    const std::vector<uint32_t> p(prompt, prompt + n);
    return longest_prefix ? sc->c->find_longest_prefix(p) : sc->c->find_exact(p);
}
int64_t rs_session_cache_insert(rs_session_cache *sc, const uint32_t *prompt, size_t n, char *err, size_t errcap) {
    std::string e;
    const long idx = sc->c->insert(std::vector<uint32_t>(prompt, prompt + n), &e);
    if (idx < 0) put_err(err, errcap, e);
    return idx;
}
// cache_info: effective prompt tokens, prompt truncated (0/1), prompt tokens found in a cached session
int rs_session_cache_generate(rs_session_cache *sc, const uint32_t *prompt, size_t n, const rs_request *r, int stream,
                              uint64_t abort_after, rs_batch_info *info, uint64_t *cache_info, char *err, size_t errcap) {
    GenerationRequest req;
    req.decode_backend = r->backend == 1 ? DecodeBackendRequest::Naive
                         : r->backend == 2 ? DecodeBackendRequest::Hip : DecodeBackendRequest::Auto;
    req.steps = r->steps; req.temperature = r->temperature; req.top_k = r->top_k; req.samples = r->samples;
    req.seed = r->seed;
    const std::vector<uint32_t> p(prompt, prompt + n);
    std::string e;
    bool ok;
    if (stream) {
        StreamCallback cb = [&](uint32_t, const std::vector<uint32_t> &sampled, const std::vector<uint32_t> &) {
            if (abort_after && sampled.size() >= abort_after) return std::string("callback asked to stop");
            return std::string();
        };
        ok = sc->c->stream_generate(p, req, cb, &sc->last, &e);
    } else {
        ok = sc->c->generate(p, req, &sc->last, &e);
    }
    if (!ok) { put_err(err, errcap, e); return 1; }
    const GenerationBatch &b = sc->last.batch;
    info->mode = (uint32_t)b.decode_selection.mode;
    info->fallback_reason = b.decode_selection.fallback_reason;
    info->auto_reason = b.decode_selection.auto_reason;
    info->base_prefill_s = b.base_prefill_elapsed; info->request_prefill_s = b.request_prefill_elapsed;
    info->prefill_s = b.prefill_elapsed; info->total_decode_s = b.total_decode_elapsed;
    info->avg_decode_s = b.avg_decode_elapsed; info->total_s = b.total_elapsed;
    info->n_results = b.results.size();
    cache_info[0] = sc->last.effective_prompt_tokens;
    cache_info[1] = sc->last.prompt_truncated ? 1 : 0;
    cache_info[2] = sc->last.cache_prefix_tokens;
    return 0;
}
uint64_t rs_session_cache_result_len(const rs_session_cache *sc, size_t i, int which) {
    const SampleResult &r = sc->last.batch.results[i];
    return which ? r.generated.size() : r.sampled.size();
}
void rs_session_cache_result_copy(const rs_session_cache *sc, size_t i, int which, uint32_t *out) {
    const SampleResult &r = sc->last.batch.results[i];
    const std::vector<uint32_t> &v = which ? r.generated : r.sampled;
    memcpy(out, v.data(), v.size() * sizeof(uint32_t));
}
uint64_t rs_session_cache_result_seed(const rs_session_cache *sc, size_t i) { return sc->last.batch.results[i].seed; }

void rs_select_decode_mode(const rs_config *c, uint32_t requested, uint64_t ctx_len, uint64_t steps, uint32_t *mode,
                           const char **fallback_reason, const char **auto_reason) {
    DecodeBackendRequest rq = requested == 1 ? DecodeBackendRequest::Naive
                              : requested == 2 ? DecodeBackendRequest::Hip : DecodeBackendRequest::Auto;
    DecodeSelection s = select_decode_mode(to_cfg(c), rq, ctx_len, steps);
    *mode = (uint32_t)s.mode;
    *fallback_reason = s.fallback_reason;
    *auto_reason = s.auto_reason;
}
int rs_parse_decode_backend(const char *raw, uint32_t *out) {
    DecodeBackendRequest r;
    if (!parse_decode_backend(raw, &r)) return 0;
    *out = r == DecodeBackendRequest::Naive ? 1 : r == DecodeBackendRequest::Hip ? 2 : 0;
    return 1;
}

// ---- one request line of the JSONL session protocol (bin/generate.rs:39-144), without running it:
// 0 = ok (request and suffix filled), 1 = rejected (err holds the message the session would answer with)
int rs_jsonl_parse(const char *line, const rs_request *defaults, rs_request *out, uint32_t *suffix, size_t cap,
                   uint64_t *n_suffix, char *err, size_t errcap) {
    GenerationRequest d, req;
    d.decode_backend = (DecodeBackendRequest)defaults->backend; d.steps = defaults->steps; d.temperature = defaults->temperature;
    d.top_k = defaults->top_k; d.samples = defaults->samples; d.seed = defaults->seed;
    JsonlRequest parsed;
    std::vector<uint32_t> sfx;
    std::string e;
    if (!parse_jsonl_request(line, &parsed, &e) || !jsonl_to_generation_request(parsed, d, &req, &e) ||
        !jsonl_prompt_suffix(parsed, &sfx, &e)) {
        put_err(err, errcap, e);
        return 1;
    }
    out->backend = (uint32_t)req.decode_backend; out->steps = req.steps; out->temperature = req.temperature;
    out->top_k = req.top_k; out->samples = req.samples; out->seed = req.seed;
    *n_suffix = sfx.size();
    for (size_t i = 0; i < sfx.size() && i < cap; ++i) suffix[i] = sfx[i];
    return 0;
}

// ---- the HTTP front end (bin/serve.rs) without a model behind it
// Reads one request from a connected socket.  0 = ok, 1 = refused (err holds the message of the 400 answer).
int rs_http_parse_request(int fd, uint64_t max_body, char *method, size_t mcap, char *path, size_t pcap, char *body,
                          size_t bcap, uint64_t *body_len, char *err, size_t errcap) {
    HttpRequest req;
    std::string e;
    if (!parse_http_request(fd, &req, &e, (size_t)max_body)) { put_err(err, errcap, e); return 1; }
    put_err(method, mcap, req.method);
    put_err(path, pcap, req.path);
    *body_len = req.body.size();
    if (body && bcap) memcpy(body, req.body.data(), req.body.size() < bcap ? req.body.size() : bcap);
    return 0;
}
// The body of POST /v1/completions (chat = 0) or /v1/chat/completions (chat = 1) turned into prompt ids and a
// generation request, as the server does before it generates.  0 = ok, 1 = refused by validation, 2 = invalid JSON.
int rs_http_prepare(const char *body, int chat, const char *model_name, uint64_t vocab, uint32_t default_backend,
                    rs_request *out, int *stream, uint32_t *ids, size_t cap, uint64_t *n_ids, char *err, size_t errcap) {
    CompletionRequest parsed;
    std::string e;
    if (!parse_completion_request(body, chat != 0, &parsed, &e)) { put_err(err, errcap, e); return 2; }
    ModelConfig cfg = ModelConfig::make(128, 256, 1, 1, 128, 16, 1, vocab);
    HttpServer server(cfg, nullptr, model_name, (DecodeBackendRequest)default_backend);
    std::vector<uint32_t> prompt;
    GenerationRequest req;
    if (!server.prepare(parsed, chat != 0, &prompt, &req, &e)) { put_err(err, errcap, e); return 1; }
    out->backend = (uint32_t)req.decode_backend; out->steps = req.steps; out->temperature = req.temperature;
    out->top_k = req.top_k; out->samples = req.samples; out->seed = req.seed;
    *stream = parsed.has_stream && parsed.stream;
    *n_ids = prompt.size();
    for (size_t i = 0; i < prompt.size() && i < cap; ++i) ids[i] = prompt[i];
    return 0;
}
// bin/serve.rs:616-633 over the "messages" of a chat request body.  0 = ok, 2 = invalid JSON.
int rs_http_render_chat_prompt(const char *body, char *out, size_t cap, char *err, size_t errcap) {
    CompletionRequest parsed;
    std::string e;
    if (!parse_completion_request(body, true, &parsed, &e)) { put_err(err, errcap, e); return 2; }
    put_err(out, cap, render_chat_prompt(parsed.messages));
    return 0;
}

uint64_t rs_next_u64(uint64_t *state) { return next_u64(state); }
float rs_next_f32(uint64_t *state) { return next_f32(state); }
uint32_t rs_sample_next(const float *logits, size_t n, float t, size_t top_k, uint64_t *rng) {
    return sample_next(logits, n, t, top_k, rng, nullptr);
}
uint32_t rs_sample_topk_candidates(const uint32_t *idxs, const float *logits, size_t n, float t, uint64_t *rng) {
    return sample_topk_candidates(idxs, logits, n, t, rng);
}
uint64_t rs_sample_block_from_stats(const float *maxes, const float *sums, size_t n, uint64_t *rng) {
    return sample_block_from_stats(maxes, sums, n, rng);
}
uint64_t rs_sample_softmax_index(const float *logits, size_t n, float t, uint64_t *rng) {
    return sample_softmax_index(logits, n, t, rng);
}
uint32_t rs_sample_block_logits(uint32_t base, const float *logits, size_t n, float t, uint64_t *rng) {
    return sample_block_logits(base, logits, n, t, rng);
}
uint64_t rs_merge_topk_candidates(const float *vals, const uint32_t *idxs, size_t count, size_t top_k, float *out_vals,
                                  uint32_t *out_idxs) {
    return merge_topk_candidates(vals, idxs, count, top_k, out_vals, out_idxs);
}
int rs_validate_token_ids(const uint32_t *ids, size_t n, size_t vocab, const char *source, char *err, size_t errcap) {
    std::string e = validate_token_ids(ids, n, vocab, source);
    put_err(err, errcap, e);
    return e.empty() ? 0 : 1;
}
uint64_t rs_fill_input_window(const uint32_t *generated, size_t n, size_t seq, uint32_t *input) {
    std::vector<uint32_t> in;
    size_t cnt = fill_input_window(std::vector<uint32_t>(generated, generated + n), seq, &in);
    memcpy(input, in.data(), seq * sizeof(uint32_t));
    return cnt;
}

}  // extern "C"
