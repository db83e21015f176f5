#include "jsonl_session.h"

#include "json_util.h"

#include <errno.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

namespace rustane {
namespace {

using namespace json;

}  // namespace

bool parse_jsonl_request(const std::string &line, JsonlRequest *out, std::string *err) {
    *out = JsonlRequest();
    Reader r(line);
    auto bad = [&]() { *err = "invalid json request: " + (r.err.empty() ? std::string("malformed object") : r.err); return false; };
    r.ws();
    if (r.i >= line.size() || line[r.i] != '{') { r.fail("expected an object"); return bad(); }
    ++r.i; r.ws();
    if (r.i < line.size() && line[r.i] == '}') ++r.i;
    else for (;;) {
        r.ws();
        std::string key;
        if (!r.string(&key)) return bad();
        r.ws();
        if (r.i >= line.size() || line[r.i] != ':') { r.fail("expected ':'"); return bad(); }
        ++r.i; r.ws();
        uint64_t u = 0;
        double d = 0.0;
        const bool is_null = line.compare(r.i, 4, "null") == 0;
        if (is_null && (key == "append_prompt_ids" || key == "append_prompt" || key == "add_special_tokens" ||
                        key == "decode_backend" || key == "steps" || key == "temperature" || key == "top_k" ||
                        key == "samples" || key == "seed")) {
            r.i += 4;                                             // Option<T>: null is "not given"
        } else if (key == "append_prompt_ids") {
            if (r.i >= line.size() || line[r.i] != '[') { r.fail("append_prompt_ids: expected an array"); return bad(); }
            ++r.i; r.ws();
            out->has_append_prompt_ids = true;
            if (r.i < line.size() && line[r.i] == ']') ++r.i;
            else for (;;) {
                r.ws();
                if (!r.unsigned_int(&u, 0xffffffffull, "a u32")) return bad();
                out->append_prompt_ids.push_back((uint32_t)u);
                r.ws();
                if (r.i < line.size() && line[r.i] == ',') { ++r.i; continue; }
                if (r.i < line.size() && line[r.i] == ']') { ++r.i; break; }
                r.fail("expected ',' or ']'");
                return bad();
            }
        } else if (key == "append_prompt") {
            std::string text;
            if (!r.string(&text)) return bad();
            out->has_append_prompt = true;
        } else if (key == "add_special_tokens") {
            if (!r.lit("true") && !r.lit("false")) { r.fail("add_special_tokens: expected a boolean"); return bad(); }
        } else if (key == "decode_backend") {
            if (!r.string(&out->decode_backend)) return bad();
            out->has_decode_backend = true;
        } else if (key == "steps") {
            if (!r.unsigned_int(&u, SIZE_MAX, "usize")) return bad();
            out->steps = (size_t)u; out->has_steps = true;
        } else if (key == "top_k") {
            if (!r.unsigned_int(&u, SIZE_MAX, "usize")) return bad();
            out->top_k = (size_t)u; out->has_top_k = true;
        } else if (key == "samples") {
            if (!r.unsigned_int(&u, SIZE_MAX, "usize")) return bad();
            out->samples = (size_t)u; out->has_samples = true;
        } else if (key == "seed") {
            if (!r.unsigned_int(&u, UINT64_MAX, "u64")) return bad();
            out->seed = u; out->has_seed = true;
        } else if (key == "temperature") {
            if (!r.real(&d)) return bad();
            out->temperature = (float)d; out->has_temperature = true;
        } else if (!r.skip()) {
            return bad();
        }
        r.ws();
        if (r.i < line.size() && line[r.i] == ',') { ++r.i; continue; }
        if (r.i < line.size() && line[r.i] == '}') { ++r.i; break; }
        r.fail("expected ',' or '}'");
        return bad();
    }
    r.ws();
    if (r.i != line.size()) { r.fail("trailing characters"); return bad(); }
    return true;
}

bool jsonl_to_generation_request(const JsonlRequest &r, const GenerationRequest &defaults, GenerationRequest *out,
                                 std::string *err) {
    *out = defaults;
    if (r.has_decode_backend && !parse_decode_backend(r.decode_backend, &out->decode_backend)) {
        *err = decode_backend_error("decode_backend", r.decode_backend);
        return false;
    }
    if (r.has_samples) out->samples = r.samples;
    if (out->samples == 0) { *err = "samples must be >= 1"; return false; }
    if (r.has_steps) out->steps = r.steps;
    if (r.has_temperature) out->temperature = r.temperature;
    if (r.has_top_k) out->top_k = r.top_k;
    if (r.has_seed) out->seed = r.seed;
    return true;
}

bool jsonl_prompt_suffix(const JsonlRequest &r, std::vector<uint32_t> *suffix, std::string *err) {
    suffix->clear();
    if (r.has_append_prompt_ids && r.has_append_prompt) { *err = "pass either append_prompt_ids or append_prompt, not both"; return false; }
    if (r.has_append_prompt_ids) { *suffix = r.append_prompt_ids; return true; }
    if (r.has_append_prompt) { *err = "append_prompt requires the session to be started with --tokenizer"; return false; }
    return true;
}

std::string jsonl_response(const std::vector<uint32_t> &base_prompt_ids, const std::vector<uint32_t> &prompt_ids,
                           const GenerationRequest &req, const GenerationBatch &b, size_t base_prompt_len) {
    const size_t decode_steps = b.results.empty() || b.results[0].sampled.empty() ? 0 : b.results[0].sampled.size() - 1;
    const double base_tps = b.base_prefill_elapsed > 0 ? (double)base_prompt_len / b.base_prefill_elapsed : 0.0;
    const double avg_tps = decode_steps > 0 && b.avg_decode_elapsed > 0 ? (double)decode_steps / b.avg_decode_elapsed : 0.0;
    const double e2e_tps = b.total_elapsed > 0 ? (double)(req.steps * req.samples) / b.total_elapsed : 0.0;
    std::string o = "{";
    o += "\"decode_backend_request\":" + json_str(decode_backend_str(req.decode_backend));
    o += ",\"decode_mode\":" + json_str(decode_mode_str(b.decode_selection.mode));
    o += ",\"fallback_reason\":" + json_opt(b.decode_selection.fallback_reason);
    o += ",\"auto_reason\":" + json_opt(b.decode_selection.auto_reason);
    o += ",\"base_prompt_ids\":" + json_ids(base_prompt_ids);
    o += ",\"prompt_ids\":" + json_ids(prompt_ids);
    o += ",\"base_prompt_text\":null,\"prompt_text\":null";
    o += ",\"base_prefill_ms\":" + json_f64(b.base_prefill_elapsed * 1000.0);
    o += ",\"base_prefill_tok_per_s\":" + json_f64(base_tps);
    o += ",\"request_prefill_ms\":" + json_f64(b.request_prefill_elapsed * 1000.0);
    o += ",\"total_prefill_ms\":" + json_f64(b.prefill_elapsed * 1000.0);
    o += ",\"request_decode_ms_total\":" + json_f64(b.total_decode_elapsed * 1000.0);
    o += ",\"request_decode_ms_avg\":" + json_f64(b.avg_decode_elapsed * 1000.0);
    o += ",\"request_avg_decode_tok_per_s\":" + json_f64(avg_tps);
    o += ",\"end_to_end_ms_including_prefill\":" + json_f64(b.total_elapsed * 1000.0);
    o += ",\"end_to_end_tok_per_s_including_prefill\":" + json_f64(e2e_tps);
    o += ",\"results\":[";
    for (size_t i = 0; i < b.results.size(); ++i) {
        const SampleResult &r = b.results[i];
        if (i) o += ",";
        o += "{\"seed\":" + std::to_string(r.seed);
        o += ",\"generated_ids\":" + json_ids(r.sampled);
        o += ",\"full_sequence\":" + json_ids(r.generated);
        o += ",\"generated_text\":null,\"full_text\":null";
        o += ",\"decode_time_ms\":" + json_f64(r.decode_elapsed * 1000.0);
        o += ",\"decode_tok_per_s\":" + json_f64(decode_steps > 0 && r.decode_elapsed > 0 ? (double)decode_steps / r.decode_elapsed : 0.0);
        o += "}";
    }
    o += "]}";
    return o;
}

std::string jsonl_error(const std::string &message) { return "{\"error\":" + json_str(message) + "}"; }

size_t run_jsonl_session(FILE *in, FILE *out, const GenerationRequest &defaults, const std::vector<uint32_t> &prompt_ids,
                         InferenceSession *session) {
    size_t answered = 0;
    std::string line;
    auto put = [&](const std::string &obj) {
        fputs(obj.c_str(), out);
        fputc('\n', out);
        fflush(out);
        ++answered;
    };
    for (;;) {
        line.clear();
        int c;
        while ((c = fgetc(in)) != EOF && c != '\n') line.push_back((char)c);
        if (c == EOF && line.empty()) break;
        if (line.find_first_not_of(" \t\r\n") == std::string::npos) { if (c == EOF) break; continue; }
        JsonlRequest parsed;
        GenerationRequest req;
        std::vector<uint32_t> suffix;
        std::string err;
        if (!parse_jsonl_request(line, &parsed, &err) || !jsonl_to_generation_request(parsed, defaults, &req, &err) ||
            !jsonl_prompt_suffix(parsed, &suffix, &err)) {
            put(jsonl_error(err));
        } else {
            std::vector<uint32_t> effective = prompt_ids;
            effective.insert(effective.end(), suffix.begin(), suffix.end());
            GenerationBatch batch;
            if (!session->generate_with_suffix(req, suffix, &batch, &err)) put(jsonl_error(err));
            else put(jsonl_response(prompt_ids, effective, req, batch, session->prompt_len()));
        }
        if (c == EOF) break;
    }
    return answered;
}

}  // namespace rustane
