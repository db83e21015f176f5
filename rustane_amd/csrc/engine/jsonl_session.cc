#include "jsonl_session.h"

#include <errno.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

namespace rustane {
namespace {

// ---- a reader for the flat objects of the protocol: strings, numbers, booleans, null, arrays of numbers
struct Reader {
    const std::string &s;
    size_t i = 0;
    std::string err;

    explicit Reader(const std::string &str) : s(str) {}
    void ws() { while (i < s.size() && (s[i] == ' ' || s[i] == '\t' || s[i] == '\r' || s[i] == '\n')) ++i; }
    bool fail(const std::string &m) { if (err.empty()) err = m + " at column " + std::to_string(i + 1); return false; }
    bool lit(const char *w) {
        const size_t n = strlen(w);
        if (s.compare(i, n, w) == 0) { i += n; return true; }
        return false;
    }
    bool string(std::string *out) {
        if (i >= s.size() || s[i] != '"') return fail("expected a string");
        ++i;
        out->clear();
        while (i < s.size() && s[i] != '"') {
            char c = s[i++];
            if (c == '\\') {
                if (i >= s.size()) return fail("unterminated escape");
                const char e = s[i++];
                switch (e) {
                    case '"': c = '"'; break;
                    case '\\': c = '\\'; break;
                    case '/': c = '/'; break;
                    case 'b': c = '\b'; break;
                    case 'f': c = '\f'; break;
                    case 'n': c = '\n'; break;
                    case 'r': c = '\r'; break;
                    case 't': c = '\t'; break;
                    case 'u': {
                        if (i + 4 > s.size()) return fail("short \\u escape");
                        unsigned v = 0;
                        for (int k = 0; k < 4; ++k) {
                            const char h = s[i++];
                            v <<= 4;
                            if (h >= '0' && h <= '9') v |= (unsigned)(h - '0');
                            else if (h >= 'a' && h <= 'f') v |= (unsigned)(h - 'a' + 10);
                            else if (h >= 'A' && h <= 'F') v |= (unsigned)(h - 'A' + 10);
                            else return fail("bad \\u escape");
                        }
                        // UTF-8 of the code unit (surrogate pairs are not joined: no field here needs them)
                        if (v < 0x80) out->push_back((char)v);
                        else if (v < 0x800) { out->push_back((char)(0xC0 | (v >> 6))); out->push_back((char)(0x80 | (v & 0x3F))); }
                        else { out->push_back((char)(0xE0 | (v >> 12))); out->push_back((char)(0x80 | ((v >> 6) & 0x3F))); out->push_back((char)(0x80 | (v & 0x3F))); }
                        continue;
                    }
                    default: return fail("bad escape");
                }
            }
            out->push_back(c);
        }
        if (i >= s.size()) return fail("unterminated string");
        ++i;
        return true;
    }
    // the characters of a JSON number
    bool number_text(std::string *out) {
        const size_t b = i;
        if (i < s.size() && s[i] == '-') ++i;
        while (i < s.size() && ((s[i] >= '0' && s[i] <= '9') || s[i] == '.' || s[i] == 'e' || s[i] == 'E' || s[i] == '+' || s[i] == '-')) ++i;
        if (i == b) return fail("expected a number");
        *out = s.substr(b, i - b);
        return true;
    }
    bool unsigned_int(uint64_t *v, uint64_t max, const char *what) {
        std::string t;
        if (!number_text(&t)) return false;
        if (t.empty() || t.find_first_not_of("0123456789") != std::string::npos) return fail(std::string("expected ") + what);
        errno = 0;
        char *end = nullptr;
        const unsigned long long x = strtoull(t.c_str(), &end, 10);
        if (errno || *end || x > max) return fail(std::string("number out of range for ") + what);
        *v = x;
        return true;
    }
    bool real(double *v) {
        std::string t;
        if (!number_text(&t)) return false;
        char *end = nullptr;
        *v = strtod(t.c_str(), &end);
        if (*end) return fail("malformed number");
        return true;
    }
    // skips any value (fields the protocol does not know)
    bool skip() {
        ws();
        if (i >= s.size()) return fail("unexpected end of input");
        std::string tmp;
        if (s[i] == '"') return string(&tmp);
        if (s[i] == '{' || s[i] == '[') {
            const char close = s[i] == '{' ? '}' : ']';
            const bool obj = s[i] == '{';
            ++i; ws();
            if (i < s.size() && s[i] == close) { ++i; return true; }
            for (;;) {
                ws();
                if (obj) { if (!string(&tmp)) return false; ws(); if (i >= s.size() || s[i] != ':') return fail("expected ':'"); ++i; }
                if (!skip()) return false;
                ws();
                if (i < s.size() && s[i] == ',') { ++i; continue; }
                if (i < s.size() && s[i] == close) { ++i; return true; }
                return fail("expected ',' or a closing bracket");
            }
        }
        if (lit("true") || lit("false") || lit("null")) return true;
        return number_text(&tmp);
    }
};

// shortest decimal form that reads back as the same double, always with a fraction or exponent
std::string json_f64(double v) {
    if (!isfinite(v)) return "null";
    char buf[40];
    for (int p = 1; p <= 17; ++p) {
        snprintf(buf, sizeof buf, "%.*g", p, v);
        if (strtod(buf, nullptr) == v) break;
    }
    if (!strpbrk(buf, ".eEn")) strcat(buf, ".0");
    return buf;
}
std::string json_str(const std::string &s) {
    std::string o = "\"";
    for (unsigned char c : s) {
        switch (c) {
            case '"': o += "\\\""; break;
            case '\\': o += "\\\\"; break;
            case '\n': o += "\\n"; break;
            case '\r': o += "\\r"; break;
            case '\t': o += "\\t"; break;
            default:
                if (c < 0x20) { char b[8]; snprintf(b, sizeof b, "\\u%04x", c); o += b; }
                else o.push_back((char)c);
        }
    }
    return o + "\"";
}
std::string json_opt(const char *s) { return s ? json_str(s) : "null"; }
std::string json_ids(const std::vector<uint32_t> &ids) {
    std::string o = "[";
    for (size_t i = 0; i < ids.size(); ++i) { if (i) o += ","; o += std::to_string(ids[i]); }
    return o + "]";
}

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
        *err = "decode_backend must be one of: auto, naive, hip; got " + r.decode_backend;
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
