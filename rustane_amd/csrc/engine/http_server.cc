#include "http_server.h"

#include <netdb.h>
#include <netinet/in.h>
#include <sys/socket.h>
#include <sys/time.h>
#include <sys/types.h>
#include <time.h>
#include <unistd.h>

#include <algorithm>

#include "json_util.h"

namespace rustane {
namespace {

using namespace json;

// ---- socket helpers
bool write_all(int fd, const std::string &data) {
    size_t off = 0;
    while (off < data.size()) {
        const ssize_t n = send(fd, data.data() + off, data.size() - off, MSG_NOSIGNAL);
        if (n < 0) {
            if (errno == EINTR) continue;
            return false;
        }
        off += (size_t)n;
    }
    return true;
}

// buffered reads of lines and byte counts from a socket
struct FdReader {
    int fd;
    std::string buf;
    size_t pos = 0;
    explicit FdReader(int f) : fd(f) {}
    // false at end of stream or on error (*err set on error only)
    bool fill(std::string *err) {
        char tmp[4096];
        for (;;) {
            const ssize_t n = recv(fd, tmp, sizeof tmp, 0);
            if (n < 0) {
                if (errno == EINTR) continue;
                *err = strerror(errno);
                return false;
            }
            if (n == 0) return false;
            if (pos > 0 && pos == buf.size()) { buf.clear(); pos = 0; }
            buf.append(tmp, (size_t)n);
            return true;
        }
    }
    // a line including its terminator, as BufRead::read_line (an unterminated last line is returned as it is)
    bool read_line(std::string *line, size_t max_len, std::string *err) {
        line->clear();
        for (;;) {
            const size_t nl = buf.find('\n', pos);
            if (nl != std::string::npos) {
                line->append(buf, pos, nl + 1 - pos);
                pos = nl + 1;
                return true;
            }
            line->append(buf, pos, buf.size() - pos);
            pos = buf.size();
            if (line->size() > max_len) { *err = "line too long"; return false; }
            std::string e;
            if (!fill(&e)) {
                if (!e.empty()) { *err = e; return false; }
                return true;                      // end of stream: what was read so far
            }
        }
    }
    bool read_exact(std::string *out, size_t n, std::string *err) {
        out->clear();
        while (out->size() < n) {
            if (pos == buf.size()) {
                std::string e;
                if (!fill(&e)) { *err = e.empty() ? "failed to fill whole buffer" : e; return false; }
            }
            const size_t take = std::min(n - out->size(), buf.size() - pos);
            out->append(buf, pos, take);
            pos += take;
        }
        return true;
    }
};

std::string trim(const std::string &s) {
    size_t b = 0, e = s.size();
    auto sp = [](unsigned char c) { return c == ' ' || c == '\t' || c == '\n' || c == '\r' || c == '\v' || c == '\f'; };
    while (b < e && sp((unsigned char)s[b])) ++b;
    while (e > b && sp((unsigned char)s[e - 1])) --e;
    return s.substr(b, e - b);
}

uint64_t now_unix() { return (uint64_t)time(nullptr); }                                     // serve.rs:563-568
std::string next_id(const char *prefix, uint64_t seed) {                                    // serve.rs:570-572
    char b[40];
    snprintf(b, sizeof b, "-%llx", (unsigned long long)(seed ^ now_unix()));
    return std::string(prefix) + b;
}

const char *status_text(int code) {                                                         // serve.rs:1173-1179
    switch (code) {
        case 200: return "OK";
        case 400: return "Bad Request";
        case 404: return "Not Found";
        case 405: return "Method Not Allowed";
        case 500: return "Internal Server Error";
        default: return "Error";
    }
}

std::string error_envelope(const std::string &message) {                                    // serve.rs:87-96
    return "{\"error\":{\"message\":" + json_str(message) + ",\"type\":\"invalid_request_error\"}}";
}

std::string usage_json(size_t prompt_tokens, const GenerationBatch &b) {                    // serve.rs:727-738
    const size_t completion = b.results.empty() ? 0 : b.results[0].sampled.size();
    return "{\"prompt_tokens\":" + std::to_string(prompt_tokens) + ",\"completion_tokens\":" + std::to_string(completion) +
           ",\"total_tokens\":" + std::to_string(prompt_tokens + completion) + "}";
}

std::string meta_json(const CacheGeneration &g) {                                           // serve.rs:740-758
    const GenerationBatch &b = g.batch;
    std::string o = "{\"effective_prompt_tokens\":" + std::to_string(g.effective_prompt_tokens);
    o += std::string(",\"prompt_truncated\":") + (g.prompt_truncated ? "true" : "false");
    o += ",\"cache_prefix_tokens\":" + std::to_string(g.cache_prefix_tokens);
    o += std::string(",\"cache_hit\":") + (g.cache_prefix_tokens > 0 ? "true" : "false");
    o += ",\"base_prefill_ms\":" + json_f64(b.base_prefill_elapsed * 1000.0);
    o += ",\"request_prefill_ms\":" + json_f64(b.request_prefill_elapsed * 1000.0);
    o += ",\"total_prefill_ms\":" + json_f64(b.prefill_elapsed * 1000.0);
    o += ",\"decode_ms_total\":" + json_f64(b.total_decode_elapsed * 1000.0);
    o += ",\"decode_ms_avg\":" + json_f64(b.avg_decode_elapsed * 1000.0);
    o += ",\"total_ms\":" + json_f64(b.total_elapsed * 1000.0);
    return o + "}";
}

// one value of an array of u32
bool read_ids(Reader &r, const char *field, std::vector<uint32_t> *out) {
    if (r.i >= r.s.size() || r.s[r.i] != '[') return r.fail(std::string(field) + ": expected an array");
    ++r.i; r.ws();
    out->clear();
    if (r.i < r.s.size() && r.s[r.i] == ']') { ++r.i; return true; }
    for (;;) {
        r.ws();
        uint64_t u = 0;
        if (!r.unsigned_int(&u, 0xffffffffull, "a u32")) return false;
        out->push_back((uint32_t)u);
        r.ws();
        if (r.i < r.s.size() && r.s[r.i] == ',') { ++r.i; continue; }
        if (r.i < r.s.size() && r.s[r.i] == ']') { ++r.i; return true; }
        return r.fail("expected ',' or ']'");
    }
}

bool read_bool(Reader &r, const char *field, bool *out) {
    if (r.lit("true")) { *out = true; return true; }
    if (r.lit("false")) { *out = false; return true; }
    return r.fail(std::string(field) + ": expected a boolean");
}

bool at_null(Reader &r) {
    if (r.s.compare(r.i, 4, "null") == 0) { r.i += 4; return true; }
    return false;
}

// walks the members of an object: calls member(key) with the cursor on the value
template <class F>
bool read_object(Reader &r, F member) {
    r.ws();
    if (r.i >= r.s.size() || r.s[r.i] != '{') return r.fail("expected an object");
    ++r.i; r.ws();
    if (r.i < r.s.size() && r.s[r.i] == '}') { ++r.i; return true; }
    for (;;) {
        r.ws();
        std::string key;
        if (!r.string(&key)) return false;
        r.ws();
        if (r.i >= r.s.size() || r.s[r.i] != ':') return r.fail("expected ':'");
        ++r.i; r.ws();
        if (!member(key)) return false;
        r.ws();
        if (r.i < r.s.size() && r.s[r.i] == ',') { ++r.i; continue; }
        if (r.i < r.s.size() && r.s[r.i] == '}') { ++r.i; return true; }
        return r.fail("expected ',' or '}'");
    }
}

bool read_messages(Reader &r, std::vector<ChatMessage> *out) {
    if (r.i >= r.s.size() || r.s[r.i] != '[') return r.fail("messages: expected an array");
    ++r.i; r.ws();
    out->clear();
    if (r.i < r.s.size() && r.s[r.i] == ']') { ++r.i; return true; }
    for (;;) {
        ChatMessage m;
        bool has_role = false;
        if (!read_object(r, [&](const std::string &key) {
                if (key == "role") { has_role = true; return r.string(&m.role); }
                if (key == "content") { m.has_content = true; return r.string(&m.content); }
                if (key == "content_ids") {
                    if (at_null(r)) return true;
                    m.has_content_ids = true;
                    return read_ids(r, "content_ids", &m.content_ids);
                }
                return r.skip();
            }))
            return false;
        if (!has_role) return r.fail("missing field `role`");
        if (!m.has_content && !m.has_content_ids) return r.fail("missing field `content`");
        out->push_back(std::move(m));
        r.ws();
        if (r.i < r.s.size() && r.s[r.i] == ',') { ++r.i; r.ws(); continue; }
        if (r.i < r.s.size() && r.s[r.i] == ']') { ++r.i; return true; }
        return r.fail("expected ',' or ']'");
    }
}

}  // namespace

bool parse_http_request(int fd, HttpRequest *out, std::string *err, size_t max_body) {
    constexpr size_t kMaxLine = 64 * 1024, kMaxHeaders = 256;
    FdReader rd(fd);
    std::string line, e;
    if (!rd.read_line(&line, kMaxLine, &e)) { *err = "failed to read request line: " + e; return false; }
    if (trim(line).empty()) { *err = "empty request"; return false; }
    // split_whitespace: method, then path
    std::vector<std::string> parts;
    {
        size_t i = 0;
        while (i < line.size() && parts.size() < 2) {
            while (i < line.size() && isspace((unsigned char)line[i])) ++i;
            size_t j = i;
            while (j < line.size() && !isspace((unsigned char)line[j])) ++j;
            if (j > i) parts.push_back(line.substr(i, j - i));
            i = j;
        }
    }
    if (parts.empty()) { *err = "missing HTTP method"; return false; }
    if (parts.size() < 2) { *err = "missing HTTP path"; return false; }
    out->method = parts[0];
    out->path = parts[1];

    bool has_length = false;
    std::string length_raw;
    for (size_t nh = 0;; ++nh) {
        if (nh > kMaxHeaders) { *err = "failed to read header line: too many header lines"; return false; }
        if (!rd.read_line(&line, kMaxLine, &e)) { *err = "failed to read header line: " + e; return false; }
        while (!line.empty() && (line.back() == '\r' || line.back() == '\n')) line.pop_back();
        if (line.empty()) break;
        const size_t colon = line.find(':');
        if (colon == std::string::npos) continue;
        std::string name = trim(line.substr(0, colon));
        std::transform(name.begin(), name.end(), name.begin(), [](unsigned char c) { return (char)tolower(c); });
        if (name == "content-length") { has_length = true; length_raw = trim(line.substr(colon + 1)); }
    }
    size_t content_length = 0;
    if (has_length) {
        if (length_raw.empty() || length_raw.find_first_not_of("0123456789") != std::string::npos || length_raw.size() > 18) {
            *err = "invalid content-length";
            return false;
        }
        content_length = (size_t)strtoull(length_raw.c_str(), nullptr, 10);
    }
    if (content_length > max_body) { *err = "request body too large"; return false; }
    if (!rd.read_exact(&out->body, content_length, &e)) { *err = "failed to read request body: " + e; return false; }
    return true;
}

bool parse_completion_request(const std::string &body, bool chat, CompletionRequest *out, std::string *err) {
    *out = CompletionRequest();
    Reader r(body);
    auto bad = [&]() { *err = "invalid JSON: " + (r.err.empty() ? std::string("malformed object") : r.err); return false; };
    uint64_t u = 0;
    double d = 0.0;
    const bool ok = read_object(r, [&](const std::string &key) {
        if (chat && key == "messages") { out->has_messages = true; return read_messages(r, &out->messages); }
        const bool known = key == "model" || key == "max_tokens" || key == "temperature" || key == "top_k" || key == "seed" ||
                           key == "n" || key == "stream" || key == "decode_backend" || key == "add_special_tokens" ||
                           (!chat && (key == "prompt" || key == "prompt_ids"));
        if (!known) return r.skip();
        if (at_null(r)) return true;                                   // Option<T>: null is "not given"
        if (key == "model") { out->has_model = true; return r.string(&out->model); }
        if (key == "prompt") { out->has_prompt = true; return r.string(&out->prompt); }
        if (key == "prompt_ids") { out->has_prompt_ids = true; return read_ids(r, "prompt_ids", &out->prompt_ids); }
        if (key == "decode_backend") { out->has_decode_backend = true; return r.string(&out->decode_backend); }
        if (key == "stream") { out->has_stream = true; return read_bool(r, "stream", &out->stream); }
        if (key == "add_special_tokens") { out->has_add_special_tokens = true; return read_bool(r, "add_special_tokens", &out->add_special_tokens); }
        if (key == "temperature") {
            if (!r.real(&d)) return false;
            out->temperature = (float)d; out->has_temperature = true;
            return true;
        }
        if (key == "seed") {
            if (!r.unsigned_int(&u, UINT64_MAX, "u64")) return false;
            out->seed = u; out->has_seed = true;
            return true;
        }
        if (!r.unsigned_int(&u, SIZE_MAX, "usize")) return false;      // max_tokens, top_k, n
        if (key == "max_tokens") { out->max_tokens = (size_t)u; out->has_max_tokens = true; }
        else if (key == "top_k") { out->top_k = (size_t)u; out->has_top_k = true; }
        else { out->n = (size_t)u; out->has_n = true; }
        return true;
    });
    if (!ok) return bad();
    r.ws();
    if (r.i != body.size()) { r.fail("trailing characters"); return bad(); }
    if (chat && !out->has_messages) { r.fail("missing field `messages`"); return bad(); }
    return true;
}

std::string render_chat_prompt(const std::vector<ChatMessage> &messages) {
    std::string out;
    for (size_t i = 0; i < messages.size(); ++i) {
        if (i) out += "\n\n";
        out += trim(messages[i].content);            // (every role is rendered the same way, serve.rs:622-630)
    }
    return out;
}

bool build_generation_request(const CompletionRequest &req, DecodeBackendRequest default_backend, GenerationRequest *out,
                              std::string *err) {
    const size_t samples = req.has_n ? req.n : 1;
    if (samples == 0) { *err = "n must be >= 1"; return false; }
    GenerationRequest g;
    g.decode_backend = default_backend;
    if (req.has_decode_backend && !parse_decode_backend(req.decode_backend, &g.decode_backend)) {      // serve.rs:574-583
        *err = decode_backend_error("decode_backend", req.decode_backend);
        return false;
    }
    g.steps = req.has_max_tokens ? req.max_tokens : 32;
    g.temperature = req.has_temperature ? req.temperature : 0.0f;
    g.top_k = req.has_top_k ? req.top_k : 0;
    g.samples = samples;
    g.seed = req.has_seed ? req.seed : 1;
    *out = g;
    return true;
}

std::string http_json_response(int status_code, const std::string &payload) {
    char head[160];
    snprintf(head, sizeof head, "HTTP/1.1 %d %s\r\nContent-Type: application/json\r\nContent-Length: %zu\r\nConnection: close\r\n\r\n",
             status_code, status_text(status_code), payload.size());
    return head + payload;
}
std::string http_error_response(int status_code, const std::string &message) {
    return http_json_response(status_code, error_envelope(message));
}
std::string sse_headers() {
    return "HTTP/1.1 200 OK\r\nContent-Type: text/event-stream\r\nCache-Control: no-cache\r\nConnection: close\r\n"
           "Transfer-Encoding: chunked\r\n\r\n";
}
std::string http_chunk(const std::string &payload) {
    char head[24];
    snprintf(head, sizeof head, "%zX\r\n", payload.size());
    return head + payload + "\r\n";
}
std::string sse_event(const std::string &json) { return http_chunk("data: " + json + "\n\n"); }
std::string sse_done() { return http_chunk("data: [DONE]\n\n") + "0\r\n\r\n"; }

HttpServer::HttpServer(const ModelConfig &cfg, SessionCache *cache, const std::string &model_name,
                       DecodeBackendRequest default_backend)
    : cfg_(cfg), cache_(cache), model_name_(model_name), default_backend_(default_backend) {}

bool HttpServer::prepare(const CompletionRequest &req, bool chat, std::vector<uint32_t> *prompt_ids, GenerationRequest *gen,
                         std::string *err) const {
    if (req.has_model && req.model != model_name_) {
        *err = "requested model " + req.model + " does not match loaded model " + model_name_;
        return false;
    }
    static const char *kNoTokenizer = "failed to encode prompt: this build carries no tokenizer; pass token ids (prompt_ids, or "
                                      "content_ids in chat messages)";
    prompt_ids->clear();
    if (!chat) {
        if (req.has_prompt && req.has_prompt_ids) { *err = "pass either prompt or prompt_ids, not both"; return false; }
        if (req.has_prompt) { *err = kNoTokenizer; return false; }
        if (!req.has_prompt_ids) { *err = "one of prompt or prompt_ids is required"; return false; }
        *prompt_ids = req.prompt_ids;
    } else {
        if (req.messages.empty()) { *err = "messages must contain at least one item"; return false; }
        for (const ChatMessage &m : req.messages) {
            if (!m.has_content_ids || !trim(m.content).empty()) { *err = kNoTokenizer; return false; }
            prompt_ids->insert(prompt_ids->end(), m.content_ids.begin(), m.content_ids.end());
        }
    }
    // serve.rs:599-613
    if (prompt_ids->empty()) { *err = "prompt encoded to zero tokens"; return false; }
    for (size_t pos = 0; pos < prompt_ids->size(); ++pos)
        if ((size_t)(*prompt_ids)[pos] >= cfg_.vocab) {
            *err = "prompt token id " + std::to_string((*prompt_ids)[pos]) + " at position " + std::to_string(pos) +
                   " exceeds model vocab " + std::to_string(cfg_.vocab);
            return false;
        }
    return build_generation_request(req, default_backend_, gen, err);
}

std::string HttpServer::full_response(const std::vector<uint32_t> &prompt_ids, const CacheGeneration &g, bool chat) const {
    const GenerationBatch &b = g.batch;
    std::string o = "{\"id\":" + json_str(next_id(chat ? "chatcmpl" : "cmpl", (uint64_t)(b.total_elapsed * 1e9)));
    o += std::string(",\"object\":") + (chat ? "\"chat.completion\"" : "\"text_completion\"");
    o += ",\"created\":" + std::to_string(now_unix());
    o += ",\"model\":" + json_str(model_name_);
    o += ",\"choices\":[";
    for (size_t i = 0; i < b.results.size(); ++i) {
        const SampleResult &r = b.results[i];
        if (i) o += ",";
        o += "{\"index\":" + std::to_string(i);
        o += chat ? ",\"message\":{\"role\":\"assistant\",\"content\":\"\"}" : ",\"text\":\"\"";
        o += ",\"finish_reason\":\"length\"";
        o += ",\"generated_ids\":" + json_ids(r.sampled);
        o += ",\"full_sequence\":" + json_ids(r.generated) + "}";
    }
    o += "],\"usage\":" + usage_json(prompt_ids.size(), b);
    o += ",\"rustane\":" + meta_json(g) + "}";
    return o;
}

bool HttpServer::stream_response(const CompletionRequest &req, bool chat, int fd) {
    std::vector<uint32_t> prompt_ids;
    GenerationRequest gen;
    std::string err;
    if (!prepare(req, chat, &prompt_ids, &gen, &err)) return write_all(fd, http_error_response(400, err));
    if (gen.samples != 1) return write_all(fd, http_error_response(400, "stream=true only supports n=1"));

    if (!write_all(fd, sse_headers())) return false;
    const uint64_t created = now_unix();
    const std::string id = next_id(chat ? "chatcmpl" : "cmpl", gen.seed ^ (uint64_t)prompt_ids.size());
    const std::string head = "{\"id\":" + json_str(id) + ",\"object\":" + (chat ? "\"chat.completion.chunk\"" : "\"text_completion\"") +
                             ",\"created\":" + std::to_string(created) + ",\"model\":" + json_str(model_name_) + ",\"choices\":[{\"index\":0,";
    // a choice: the text part (completion: "text", chat: "delta"), finish_reason, the ids new in this event
    auto event = [&](const std::string &text_part, const char *finish, const std::vector<uint32_t> &new_ids, const std::string &meta) {
        std::string o = head + text_part + ",\"finish_reason\":" + (finish ? json_str(finish) : "null") +
                        ",\"generated_ids\":" + json_ids(new_ids) + "}]";
        if (!meta.empty()) o += ",\"rustane\":" + meta;
        return sse_event(o + "}");
    };
    if (chat && !write_all(fd, event("\"delta\":{\"role\":\"assistant\"}", nullptr, {}, ""))) return false;     // serve.rs:1081-1099

    size_t sent = 0;
    CacheGeneration outcome;
    const bool ok = cache_->stream_generate(
        prompt_ids, gen,
        [&](uint32_t, const std::vector<uint32_t> &sampled, const std::vector<uint32_t> &) -> std::string {
            std::vector<uint32_t> fresh(sampled.begin() + (long)std::min(sent, sampled.size()), sampled.end());
            sent = sampled.size();
            if (fresh.empty()) return "";
            if (!write_all(fd, event(chat ? "\"delta\":{\"content\":\"\"}" : "\"text\":\"\"", nullptr, fresh, "")))
                return "client closed the stream";
            return "";
        },
        &outcome, &err);
    if (!ok) return write_all(fd, sse_event(error_envelope(err)) + sse_done());                                  // serve.rs:976-985
    return write_all(fd, event(chat ? "\"delta\":{}" : "\"text\":\"\"", "length", {}, meta_json(outcome)) + sse_done());
}

bool HttpServer::route(const HttpRequest &req, int fd, std::string *bad_request) {
    const bool get = req.method == "GET", post = req.method == "POST";
    if (get && req.path == "/healthz") {
        const std::string body = "{\"ok\":true,\"model\":" + json_str(model_name_) + ",\"vocab\":" + std::to_string(cfg_.vocab) +
                                 ",\"seq\":" + std::to_string(cfg_.seq) + ",\"cache_entries\":" + std::to_string(cache_->len()) +
                                 ",\"max_cache_sessions\":" + std::to_string(cache_->max_entries()) + "}";
        return write_all(fd, http_json_response(200, body));
    }
    if (get && req.path == "/v1/models") {
        const std::string body = "{\"object\":\"list\",\"data\":[{\"id\":" + json_str(model_name_) +
                                 ",\"object\":\"model\",\"owned_by\":\"rustane\"}]}";
        return write_all(fd, http_json_response(200, body));
    }
    const bool completions = req.path == "/v1/completions", chat = req.path == "/v1/chat/completions";
    if (post && (completions || chat)) {
        CompletionRequest parsed;
        if (!parse_completion_request(req.body, chat, &parsed, bad_request)) return true;       // answered by the caller with 400
        if (parsed.has_stream && parsed.stream) return stream_response(parsed, chat, fd);
        std::vector<uint32_t> prompt_ids;
        GenerationRequest gen;
        CacheGeneration outcome;
        std::string err;
        if (!prepare(parsed, chat, &prompt_ids, &gen, &err) || !cache_->generate(prompt_ids, gen, &outcome, &err))
            return write_all(fd, http_error_response(400, err));
        return write_all(fd, http_json_response(200, full_response(prompt_ids, outcome, chat)));
    }
    if (get || post) return write_all(fd, http_error_response(404, "unknown route"));
    return write_all(fd, http_error_response(405, "unsupported HTTP method"));
}

void HttpServer::serve_connection(int fd) {
    HttpRequest req;
    std::string err;
    if (!parse_http_request(fd, &req, &err)) {
        write_all(fd, http_error_response(400, err));
        return;
    }
    std::string bad_request;
    if (route(req, fd, &bad_request) && !bad_request.empty()) write_all(fd, http_error_response(400, bad_request));
}

bool HttpServer::listen_and_serve(const std::string &bind_addr, std::string *err) {
    const size_t colon = bind_addr.rfind(':');
    if (colon == std::string::npos) { *err = "--bind must be HOST:PORT, got " + bind_addr; return false; }
    const std::string host = bind_addr.substr(0, colon), port = bind_addr.substr(colon + 1);
    addrinfo hints{}, *res = nullptr;
    hints.ai_family = AF_UNSPEC;
    hints.ai_socktype = SOCK_STREAM;
    hints.ai_flags = AI_PASSIVE | AI_NUMERICSERV;
    const int gai = getaddrinfo(host.empty() ? nullptr : host.c_str(), port.c_str(), &hints, &res);
    if (gai != 0) { *err = "failed to bind server: " + std::string(gai_strerror(gai)); return false; }
    int lfd = -1;
    std::string last = "no usable address";
    for (addrinfo *a = res; a; a = a->ai_next) {
        lfd = socket(a->ai_family, a->ai_socktype, a->ai_protocol);
        if (lfd < 0) { last = strerror(errno); continue; }
        const int one = 1;
        setsockopt(lfd, SOL_SOCKET, SO_REUSEADDR, &one, sizeof one);
        if (::bind(lfd, a->ai_addr, a->ai_addrlen) == 0 && listen(lfd, 64) == 0) break;
        last = strerror(errno);
        close(lfd);
        lfd = -1;
    }
    freeaddrinfo(res);
    if (lfd < 0) { *err = "failed to bind server: " + last; return false; }

    // the address actually bound (a requested port 0 becomes the port the system chose)
    std::string shown = bind_addr;
    sockaddr_storage ss{};
    socklen_t sl = sizeof ss;
    if (getsockname(lfd, (sockaddr *)&ss, &sl) == 0) {
        const unsigned p = ss.ss_family == AF_INET6 ? ntohs(((sockaddr_in6 *)&ss)->sin6_port) : ntohs(((sockaddr_in *)&ss)->sin_port);
        shown = host + ":" + std::to_string(p);
    }
    fprintf(stderr, "rustane_serve_ready bind=%s model=%s vocab=%zu seq=%zu cache_sessions=%zu\n", shown.c_str(),
            model_name_.c_str(), cfg_.vocab, cfg_.seq, cache_->max_entries());                     // serve.rs:1264-1267
    fflush(stderr);

    for (;;) {
        const int fd = accept(lfd, nullptr, nullptr);
        if (fd < 0) {
            if (errno == EINTR) continue;
            fprintf(stderr, "accept failed: %s\n", strerror(errno));
            usleep(100 * 1000);                       // (out of descriptors and the like: do not spin on it)
            continue;
        }
        timeval tv{30, 0};                            // a client that stops sending does not hold the one connection for ever
        setsockopt(fd, SOL_SOCKET, SO_RCVTIMEO, &tv, sizeof tv);
        setsockopt(fd, SOL_SOCKET, SO_SNDTIMEO, &tv, sizeof tv);
        serve_connection(fd);
        shutdown(fd, SHUT_WR);
        close(fd);
    }
}

}  // namespace rustane
