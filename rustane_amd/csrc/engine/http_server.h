// The HTTP front end of the reference's server (crates/engine/src/bin/serve.rs:17-223, :473-1244)
// over the session cache of session_cache.h: one blocking connection at a time, the routes
//   GET  /healthz               liveness, model shape, cache fill
//   GET  /v1/models             the one loaded model
//   POST /v1/completions        prompt_ids (+ max_tokens, temperature, top_k, seed, n, stream, decode_backend)
//   POST /v1/chat/completions   messages, flattened into one prompt
// with JSON answers, or server-sent events over chunked transfer encoding when "stream": true.
// Field names and order, status codes and error texts are the reference's.  This engine carries no
// tokenizer (prompts are token ids): a text prompt is refused with the tokenizer's error prefix,
// every "text" / "content" field of an answer is empty, and -- so that a stream still says what
// was generated -- every streamed choice also carries the ids that are new in it ("generated_ids").
// A chat message may give "content_ids" instead of "content"; the ids of all messages are joined.
#pragma once
#include <stdint.h>

#include <string>
#include <vector>

#include "inference.h"
#include "session_cache.h"

namespace rustane {

// serve.rs:209-213
struct HttpRequest {
    std::string method, path, body;
};

// serve.rs:877-927: request line, headers up to the empty line, Content-Length bytes of body.
// max_body bounds the body a client can make the server allocate.
bool parse_http_request(int fd, HttpRequest *out, std::string *err, size_t max_body = 64u << 20);

// serve.rs:59-63 (+ content_ids, see above)
struct ChatMessage {
    std::string role, content;
    bool has_content = false, has_content_ids = false;
    std::vector<uint32_t> content_ids;
};

// serve.rs:30-57: the fields of a completion request and of a chat completion request (messages
// instead of prompt / prompt_ids); every field but messages is optional, null counts as absent,
// unknown fields are ignored
struct CompletionRequest {
    bool has_model = false, has_prompt = false, has_prompt_ids = false, has_max_tokens = false, has_temperature = false,
         has_top_k = false, has_seed = false, has_n = false, has_stream = false, has_decode_backend = false,
         has_add_special_tokens = false, has_messages = false;
    std::string model, prompt, decode_backend;
    std::vector<uint32_t> prompt_ids;
    std::vector<ChatMessage> messages;
    size_t max_tokens = 0, top_k = 0, n = 0;
    float temperature = 0.0f;
    uint64_t seed = 0;
    bool stream = false, add_special_tokens = false;
};

// On failure *err starts with "invalid JSON: " (serve.rs:1215-1217, :1227-1230); a chat request needs "messages".
bool parse_completion_request(const std::string &body, bool chat, CompletionRequest *out, std::string *err);

// serve.rs:616-633: the trimmed contents of all messages, joined by an empty line
std::string render_chat_prompt(const std::vector<ChatMessage> &messages);

// serve.rs:635-656
bool build_generation_request(const CompletionRequest &req, DecodeBackendRequest default_backend, GenerationRequest *out,
                              std::string *err);

// Pieces of the wire format (serve.rs:929-985, :1162-1181)
std::string http_json_response(int status_code, const std::string &payload);
std::string http_error_response(int status_code, const std::string &message);
std::string sse_headers();
std::string http_chunk(const std::string &payload);
std::string sse_event(const std::string &json);          // one "data: ...\n\n" chunk
std::string sse_done();                                  // "data: [DONE]\n\n" and the terminating chunk

class HttpServer {
public:
    // serve.rs:215-223.  cfg and cache must outlive the server.
    HttpServer(const ModelConfig &cfg, SessionCache *cache, const std::string &model_name, DecodeBackendRequest default_backend);

    // serve.rs:658-725: the prompt ids and the generation request of a parsed body
    bool prepare(const CompletionRequest &req, bool chat, std::vector<uint32_t> *prompt_ids, GenerationRequest *gen,
                 std::string *err) const;

    // One connection (serve.rs:1268-1279): reads a request from fd and answers it; I/O errors end the
    // connection silently.  The caller closes fd.
    void serve_connection(int fd);

    // serve.rs:1247-1281: binds HOST:PORT (port 0: any free port), prints the ready line to stderr and
    // serves connections until the process ends.  Returns only on a set-up error (in *err).
    bool listen_and_serve(const std::string &bind, std::string *err);

private:
    bool route(const HttpRequest &req, int fd, std::string *bad_request);                      // serve.rs:1183-1244
    bool stream_response(const CompletionRequest &req, bool chat, int fd);                    // serve.rs:987-1160
    std::string full_response(const std::vector<uint32_t> &prompt_ids, const CacheGeneration &g, bool chat) const;   // serve.rs:770-851

    const ModelConfig &cfg_;
    SessionCache *cache_;
    std::string model_name_;
    DecodeBackendRequest default_backend_;
};

}  // namespace rustane
