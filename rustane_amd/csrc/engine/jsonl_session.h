// The line protocol of `generate --jsonl-session` (crates/engine/src/bin/generate.rs:39-144,
// :336-491): one JSON object per stdin line, every field optional, answered by one JSON object per
// stdout line.  The prompt the session was started with stays in the device cache between requests
// (InferenceSession::generate_with_suffix prefills only the appended ids).
#pragma once
#include <stdio.h>

#include <string>
#include <vector>

#include "inference.h"

namespace rustane {

// generate.rs:39-50.  Text prompts need a tokenizer, which this engine does not carry (prompts are ids).
struct JsonlRequest {
    bool has_append_prompt_ids = false, has_append_prompt = false;
    std::vector<uint32_t> append_prompt_ids;
    bool has_decode_backend = false, has_steps = false, has_temperature = false, has_top_k = false, has_samples = false,
         has_seed = false;
    std::string decode_backend;
    size_t steps = 0, top_k = 0, samples = 0;
    float temperature = 0.0f;
    uint64_t seed = 0;
};

// Parses one request line (unknown fields are ignored, as serde does).  On failure *err starts with
// "invalid json request: " (generate.rs:442-451).
bool parse_jsonl_request(const std::string &line, JsonlRequest *out, std::string *err);
// generate.rs:90-112: defaults come from the command line
bool jsonl_to_generation_request(const JsonlRequest &r, const GenerationRequest &defaults, GenerationRequest *out,
                                 std::string *err);
// generate.rs:114-143
bool jsonl_prompt_suffix(const JsonlRequest &r, std::vector<uint32_t> *suffix, std::string *err);
// generate.rs:336-420: the response object, fields in the reference's order (text fields are null)
std::string jsonl_response(const std::vector<uint32_t> &base_prompt_ids, const std::vector<uint32_t> &prompt_ids,
                           const GenerationRequest &req, const GenerationBatch &batch, size_t base_prompt_len);
std::string jsonl_error(const std::string &message);                 // {"error": "..."}
// generate.rs:422-491: serves requests until end of input; returns the number of lines answered
size_t run_jsonl_session(FILE *in, FILE *out, const GenerationRequest &defaults, const std::vector<uint32_t> &prompt_ids,
                         InferenceSession *session);

}  // namespace rustane
