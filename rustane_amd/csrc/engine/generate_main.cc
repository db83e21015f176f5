// `generate`: token-id generation over the HIP decode backend with the flags and report lines of
// the reference's CLI (crates/engine/src/bin/generate.rs:145-280 flags, :603-728 report).  Text
// tokenisation and checkpoint files are outside this build: prompts are token ids and weights are
// synthetic (seeded) for a named or custom shape.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "checkpoint.h"
#include "inference.h"
#include "jsonl_session.h"
#include "synth.h"

using namespace rustane;

namespace {

[[noreturn]] void fail(const std::string &msg) {
    fprintf(stderr, "error: %s\n", msg.c_str());
    exit(2);
}

void usage() {
    printf("usage: generate (--checkpoint PATH | --model <preset|custom:dim,hidden,nlayers,seq[,heads,hd,vocab]>) --prompt-ids 1,2,3\n"
           "  [--steps N] [--temperature T] [--top-k K] [--softcap C] [--samples N] [--seed S]\n"
           "  [--decode-backend auto|naive|hip] [--kv-cache] [--weight-dtype f32|bf16|fp8|int4] [--kv-dtype f32|bf16]\n"
           "  [--weight-seed S] [--weight-std X] [--random-prompt N] [--jsonl-session]\n"
           "presets: gpt_karpathy gpt_1024 target_600m target_800m target_1b target_1_5b bench_tiny bench_600m bench_5b\n");
}

std::vector<uint32_t> parse_ids(const std::string &s) {
    std::vector<uint32_t> ids;
    size_t i = 0;
    while (i < s.size()) {
        size_t j = s.find(',', i);
        if (j == std::string::npos) j = s.size();
        std::string tok = s.substr(i, j - i);
        if (!tok.empty()) {
            char *end = nullptr;
            unsigned long v = strtoul(tok.c_str(), &end, 10);
            if (*end) fail("prompt ids must be comma-separated integers, got '" + tok + "'");
            ids.push_back((uint32_t)v);
        }
        i = j + 1;
    }
    return ids;
}

bool model_from_name(const std::string &name, ModelConfig *cfg) {
    if (name == "gpt_karpathy") *cfg = ModelConfig::gpt_karpathy();
    else if (name == "gpt_1024") *cfg = ModelConfig::gpt_1024();
    else if (name == "target_600m") *cfg = ModelConfig::target_600m();
    else if (name == "target_800m") *cfg = ModelConfig::target_800m();
    else if (name == "target_1b") *cfg = ModelConfig::target_1b();
    else if (name == "target_1_5b") *cfg = ModelConfig::target_1_5b();
    else if (name == "bench_tiny") *cfg = ModelConfig::bench_tiny();
    else if (name == "bench_600m") *cfg = ModelConfig::bench_600m();
    else if (name == "bench_5b") *cfg = ModelConfig::bench_5b();
    else if (name.rfind("custom:", 0) == 0) {            // bin/train.rs:669-690 custom:dim,hidden,nlayers,seq
        std::vector<uint32_t> v = parse_ids(name.substr(7));
        if (v.size() < 4) return false;
        size_t heads = v.size() > 4 ? v[4] : v[0] / 128, hd = v.size() > 5 ? v[5] : 128, vocab = v.size() > 6 ? v[6] : 8192;
        if (!heads) return false;
        *cfg = ModelConfig::make(v[0], v[1], heads, heads, hd, v[3], v[2], vocab);
    } else return false;
    return true;
}

std::string format_ids(const std::vector<uint32_t> &ids) {
    std::string s;
    for (size_t i = 0; i < ids.size(); ++i) { if (i) s += ","; s += std::to_string(ids[i]); }
    return s;
}

}  // namespace

int main(int argc, char **argv) {
    std::string model = "gpt_1024", checkpoint, prompt_ids_raw, wdt = "f32", kvdt = "f32";
    GenerationRequest req;
    float softcap = 0.0f, weight_std = 0.02f;
    uint64_t weight_seed = 1234;
    size_t random_prompt = 0;
    bool jsonl_session = false;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        auto val = [&]() -> std::string { if (i + 1 >= argc) fail(a + " needs a value"); return argv[++i]; };
        if (a == "--model") model = val();
        else if (a == "--checkpoint") checkpoint = val();                               // generate.rs:165-167
        else if (a == "--prompt-ids") prompt_ids_raw = val();
        else if (a == "--random-prompt") random_prompt = strtoull(val().c_str(), nullptr, 10);
        else if (a == "--steps") req.steps = strtoull(val().c_str(), nullptr, 10);
        else if (a == "--temperature") req.temperature = strtof(val().c_str(), nullptr);
        else if (a == "--top-k") req.top_k = strtoull(val().c_str(), nullptr, 10);
        else if (a == "--softcap") softcap = strtof(val().c_str(), nullptr);
        else if (a == "--samples") req.samples = strtoull(val().c_str(), nullptr, 10);
        else if (a == "--seed") req.seed = strtoull(val().c_str(), nullptr, 10);
        else if (a == "--weight-seed") weight_seed = strtoull(val().c_str(), nullptr, 10);
        else if (a == "--weight-std") weight_std = strtof(val().c_str(), nullptr);
        else if (a == "--weight-dtype") wdt = val();
        else if (a == "--kv-dtype") kvdt = val();
        else if (a == "--jsonl-session") jsonl_session = true;                          // generate.rs:236-238
        else if (a == "--kv-cache") req.decode_backend = DecodeBackendRequest::Hip;     // generate.rs:189-192
        else if (a == "--decode-backend") {
            std::string raw = val();
            if (!parse_decode_backend(raw, &req.decode_backend))
                fail("--decode-backend must be one of: auto, naive, hip; got " + raw);
        } else if (a == "--help" || a == "-h") { usage(); return 0; }
        else if (a == "--prompt" || a == "--tokenizer" || a == "--add-special-tokens" || a == "--no-skip-special-tokens")
            // generate.rs:173-188: text goes through the tokenizers crate there; this engine works on ids
            fail(a + " needs a tokenizer, which this build does not carry: pass the prompt as --prompt-ids");
        else fail("unknown argument " + a);
    }
    if (req.samples == 0) fail("samples must be >= 1");
    ModelConfig cfg;
    Checkpoint ckpt;
    if (!checkpoint.empty()) {
        std::string cerr;
        if (!load_checkpoint(checkpoint, &ckpt, &cerr)) fail("failed to load checkpoint: " + cerr);   // generate.rs:495
        cfg = ckpt.cfg;
        model = checkpoint;
        if (!jsonl_session)                                                              // generate.rs:523 (stdout carries only answers)
            printf("loaded checkpoint: step=%u model=%zuL %zuD %zuH %zuV seq=%zu\n", ckpt.step, cfg.nlayers, cfg.dim, cfg.hidden,
               cfg.vocab, cfg.seq);                                                       // generate.rs:526
    } else if (!model_from_name(model, &cfg)) fail("unknown --model " + model);
    SessionOptions opts;
    if (wdt == "f32") opts.weight_dtype = WeightDtype::F32;
    else if (wdt == "bf16") opts.weight_dtype = WeightDtype::BF16;
    else if (wdt == "fp8") opts.weight_dtype = WeightDtype::FP8_E4M3;
    else if (wdt == "int4") opts.weight_dtype = WeightDtype::INT4_G128;
    else fail("--weight-dtype must be one of: f32, bf16, fp8, int4");
    if (kvdt == "f32") opts.kv_dtype = KvDtype::F32;
    else if (kvdt == "bf16") opts.kv_dtype = KvDtype::BF16;
    else fail("--kv-dtype must be f32 or bf16");

    std::vector<uint32_t> prompt = parse_ids(prompt_ids_raw);
    if (prompt.empty() && random_prompt) {
        prompt.resize(random_prompt);
        rs_synth_prompt(7, (uint32_t)cfg.vocab, random_prompt, prompt.data());
    }
    if (prompt.empty()) fail("pass --prompt-ids or --random-prompt");

    if (!jsonl_session)
        printf("model=%s dim=%zu hidden=%zu heads=%zu hd=%zu nlayers=%zu seq=%zu vocab=%zu params=%zu\n", model.c_str(),
               cfg.dim, cfg.hidden, cfg.heads, cfg.hd, cfg.nlayers, cfg.seq, cfg.vocab, cfg.param_count());
    DecodeSelection planned = select_decode_mode(cfg, req.decode_backend, prompt.size() < cfg.seq ? prompt.size() : cfg.seq,
                                                 req.steps);
    if (!jsonl_session) {
        printf("decode_backend_request=%s decode_mode=%s", decode_backend_str(req.decode_backend), decode_mode_str(planned.mode));
        if (planned.fallback_reason) printf(" fallback_reason=%s", planned.fallback_reason);
        if (planned.auto_reason) printf(" auto_reason=%s", planned.auto_reason);
        printf("\n");
    }

    ModelWeights weights = checkpoint.empty()
                               ? ModelWeights::synthetic(cfg, weight_seed, weight_std, opts.weight_dtype != WeightDtype::F32)
                               : std::move(ckpt.weights);
    std::string err;
    InferenceSession session(cfg, weights, prompt, softcap, opts, &err);
    if (!session.ok()) fail(err);
    if (jsonl_session) {                                                                 // generate.rs:571-588
        fprintf(stderr, "jsonl_session_ready checkpoint_step=%u prompt_len=%zu decode_backend_default=%s\n", ckpt.step,
                prompt.size(), decode_backend_str(req.decode_backend));
        run_jsonl_session(stdin, stdout, req, prompt, &session);
        return 0;
    }
    GenerationBatch batch;
    if (!session.generate(req, &batch, &err)) fail(err);

    const double prefill_tps = batch.prefill_elapsed > 0 ? (double)session.prompt_len() / batch.prefill_elapsed : 0.0;
    const size_t decode_steps = req.steps ? req.steps - 1 : 0;                                       // generate.rs:612
    const double total_tps = batch.total_elapsed > 0 ? (double)(req.steps * req.samples) / batch.total_elapsed : 0.0;
    printf("prompt_ids=%s\n", format_ids(prompt).c_str());
    for (size_t i = 0; i < batch.results.size(); ++i) {
        const SampleResult &r = batch.results[i];
        if (req.samples > 1) printf("sample=%zu seed=%llu\n", i, (unsigned long long)r.seed);
        printf("generated_ids=%s\n", format_ids(r.sampled).c_str());
        printf("full_sequence=%s\n", format_ids(r.generated).c_str());
        printf("decode_steps=%zu decode_time=%.2fms decode_tok/s=%.2f\n", decode_steps, r.decode_elapsed * 1e3,
               decode_steps && r.decode_elapsed > 0 ? (double)decode_steps / r.decode_elapsed : 0.0);
    }
    printf("prefill_time=%.2fms prefill_tok/s=%.2f\n", batch.prefill_elapsed * 1e3, prefill_tps);
    printf("total_generation_time=%.2fms overall_tok/s=%.2f\n", batch.total_elapsed * 1e3, total_tps);
    return 0;
}
