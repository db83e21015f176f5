// `generate`: token-id generation over the HIP decode backend with the flags and report lines of
// the reference's CLI (crates/engine/src/bin/generate.rs:145-280 flags, :603-728 report).  Text
// tokenisation and checkpoint files are outside this build: prompts are token ids and weights are
// synthetic (seeded) for a named or custom shape.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <stdexcept>
#include <string>
#include <vector>

#include "checkpoint.h"
#include "cli_common.h"
#include "decode_context.h"
#include "inference.h"
#include "jsonl_session.h"
#include "synth.h"

using namespace rustane;
using namespace rustane::cli;

namespace {

void usage() {
    printf("usage: generate (--checkpoint PATH | --model <preset|custom:dim,hidden,nlayers,seq[,heads,hd,vocab]>) --prompt-ids 1,2,3\n"
           "  [--steps N] [--temperature T] [--top-k K] [--softcap C] [--samples N] [--seed S]\n"
           "  [--decode-backend auto|naive|hip] [--kv-cache] [--weight-dtype f32|bf16|fp8|int4] [--kv-dtype f32|bf16]\n"
           "  [--weight-seed S] [--weight-std X] [--random-prompt N] [--jsonl-session]\n"
           "  [--convert-to OUT: write the model's weights in the --weight-dtype format as a converted checkpoint and exit]\n"
           "presets: %s\n", kPresets);
}

// a float as the reference's "{}" prints it: the shortest decimal that reads back as the same f32, never an exponent
std::string format_f32(float v) {
    char buf[64];
    for (int p = 1; p <= 9; ++p) {
        snprintf(buf, sizeof buf, "%.*g", p, (double)v);
        if (strtof(buf, nullptr) == v) break;
    }
    if (strchr(buf, 'e') || strchr(buf, 'E')) {
        snprintf(buf, sizeof buf, "%.12f", (double)v);
        size_t n = strlen(buf);
        while (n > 1 && buf[n - 1] == '0') buf[--n] = 0;
        if (n > 1 && buf[n - 1] == '.') buf[--n] = 0;
    }
    return buf;
}

std::string format_ids(const std::vector<uint32_t> &ids) {
    std::string s;
    for (size_t i = 0; i < ids.size(); ++i) { if (i) s += ","; s += std::to_string(ids[i]); }
    return s;
}

}  // namespace

int main(int argc, char **argv) {
    std::string model = "gpt_1024", checkpoint, prompt_ids_raw, wdt = "f32", kvdt = "f32", convert_to;
    bool wdt_given = false;
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
        else if (a == "--weight-dtype") { wdt = val(); wdt_given = true; }
        else if (a == "--convert-to") convert_to = val();
        else if (a == "--kv-dtype") kvdt = val();
        else if (a == "--jsonl-session") jsonl_session = true;                          // generate.rs:236-238
        else if (a == "--kv-cache") req.decode_backend = DecodeBackendRequest::Hip;     // generate.rs:189-192
        else if (a == "--decode-backend") {
            std::string raw = val();
            if (!parse_decode_backend(raw, &req.decode_backend))
                fail(decode_backend_error("--decode-backend", raw));
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
    parse_formats(wdt, kvdt, &opts);
    if (ckpt.weights.packed) {
        // a checkpoint converted ahead of time carries its weight format
        if (!wdt_given) opts.weight_dtype = ckpt.weights.packed->dtype;
        else if (opts.weight_dtype != ckpt.weights.packed->dtype)
            fail("--weight-dtype " + wdt + " does not match the format this converted checkpoint holds");
    }
    if (!convert_to.empty()) {
        // offline conversion: build the model once in the asked weight format, write its stored weights
        if (ckpt.weights.packed) fail("--convert-to needs the fp32 checkpoint, this one is converted already");
        try {
            const ModelWeights src = checkpoint.empty()
                                         ? ModelWeights::synthetic(cfg, weight_seed, weight_std, opts.weight_dtype != WeightDtype::F32)
                                         : std::move(ckpt.weights);
            DecodeContext ctx(cfg, src, opts.weight_dtype, KvDtype::F32, 0, 0);
            PackedWeights packed;
            ctx.export_packed(cfg, opts.weight_dtype, &packed);
            std::string werr;
            if (!write_packed_checkpoint(convert_to, cfg, packed, ckpt.step, &werr)) fail(werr);
        } catch (const std::exception &e) {
            fail(e.what());
        }
        printf("converted_checkpoint=%s weight_dtype=%s step=%u\n", convert_to.c_str(), wdt.c_str(), ckpt.step);
        return 0;
    }

    std::vector<uint32_t> prompt = parse_ids(prompt_ids_raw);
    if (prompt.empty() && random_prompt) {
        prompt.resize(random_prompt);
        rs_synth_prompt(7, (uint32_t)cfg.vocab, random_prompt, prompt.data());
    }
    if (prompt.empty()) fail("pass --prompt-ids or --random-prompt");

    if (!jsonl_session && checkpoint.empty())        // (a synthetic model has no "loaded checkpoint" line: its shape instead)
        printf("model=%s dim=%zu hidden=%zu heads=%zu hd=%zu nlayers=%zu seq=%zu vocab=%zu params=%zu\n", model.c_str(),
               cfg.dim, cfg.hidden, cfg.heads, cfg.hd, cfg.nlayers, cfg.seq, cfg.vocab, cfg.param_count());
    const size_t effective_context_len = prompt.size() < cfg.seq ? prompt.size() : cfg.seq;         // generate.rs:519
    DecodeSelection planned = select_decode_mode(cfg, req.decode_backend, effective_context_len, req.steps);
    const bool greedy_sampling = req.temperature <= 0.0f || req.top_k == 1;                          // generate.rs:522
    if (!jsonl_session) {                                                                            // generate.rs:524-566
        printf("prompt_len=%zu effective_context_len=%zu steps=%zu temperature=%s top_k=%zu decode_backend_request=%s "
               "decode_mode=%s greedy_sampling=%s\n",
               prompt.size(), effective_context_len, req.steps, format_f32(req.temperature).c_str(), req.top_k,
               decode_backend_str(req.decode_backend), decode_mode_str(planned.mode), greedy_sampling ? "true" : "false");
        if (prompt.size() > cfg.seq) printf("prompt_truncated=true kept_last_tokens=%zu\n", effective_context_len);
        if (planned.auto_reason)         // (the threshold keeps the reference's key: log readers look for it)
            printf("decode_backend_auto_reason=%s model_params=%zu auto_metal_threshold=%zu\n", planned.auto_reason,
                   cfg.param_count(), AUTO_KV_PARAM_THRESHOLD);
        if (planned.fallback_reason) printf("decode_backend_fallback=true reason=%s\n", planned.fallback_reason);
        printf("samples=%zu prefix_reuse=%s\n", req.samples, req.samples > 1 ? "enabled" : "disabled");
        if (planned.mode == DecodeMode::KvCacheHip && !greedy_sampling) {                            // generate.rs:312-333
            if (req.top_k > 0) {
                if (req.top_k <= MAX_GPU_TOPK)
                    printf("cached_sampling_path=gpu_topk_candidates top_k=%zu gpu_topk_capacity=%zu\n", req.top_k, MAX_GPU_TOPK);
                else
                    printf("cached_sampling_path=full_logits_cpu_sample reason=top_k_exceeds_gpu_capacity requested_top_k=%zu "
                           "gpu_topk_capacity=%zu\n", req.top_k, MAX_GPU_TOPK);
            } else {
                printf("cached_sampling_path=gpu_block_stats_exact\n");
            }
        }
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

    // generate.rs:609-728
    const double prefill_tps = batch.prefill_elapsed > 0 ? (double)session.prompt_len() / batch.prefill_elapsed : 0.0;
    const size_t decode_steps = req.steps ? req.steps - 1 : 0;
    const double avg_decode_tps = decode_steps > 0 && batch.avg_decode_elapsed > 0 ? (double)decode_steps / batch.avg_decode_elapsed : 0.0;
    const double total_tps = batch.total_elapsed > 0 ? (double)(req.steps * req.samples) / batch.total_elapsed : 0.0;
    auto sample_tps = [&](const SampleResult &r) {
        return decode_steps > 0 && r.decode_elapsed > 0 ? (double)decode_steps / r.decode_elapsed : 0.0;
    };
    printf("prompt_ids=%s\n", format_ids(prompt).c_str());
    if (req.samples == 1) {
        const SampleResult &r = batch.results[0];
        printf("generated_ids=%s\n", format_ids(r.sampled).c_str());
        printf("full_sequence=%s\n", format_ids(r.generated).c_str());
        printf("prefill_time=%.2fms prefill_tok/s=%.2f\n", batch.prefill_elapsed * 1e3, prefill_tps);
        printf("decode_steps=%zu decode_time=%.2fms decode_tok/s=%.2f\n", decode_steps, r.decode_elapsed * 1e3, sample_tps(r));
    } else {
        for (size_t i = 0; i < batch.results.size(); ++i) {
            const SampleResult &r = batch.results[i];
            printf("sample%zu_seed=%llu\n", i, (unsigned long long)r.seed);
            printf("sample%zu_generated_ids=%s\n", i, format_ids(r.sampled).c_str());
            printf("sample%zu_full_sequence=%s\n", i, format_ids(r.generated).c_str());
            printf("sample%zu_decode_steps=%zu sample%zu_decode_time=%.2fms sample%zu_decode_tok/s=%.2f\n", i, decode_steps, i,
                   r.decode_elapsed * 1e3, i, sample_tps(r));
        }
        printf("prefill_time=%.2fms prefill_tok/s=%.2f\n", batch.prefill_elapsed * 1e3, prefill_tps);
        printf("samples_decode_time_total=%.2fms samples_decode_time_avg=%.2fms avg_decode_tok/s=%.2f\n",
               batch.total_decode_elapsed * 1e3, batch.avg_decode_elapsed * 1e3, avg_decode_tps);
    }
    printf("total_generation_time=%.2fms overall_tok/s=%.2f\n", batch.total_elapsed * 1e3, total_tps);
    return 0;
}
