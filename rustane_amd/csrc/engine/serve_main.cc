// `serve`: the reference's HTTP inference server (crates/engine/src/bin/serve.rs:473-561 flags,
// :1247-1281 main) over the HIP decode backend: a checkpoint (or a synthetic model of a named shape)
// is loaded once, requests are answered one at a time out of a cache of prefix-sharing sessions.
#include <signal.h>
#include <stdio.h>
#include <stdlib.h>

#include <string>

#include "checkpoint.h"
#include "cli_common.h"
#include "http_server.h"
#include "session_cache.h"

using namespace rustane;
using namespace rustane::cli;

namespace {

void usage(FILE *f) {
    fprintf(f, "Usage: serve (--checkpoint PATH | --model <preset|custom:dim,hidden,nlayers,seq[,heads,hd,vocab]>) [--bind HOST:PORT]\n"
               "  [--model-name NAME] [--decode-backend auto|naive|hip] [--softcap S] [--max-cache-sessions N]\n"
               "  [--weight-dtype f32|bf16|fp8|int4] [--kv-dtype f32|bf16] [--weight-seed S] [--weight-std X]\n"
               "presets: %s\n", kPresets);
}

}  // namespace

int main(int argc, char **argv) {
    std::string checkpoint, model, bind = "127.0.0.1:8080", model_name = "rustane", wdt = "f32", kvdt = "f32";
    DecodeBackendRequest backend = DecodeBackendRequest::Auto;
    float softcap = 0.0f, weight_std = 0.02f;
    uint64_t weight_seed = 1234;
    size_t max_cache_sessions = 32;
    bool wdt_given = false;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        auto val = [&]() -> std::string { if (i + 1 >= argc) fail(a + " needs a value"); return argv[++i]; };
        auto count = [&](const char *what) -> size_t {
            const std::string v = val();
            if (v.empty() || v.find_first_not_of("0123456789") != std::string::npos) fail(a + " must be " + what);
            return strtoull(v.c_str(), nullptr, 10);
        };
        if (a == "--checkpoint") checkpoint = val();
        else if (a == "--model") model = val();
        else if (a == "--bind") bind = val();
        else if (a == "--model-name") model_name = val();
        else if (a == "--decode-backend") {
            const std::string raw = val();
            if (!parse_decode_backend(raw, &backend)) fail(decode_backend_error("--decode-backend", raw));
        } else if (a == "--softcap") softcap = strtof(val().c_str(), nullptr);
        else if (a == "--max-cache-sessions") max_cache_sessions = count("an integer");
        else if (a == "--weight-dtype") { wdt = val(); wdt_given = true; }
        else if (a == "--kv-dtype") kvdt = val();
        else if (a == "--weight-seed") weight_seed = count("an integer");
        else if (a == "--weight-std") weight_std = strtof(val().c_str(), nullptr);
        else if (a == "--tokenizer" || a == "--add-special-tokens" || a == "--no-skip-special-tokens")
            // serve.rs:492-495, :515-522: text goes through the tokenizers crate there; this engine works on ids
            fail(a + " needs a tokenizer, which this build does not carry: requests pass token ids");
        else if (a == "--help" || a == "-h") { usage(stdout); return 0; }
        else {
            fprintf(stderr, "Unknown arg: %s\n", a.c_str());
            usage(stderr);
            return 1;
        }
    }
    if (checkpoint.empty() && model.empty()) {
        fprintf(stderr, "--checkpoint required (or --model for synthetic weights)\n");
        usage(stderr);
        return 1;
    }
    ModelConfig cfg;
    Checkpoint ckpt;
    SessionOptions opts;
    parse_formats(wdt, kvdt, &opts);
    if (!checkpoint.empty()) {
        std::string cerr;
        if (!load_checkpoint(checkpoint, &ckpt, &cerr)) fail("failed to load checkpoint: " + cerr);
        cfg = ckpt.cfg;
        if (ckpt.weights.packed) {               // a checkpoint converted ahead of time carries its weight format
            if (!wdt_given) opts.weight_dtype = ckpt.weights.packed->dtype;
            else if (opts.weight_dtype != ckpt.weights.packed->dtype)
                fail("--weight-dtype " + wdt + " does not match the format this converted checkpoint holds");
        }
    } else if (!model_from_name(model, &cfg)) fail("unknown --model " + model);
    const ModelWeights weights = checkpoint.empty()
                                     ? ModelWeights::synthetic(cfg, weight_seed, weight_std, opts.weight_dtype != WeightDtype::F32)
                                     : std::move(ckpt.weights);

    signal(SIGPIPE, SIG_IGN);              // a client that goes away mid-answer is an error return, not the end of the server
    SessionCache cache(cfg, weights, softcap, max_cache_sessions, opts);
    HttpServer server(cfg, &cache, model_name, backend);
    std::string err;
    if (!server.listen_and_serve(bind, &err)) fail(err);
    return 0;
}
