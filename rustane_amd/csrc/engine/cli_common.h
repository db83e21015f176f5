// What the command-line programs (`generate`, `serve`) share: error exit, id lists, model presets,
// weight / cache formats by name.
#pragma once
#include <stdio.h>
#include <stdlib.h>

#include <string>
#include <vector>

#include "inference.h"

namespace rustane {
namespace cli {

[[noreturn]] inline void fail(const std::string &msg) {
    fprintf(stderr, "error: %s\n", msg.c_str());
    exit(2);
}

inline std::vector<uint32_t> parse_ids(const std::string &s) {
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

inline bool model_from_name(const std::string &name, ModelConfig *cfg) {
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

// --weight-dtype / --kv-dtype
inline void parse_formats(const std::string &wdt, const std::string &kvdt, SessionOptions *opts) {
    if (wdt == "f32") opts->weight_dtype = WeightDtype::F32;
    else if (wdt == "bf16") opts->weight_dtype = WeightDtype::BF16;
    else if (wdt == "fp8") opts->weight_dtype = WeightDtype::FP8_E4M3;
    else if (wdt == "int4") opts->weight_dtype = WeightDtype::INT4_G128;
    else fail("--weight-dtype must be one of: f32, bf16, fp8, int4");
    if (kvdt == "f32") opts->kv_dtype = KvDtype::F32;
    else if (kvdt == "bf16") opts->kv_dtype = KvDtype::BF16;
    else fail("--kv-dtype must be f32 or bf16");
}

inline const char *kPresets = "gpt_karpathy gpt_1024 target_600m target_800m target_1b target_1_5b bench_tiny bench_600m bench_5b";

}  // namespace cli
}  // namespace rustane
