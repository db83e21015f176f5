// Model configuration and weights as the engine sees them
// (crates/engine/src/model.rs:28-41, :182-187; crates/engine/src/full_model.rs:19-23;
// crates/engine/src/layer.rs:19-36).
#pragma once
#include <stddef.h>
#include <stdint.h>

#include <string>
#include <memory>
#include <vector>

namespace rustane {

enum class FfnActivation : uint32_t { SwiGlu = 0, LeakyReluSq = 1 };   // model.rs:3-7, checkpoint codes :10-24

struct ModelConfig {
    size_t dim = 0, hidden = 0, heads = 0, kv_heads = 0, hd = 0, seq = 0, nlayers = 0, vocab = 0;
    size_t q_dim = 0, kv_dim = 0, gqa_ratio = 1;
    FfnActivation ffn_activation = FfnActivation::SwiGlu;

    static ModelConfig make(size_t dim, size_t hidden, size_t heads, size_t kv_heads, size_t hd, size_t seq,
                            size_t nlayers, size_t vocab, FfnActivation act = FfnActivation::SwiGlu) {
        ModelConfig c;
        c.dim = dim; c.hidden = hidden; c.heads = heads; c.kv_heads = kv_heads; c.hd = hd; c.seq = seq;
        c.nlayers = nlayers; c.vocab = vocab; c.q_dim = heads * hd; c.kv_dim = kv_heads * hd;
        c.gqa_ratio = kv_heads ? heads / kv_heads : 1; c.ffn_activation = act;
        return c;
    }
    // presets of model.rs:45-226
    static ModelConfig gpt_karpathy() { return make(768, 2048, 6, 6, 128, 512, 6, 8192); }
    static ModelConfig gpt_karpathy_gqa() { return make(768, 2048, 6, 3, 128, 512, 6, 8192); }
    static ModelConfig gpt_1024() { return make(1024, 2816, 8, 8, 128, 512, 8, 8192); }
    static ModelConfig target_600m() { return make(1536, 4096, 12, 12, 128, 512, 20, 8192); }
    static ModelConfig target_800m() { return make(1792, 4864, 14, 14, 128, 512, 24, 8192); }
    static ModelConfig target_1b() { return make(2048, 5632, 16, 16, 128, 512, 28, 8192); }
    static ModelConfig target_1_5b() { return make(2304, 6144, 18, 18, 128, 512, 32, 8192); }
    // the benchmark configurations of this build
    static ModelConfig bench_tiny() { return make(512, 1536, 8, 8, 64, 512, 8, 8192); }
    static ModelConfig bench_600m() { return make(1536, 4096, 12, 12, 128, 2048, 24, 32768); }
    static ModelConfig bench_5b() { return make(4096, 11008, 32, 32, 128, 4096, 32, 32768); }

    // model.rs:182-187
    size_t param_count() const {
        const size_t per_layer = 4 * dim * dim + 3 * dim * hidden;
        return nlayers * per_layer + vocab * dim + dim * (2 * nlayers + 1);
    }
};

// layer.rs:19-36 (forward weights only; the reference's *t transposes are backward-only)
struct LayerWeights {
    std::vector<float> wq, wk, wv, wo, w1, w3, w2, gamma1, gamma2;
};
enum class WeightDtype : uint32_t { F32 = 0, BF16 = 1, FP8_E4M3 = 2, INT4_G128 = 3 };
enum class KvDtype : uint32_t { F32 = 0, BF16 = 1 };

// Weights as the decode library stores them on the device (converted ahead of time, checkpoint.h): per layer
// the fused q/k/v, wo, interleaved gate/up and w2 matrices in the weight format, their scales, the norm gains.
struct PackedLayer {
    std::vector<uint8_t> wqkv, wo, w13, w2, s_qkv, s_wo, s_w13, s_w2;
    std::vector<float> gamma1, gamma2;
};
struct PackedWeights {
    WeightDtype dtype = WeightDtype::F32;
    std::vector<PackedLayer> layers;
    std::vector<float> gamma_final;
    std::vector<uint8_t> embed;              // fp32 with fp32 weights, bf16 otherwise
};

// full_model.rs:19-23
struct ModelWeights {
    std::vector<float> embed, gamma_final;
    std::vector<LayerWeights> layers;
    // set instead of the fp32 tensors above by a checkpoint that was converted ahead of time
    std::shared_ptr<const PackedWeights> packed;

    // every matrix N(0, std) from the counter-based generator, norm gains 1
    static ModelWeights synthetic(const ModelConfig &cfg, uint64_t seed, float std, bool round_bf16);
};

}  // namespace rustane
