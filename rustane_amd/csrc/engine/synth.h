// Deterministic synthetic weights and prompts for the benchmark configurations.
//
// The reference initialises test weights with a 64-bit LCG (engine/src/layer.rs:806-817) whose
// wo / w2 are zero; the benchmark configurations instead ask for N(0, 0.02) in every matrix.
// This generator is counter based -- element i of tensor t under seed s depends on (s, t, i)
// only -- uses integer arithmetic plus one double multiply, and therefore produces the same bits
// on every host, thread count and compiler.
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// Tensor ids: 0 embed, 1 gamma_final; per layer l: 16*(l+1) + {0 wq, 1 wk, 2 wv, 3 wo, 4 w1, 5 w3, 6 w2}.
#define RS_TENSOR_EMBED 0ull
#define RS_TENSOR_LAYER(l, k) (16ull * ((uint64_t)(l) + 1ull) + (uint64_t)(k))

// out[i] = std * z_i, z_i an Irwin-Hall(12) approximation of N(0,1) built from twelve 16-bit
// uniforms; when round_bf16 is non-zero every value is rounded to the nearest-even bf16 and
// stored as that fp32 value.
void rs_synth_normal(uint64_t seed, uint64_t tensor_id, size_t n, float std, int round_bf16, float *out);

// Uniform token ids in [0, vocab) from the reference's LCG (engine/src/inference.rs:759-764):
// id = (next_u64 >> 33) % vocab.
void rs_synth_prompt(uint64_t seed, uint32_t vocab, size_t n, uint32_t *out);

#ifdef __cplusplus
}
#endif
