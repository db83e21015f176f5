#include "synth.h"

#include <string.h>

static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline uint32_t lanes16(uint64_t h) {
    return (uint32_t)(h & 0xffff) + (uint32_t)((h >> 16) & 0xffff) + (uint32_t)((h >> 32) & 0xffff) +
           (uint32_t)(h >> 48);
}

static inline float bf16_rne(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&f, &u, 4);
    return f;
}

extern "C" void rs_synth_normal(uint64_t seed, uint64_t tensor_id, size_t n, float std, int round_bf16, float *out) {
    const uint64_t key = splitmix64(seed ^ splitmix64(tensor_id));
    // sum of twelve uniforms on 0..65535: mean 12*32767.5, variance 65536^2 - 1
    const double scale = (double)std / 65535.99999237060546875;   // sqrt(65536^2 - 1) to double precision
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        uint64_t c = key + 3ull * (uint64_t)i;
        uint32_t s = lanes16(splitmix64(c)) + lanes16(splitmix64(c + 1)) + lanes16(splitmix64(c + 2));
        float v = (float)(((double)s - 393210.0) * scale);
        out[i] = round_bf16 ? bf16_rne(v) : v;
    }
}

extern "C" void rs_synth_prompt(uint64_t seed, uint32_t vocab, size_t n, uint32_t *out) {
    uint64_t s = seed;
    for (size_t i = 0; i < n; ++i) {
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        out[i] = (uint32_t)((s >> 33) % vocab);
    }
}
