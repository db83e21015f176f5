// The full-vocabulary draw kernel (kernel_sample_fv.inc: k_sample_fullvocab with the restated host expf / tanhf and
// the run state, cut out of hipdec_sample.h by the test) run on the CPU: the block drawn from the per-block softmax
// statistics, then the token drawn inside the block, against the oracle's restatement of the reference's host code
// (oracle/rustane_oracle.c, linked in as the checker), token for token and RNG state for RNG state.
#include "emu.h"
#include "kernel_sample_fv.inc"
#include <cstdio>
#include <random>

extern "C" void orc_block_stats(const float *raw_logits, int V, float inv_temperature, float softcap, float *maxes, float *sums);
extern "C" size_t orc_sample_block_from_stats(const float *maxes, const float *sums, int B, uint64_t *rng);
extern "C" uint32_t orc_sample_block_logits(uint32_t base, const float *logits, int n, float temperature, uint64_t *rng);

static std::mt19937 rng32(29);
static int failures = 0;

static void draw_case(int rows, int V, float temperature, float softcap, int steps, int dead_blocks) {
    const int blocks = (V + 255) / 256;
    float *logits = (float *)std::malloc((size_t)rows * V * 4);
    float *maxes = (float *)std::malloc((size_t)rows * blocks * 4), *sums = (float *)std::malloc((size_t)rows * blocks * 4);
    uint64_t *rng = (uint64_t *)std::malloc((size_t)rows * 8), *rng_ref = (uint64_t *)std::malloc((size_t)rows * 8);
    uint32_t *tok = (uint32_t *)std::malloc((size_t)rows * 4), *ring = (uint32_t *)std::malloc((size_t)steps * rows * 4);
    SampleParams *ss = (SampleParams *)std::calloc(1, sizeof(SampleParams));
    *ss = SampleParams{temperature, softcap, 0, 0, steps, 0u};
    for (int r = 0; r < rows; ++r) rng[r] = rng_ref[r] = 0xd1342543de82ef95ull * (uint64_t)(r + 3) + rng32();
    long bad = 0;
    for (int step = 0; step < steps; ++step) {
        for (size_t i = 0; i < (size_t)rows * V; ++i) {
            const unsigned u = rng32();
            logits[i] = (u % 19 == 0) ? -INFINITY : (float)((int)(u % 2001) - 1000) * 0.01f;
        }
        for (int r = 0; r < rows; ++r)
            for (int b = 0; b < dead_blocks && b < blocks - 1; ++b)                       // blocks of nothing but -inf
                for (int i = 256 * (b + 1); i < std::min(V, 256 * (b + 2)); ++i) logits[(size_t)r * V + i] = -INFINITY;
        for (int r = 0; r < rows; ++r) orc_block_stats(logits + (size_t)r * V, V, 1.0f / temperature, softcap, maxes + (size_t)r * blocks, sums + (size_t)r * blocks);
        emu::launch_fn([&] { k_sample_fullvocab(logits, V, maxes, sums, blocks, ss, rng, tok, ring, nullptr); }, dim3{(unsigned)rows, 1, 1}, 256, 0);
        for (int r = 0; r < rows; ++r) {
            const size_t blk = orc_sample_block_from_stats(maxes + (size_t)r * blocks, sums + (size_t)r * blocks, blocks, &rng_ref[r]);
            const int start = (int)blk * 256, valid = std::min(256, V - start);
            std::vector<float> bl(valid);
            for (int i = 0; i < valid; ++i) { const float x = logits[(size_t)r * V + start + i]; bl[i] = softcap > 0.0f ? softcap * tanhf(x / softcap) : x; }
            const uint32_t want = orc_sample_block_logits((uint32_t)start, bl.data(), valid, temperature, &rng_ref[r]);
            if (tok[r] != want || rng[r] != rng_ref[r] || ring[(size_t)step * rows + r] != want) ++bad;
        }
        if (ss->step != step + 1 || ss->done != 0) ++bad;
    }
    std::printf("k_sample_fullvocab rows %d vocabulary %d temperature %g softcap %g steps %d: %ld mismatches%s\n", rows, V, temperature, softcap, steps, bad,
                bad ? "  FAIL" : "");
    if (bad) ++failures;
    std::free(logits); std::free(maxes); std::free(sums); std::free(rng); std::free(rng_ref); std::free(tok); std::free(ring); std::free(ss);
}

int main() {
    draw_case(3, 1000, 1.0f, 0.0f, 6, 0);
    draw_case(2, 2500, 0.7f, 30.0f, 4, 2);        // softcap, two blocks of nothing but -inf
    draw_case(1, 300, 1.5f, 0.0f, 5, 0);          // a last block that is not full
    draw_case(2, 70000, 1.0f, 15.0f, 2, 1);       // more blocks than threads
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
