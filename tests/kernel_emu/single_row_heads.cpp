// The single-row head kernels (kernels_heads.inc: k_head_argmax, k_head_topk, k_head_block_stats and k_softcap_copy,
// cut out of hipdec_kernels.h by the test, and the multi-row k_bd_block_stats of hipdec_batch.h) run on the CPU against
// the oracle's restatements (oracle/rustane_oracle.c, linked in as the checker): greedy token with the step state
// advanced, per-block top-k lists exactly, per-block softmax statistics and the softcapped block copy.
#include "emu.h"
#include "kernels_heads.inc"
#include <cstdio>
#include <random>

extern "C" void orc_block_topk(const float *logits, int V, int top_k, float *out_vals, uint32_t *out_idxs);
extern "C" void orc_block_stats(const float *raw_logits, int V, float inv_temperature, float softcap, float *maxes, float *sums);

static std::mt19937 rng32(31);
static int failures = 0;

static void heads_case(int V, int top_k, float temperature, float softcap) {
    const int blocks = (V + 255) / 256;
    float *logits = (float *)std::malloc((size_t)V * 4);
    for (int i = 0; i < V; ++i) { const unsigned u = rng32(); logits[i] = (u % 17 == 0) ? -INFINITY : (float)((int)(u % 61) - 30) * 0.25f; }
    if (V > 600) for (int i = 256; i < 512; ++i) logits[i] = -INFINITY;                  // a block of nothing
    StepParams *sp = (StepParams *)std::calloc(1, sizeof(StepParams));
    *sp = StepParams{7, 11, 2, top_k, 1.0f / temperature, softcap, 0, 0};
    uint32_t *ring = (uint32_t *)std::calloc(4, 4);
    float *vals = (float *)std::malloc((size_t)blocks * top_k * 4), *maxes = (float *)std::malloc((size_t)blocks * 4), *sums = (float *)std::malloc((size_t)blocks * 4);
    float *bmax = (float *)std::malloc((size_t)blocks * 4), *bsum = (float *)std::malloc((size_t)blocks * 4);
    uint32_t *idxs = (uint32_t *)std::malloc((size_t)blocks * top_k * 4);
    BatchParams *bp = (BatchParams *)std::calloc(1, sizeof(BatchParams));
    *bp = BatchParams{0, 0, 0, top_k, 1.0f / temperature, softcap};
    emu::launch_fn([&] { k_head_topk(logits, V, sp, vals, idxs); }, dim3{(unsigned)blocks, 1, 1}, 256, 0);
    emu::launch_fn([&] { k_head_block_stats(logits, V, sp, maxes, sums); }, dim3{(unsigned)blocks, 1, 1}, 256, 0);
    emu::launch_fn([&] { k_bd_block_stats(logits, V, bp, bmax, bsum); }, dim3{(unsigned)blocks, 1, 1}, 256, 0);
    const int start = 256 * (blocks - 1), n = V - start;
    float *copy = (float *)std::malloc((size_t)n * 4);
    emu::launch_fn([&] { k_softcap_copy(logits, copy, start, n, softcap); }, dim3{(unsigned)((n + 255) / 256), 1, 1}, 256, 0);
    emu::launch_fn([&] { k_head_argmax(logits, V, sp, ring, 4); }, dim3{1, 1, 1}, 1024, 0);
    long bad = 0;
    double worst = 0;
    uint32_t best = 0;
    for (int i = 1; i < V; ++i) if (logits[i] > logits[best]) best = (uint32_t)i;          // the first of the largest
    if ((uint32_t)sp->tok != best || ring[2] != best || sp->pos != 12 || sp->step != 3) ++bad;
    std::vector<float> rv((size_t)blocks * top_k), rm(blocks), rs(blocks);
    std::vector<uint32_t> ri((size_t)blocks * top_k);
    orc_block_topk(logits, V, top_k, rv.data(), ri.data());
    for (size_t i = 0; i < rv.size(); ++i) if (!(vals[i] == rv[i]) || idxs[i] != ri[i]) ++bad;
    orc_block_stats(logits, V, 1.0f / temperature, softcap, rm.data(), rs.data());
    for (int b = 0; b < blocks; ++b) {
        if (!(maxes[b] == rm[b]) || !(bmax[b] == rm[b])) ++bad;                             // (also -inf == -inf)
        worst = std::fmax(worst, std::fmax(std::fabs(sums[b] - rs[b]), std::fabs(bsum[b] - rs[b])) / (1.0 + std::fabs(rs[b])));
    }
    for (int i = 0; i < n; ++i) { const float x = logits[start + i], want = softcap > 0.0f ? softcap * tanhf(x / softcap) : x; if (!(copy[i] == want)) ++bad; }
    const bool ok = bad == 0 && worst <= 1e-5;
    std::printf("single-row heads vocabulary %d k %d temperature %g softcap %g: %ld mismatches, block sums within %.3g (allowed 1e-5)%s\n", V, top_k, temperature,
                softcap, bad, worst, ok ? "" : "  FAIL");
    if (!ok) ++failures;
    std::free(logits); std::free(sp); std::free(ring); std::free(vals); std::free(maxes); std::free(sums); std::free(bmax); std::free(bsum); std::free(idxs); std::free(bp); std::free(copy);
}

int main() {
    heads_case(1000, 8, 0.8f, 0.0f);
    heads_case(256, 1, 1.0f, 30.0f);
    heads_case(70, 32, 1.3f, 0.0f);
    heads_case(2500, 5, 0.7f, 15.0f);
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
