// The top-k draw kernel (kernel_sample.inc: k_sample_topk with the restated host expf / tanhf and the run state, cut
// out of hipdec_sample.h by the test) run on the CPU: merged candidate list, softcap, draw and RNG state against the
// oracle's restatement of the reference's host code (oracle/rustane_oracle.c, linked in as the checker), token for
// token and state for state, over several rows, consecutive steps, ties, -inf logits, k above a block's valid rows.
#include "emu.h"
#include "kernel_sample.inc"
#include <cstdio>
#include <random>

extern "C" void orc_block_topk(const float *logits, int V, int top_k, float *out_vals, uint32_t *out_idxs);
extern "C" int orc_topk_candidates(const float *raw_logits, int V, int top_k, float softcap, uint32_t *out_idxs, float *out_vals);
extern "C" uint32_t orc_sample_topk_candidates(const uint32_t *idxs, const float *logits, int n, float temperature, uint64_t *rng);

static std::mt19937 rng32(23);
static int failures = 0;

static void draw_case(int rows, int V, int top_k, float temperature, float softcap, int steps) {
    const int blocks = (V + 255) / 256;
    float *logits = (float *)std::malloc((size_t)rows * V * 4);
    float *vals = (float *)std::malloc((size_t)rows * blocks * top_k * 4);
    uint32_t *idxs = (uint32_t *)std::malloc((size_t)rows * blocks * top_k * 4);
    uint64_t *rng = (uint64_t *)std::malloc((size_t)rows * 8), *rng_ref = (uint64_t *)std::malloc((size_t)rows * 8);
    uint32_t *tok = (uint32_t *)std::malloc((size_t)rows * 4), *ring = (uint32_t *)std::malloc((size_t)steps * rows * 4);
    SampleParams *ss = (SampleParams *)std::calloc(1, sizeof(SampleParams));
    BatchParams *bp = (BatchParams *)std::calloc(1, sizeof(BatchParams));
    *ss = SampleParams{temperature, softcap, top_k, 0, steps, 0u};
    *bp = BatchParams{40, 0, 40, top_k, 1.0f, softcap};
    for (int r = 0; r < rows; ++r) rng[r] = rng_ref[r] = 0x9e3779b97f4a7c15ull * (uint64_t)(r + 1) + rng32();
    long bad = 0;
    for (int step = 0; step < steps; ++step) {
        for (size_t i = 0; i < (size_t)rows * V; ++i) {
            const unsigned u = rng32();
            logits[i] = (u % 13 == 0) ? -INFINITY : (float)((int)(u % 1001) - 500) * 0.01f + (float)(u % 3);   // ties and -inf among them
        }
        for (int r = 0; r < rows; ++r) orc_block_topk(logits + (size_t)r * V, V, top_k, vals + (size_t)r * blocks * top_k, idxs + (size_t)r * blocks * top_k);
        emu::launch_fn([&] { k_sample_topk(vals, idxs, blocks, ss, rng, tok, ring, bp); }, dim3{(unsigned)rows, 1, 1}, 256, 0);
        for (int r = 0; r < rows; ++r) {
            std::vector<uint32_t> ci(top_k);
            std::vector<float> cv(top_k);
            const int n = orc_topk_candidates(logits + (size_t)r * V, V, top_k, softcap, ci.data(), cv.data());
            const uint32_t want = orc_sample_topk_candidates(ci.data(), cv.data(), n, temperature, &rng_ref[r]);
            if (tok[r] != want || rng[r] != rng_ref[r] || ring[(size_t)step * rows + r] != want) ++bad;
        }
        if (ss->step != step + 1 || ss->done != 0 || bp->pos != 41 + step || bp->slot != step + 1) ++bad;
    }
    std::printf("k_sample_topk rows %d vocabulary %d k %d temperature %g softcap %g steps %d: %ld mismatches%s\n", rows, V, top_k, temperature, softcap,
                steps, bad, bad ? "  FAIL" : "");
    if (bad) ++failures;
    std::free(logits); std::free(vals); std::free(idxs); std::free(rng); std::free(rng_ref); std::free(tok); std::free(ring); std::free(ss); std::free(bp);
}

int main() {
    draw_case(3, 1000, 8, 0.8f, 0.0f, 6);
    draw_case(2, 2500, 32, 1.3f, 30.0f, 4);       // softcap on the merged candidates
    draw_case(1, 300, 5, 0.0f, 0.0f, 3);          // temperature 0: the best candidate, the RNG untouched
    draw_case(2, 20, 32, 0.7f, 5.0f, 3);          // fewer rows than k: padded lists
    draw_case(4, 70000, 4, 1.0f, 0.0f, 2);        // more blocks than threads: a thread owns several lists
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
