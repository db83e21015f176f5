// The multi-row step's greedy and top-k head kernels (kernels_sel.inc: their own source, cut out of hipdec_batch.h
// and hipdec_common.h by the test) run on the CPU against a sort by the reference's ordering (value descending, index
// ascending), on logits with ties, -inf entries and vocabularies that end inside a block of 256.
#include "emu.h"
#include "kernels_sel.inc"
#include <algorithm>
#include <cstdio>
#include <random>

static std::mt19937 rng(3);
static int failures = 0;

static void selection_case(int R, int V, int top_k) {
    const int blocks = (V + 255) / 256;
    float *logits = (float *)std::malloc((size_t)R * V * 4);
    for (size_t i = 0; i < (size_t)R * V; ++i) {
        const unsigned u = rng();
        logits[i] = (u % 17 == 0) ? -INFINITY : (float)((int)(u % 41) - 20) * 0.25f;      // few distinct values: many ties
    }
    if (V > 300) for (int r = 0; r < R; ++r) for (int i = 256; i < std::min(V, 512); ++i) logits[(size_t)r * V + i] = -INFINITY;   // a block of nothing
    uint32_t *tok = (uint32_t *)std::malloc((size_t)R * 4);
    float *vals = (float *)std::malloc((size_t)R * blocks * top_k * 4);
    uint32_t *idxs = (uint32_t *)std::malloc((size_t)R * blocks * top_k * 4);
    BatchParams *bp = (BatchParams *)std::malloc(sizeof(BatchParams));
    *bp = BatchParams{0, 0, 0, top_k, 1.0f, 0.0f};
    emu::launch_fn([&] { k_bd_argmax(logits, V, tok); }, dim3{(unsigned)R, 1, 1}, 1024, 0);
    emu::launch_fn([&] { k_bd_topk(logits, V, bp, vals, idxs); }, dim3{(unsigned)blocks, (unsigned)R, 1}, 256, 0);
    long bad = 0;
    for (int r = 0; r < R; ++r) {
        const float *lg = logits + (size_t)r * V;
        std::vector<uint32_t> order(V);
        for (int i = 0; i < V; ++i) order[i] = (uint32_t)i;
        auto before = [&](uint32_t a, uint32_t b) { return lg[a] > lg[b] || (lg[a] == lg[b] && a < b); };
        if (tok[r] != *std::min_element(order.begin(), order.end(), before)) ++bad;
        for (int b = 0; b < blocks; ++b) {
            std::vector<uint32_t> in(order.begin() + b * 256, order.begin() + std::min(V, (b + 1) * 256));
            std::sort(in.begin(), in.end(), before);
            for (int k = 0; k < top_k; ++k) {
                const size_t o = ((size_t)r * blocks + b) * top_k + k;
                const float want_v = k < (int)in.size() ? lg[in[k]] : -INFINITY;
                const uint32_t want_i = k < (int)in.size() ? in[k] : 0xffffffffu;
                if (!(vals[o] == want_v) || idxs[o] != want_i) ++bad;
            }
        }
    }
    std::printf("k_bd_argmax / k_bd_topk rows %d vocabulary %d k %d: %ld mismatches%s\n", R, V, top_k, bad, bad ? "  FAIL" : "");
    if (bad) ++failures;
    std::free(logits); std::free(tok); std::free(vals); std::free(idxs); std::free(bp);
}

int main() {
    selection_case(3, 1000, 8);
    selection_case(2, 256, 1);
    selection_case(1, 70, 32);
    selection_case(2, 20, 32);        // fewer rows than k: the list is padded with (-inf, no index)
    selection_case(2, 2500, 5);
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
