// The single-row attention kernel of the one-kernel-per-product path (kernel_attn_decode.inc: its own source, cut out
// of hipdec_kernels.h by the test, with the cache-row decoders) run on the CPU against a plain fp64 softmax attention:
// (head, split) workgroups, the last one of a head folding the partial records and clearing the head's counter.
#include "emu.h"
#include "kernel_attn_decode.inc"
#include <cstdio>
#include <random>

static std::mt19937 rng(13);
static float urand(float a) { return std::uniform_real_distribution<float>(-a, a)(rng); }
static int failures = 0;

template <int KVBF16, int HD>
static void attn_case(int heads, int gqa, int pos, int NS) {
    const int Q = heads * HD, KV = (heads / gqa) * HD, n = pos + 1;
    const size_t esz = KVBF16 ? 2 : 4;
    float *q = (float *)std::malloc((size_t)Q * 4), *att = (float *)std::malloc((size_t)Q * 4);
    void *kc = std::malloc((size_t)n * KV * esz), *vc = std::malloc((size_t)n * KV * esz);
    float *part = (float *)std::malloc((size_t)heads * NS * (HD + 2) * 4);
    unsigned *counters = (unsigned *)std::calloc(heads, 4);
    auto fill = [&](void *p, size_t count) {
        for (size_t i = 0; i < count; ++i) {
            const float v = urand(1.5f);
            if (KVBF16) ((uint16_t *)p)[i] = f32_to_bf16_rne(v); else ((float *)p)[i] = v;
        }
    };
    auto at = [&](const void *p, size_t i) -> double { return KVBF16 ? (double)bf16_to_f32(((const uint16_t *)p)[i]) : (double)((const float *)p)[i]; };
    for (int i = 0; i < Q; ++i) { q[i] = urand(2.0f); att[i] = std::nanf(""); }
    fill(kc, (size_t)n * KV); fill(vc, (size_t)n * KV);
    StepParams *sp = (StepParams *)std::calloc(1, sizeof(StepParams));
    sp->pos = pos;
    const float scale = 1.0f / std::sqrt((float)HD);
    emu::launch_fn([&] { k_attn_decode<KVBF16, HD>(q, kc, vc, sp, part, counters, att, KV, gqa, NS, scale); }, dim3{(unsigned)heads, (unsigned)NS, 1}, 256, 0);
    double worst = 0.0;
    long counters_left = 0;
    std::vector<double> sc(n), o(HD);
    for (int h = 0; h < heads; ++h) {
        const int g = h / gqa;
        double m = -1e300;
        for (int t = 0; t < n; ++t) {
            double d = 0.0;
            for (int e = 0; e < HD; ++e) d += (double)(q[h * HD + e] * scale) * at(kc, (size_t)t * KV + (size_t)g * HD + e);
            sc[t] = d; m = std::fmax(m, d);
        }
        double l = 0.0;
        std::fill(o.begin(), o.end(), 0.0);
        for (int t = 0; t < n; ++t) {
            const double p = std::exp(sc[t] - m);
            l += p;
            for (int e = 0; e < HD; ++e) o[e] += p * at(vc, (size_t)t * KV + (size_t)g * HD + e);
        }
        for (int e = 0; e < HD; ++e) worst = std::fmax(worst, std::fabs((double)att[h * HD + e] - o[e] / l) / (0.05 + std::fabs(o[e] / l)));
        if (counters[h]) ++counters_left;
    }
    const bool ok = worst <= 2e-5 && counters_left == 0;
    std::printf("k_attn_decode<%d, %d> heads %d gqa %d rows %d splits %d: worst %.3g (allowed 2e-5), counters not cleared %ld%s\n", KVBF16, HD, heads,
                gqa, n, NS, worst, counters_left, ok ? "" : "  FAIL");
    if (!ok) ++failures;
    std::free(q); std::free(att); std::free(kc); std::free(vc); std::free(part); std::free(counters); std::free(sp);
}

int main() {
    attn_case<1, 128>(2, 1, 0, 1);           // one cache row, one split
    attn_case<1, 128>(4, 2, 299, 3);         // grouped heads, a last split shorter than the others
    attn_case<1, 64>(4, 4, 130, 8);          // more splits than some have rows for in a wave pass
    attn_case<0, 128>(2, 2, 70, 2);          // fp32 cache: 32 lanes per cache row
    attn_case<0, 64>(3, 1, 5, 4);            // fewer rows than splits x slots: empty partial records
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
