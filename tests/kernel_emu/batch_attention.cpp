// The multi-row step's attention kernel (kernel_bd_attn.inc: its own source, cut out of hipdec_batch.h by the test,
// with the cache-row decoders and the pair split it calls) run on the CPU against a plain fp64 softmax attention over
// the shared prefix rows and each row's own suffix rows.  Every operand lives in a heap block of its exact size.
#include "emu.h"
#include "kernel_bd_attn.inc"
#include <cstdio>
#include <random>

static std::mt19937 rng(11);
static float urand(float a) { return std::uniform_real_distribution<float>(-a, a)(rng); }
static int failures = 0;

template <int KVBF16, int HD>
static void attn_case(int R, int heads, int gqa, int prefix, int slot, int suf_rows) {
    const int Q = heads * HD, KV = (heads / gqa) * HD, n = prefix + slot + 1;
    const size_t esz = KVBF16 ? 2 : 4;
    float *q = (float *)std::malloc((size_t)R * Q * 4);
    void *kc = std::malloc((size_t)(prefix ? prefix : 1) * KV * esz), *vc = std::malloc((size_t)(prefix ? prefix : 1) * KV * esz);
    void *ks = std::malloc((size_t)R * suf_rows * KV * esz), *vs = std::malloc((size_t)R * suf_rows * KV * esz);
    uint16_t *ohi = (uint16_t *)std::malloc((size_t)R * Q * 2), *olo = (uint16_t *)std::malloc((size_t)R * Q * 2);
    auto fill = [&](void *p, size_t count) {
        for (size_t i = 0; i < count; ++i) {
            const float v = urand(1.5f);
            if (KVBF16) ((uint16_t *)p)[i] = f32_to_bf16_rne(v); else ((float *)p)[i] = v;
        }
    };
    auto at = [&](const void *p, size_t i) -> double { return KVBF16 ? (double)bf16_to_f32(((const uint16_t *)p)[i]) : (double)((const float *)p)[i]; };
    for (size_t i = 0; i < (size_t)R * Q; ++i) { q[i] = urand(2.0f); ohi[i] = olo[i] = 0x7fc0; }
    fill(kc, (size_t)prefix * KV); fill(vc, (size_t)prefix * KV); fill(ks, (size_t)R * suf_rows * KV); fill(vs, (size_t)R * suf_rows * KV);
    BatchParams *bp = (BatchParams *)std::malloc(sizeof(BatchParams));
    *bp = BatchParams{prefix + slot, slot, prefix, 0, 1.0f, 0.0f};
    const float scale = 1.0f / std::sqrt((float)HD);
    emu::launch_fn([&] { k_bd_attn<KVBF16, HD>(q, kc, vc, ks, vs, (size_t)suf_rows, bp, ohi, olo, Q, KV, gqa, scale); },
                   dim3{(unsigned)heads, (unsigned)R, 1}, BD_ATT_THREADS, 0);
    double worst = 0.0;
    std::vector<double> sc(n), o(HD);
    for (int r = 0; r < R; ++r)
        for (int h = 0; h < heads; ++h) {
            const int g = h / gqa;
            double m = -1e300;
            for (int t = 0; t < n; ++t) {
                const void *kp = t < prefix ? kc : ks;
                const size_t base = t < prefix ? (size_t)t * KV : ((size_t)r * suf_rows + (t - prefix)) * KV;
                double d = 0.0;
                for (int e = 0; e < HD; ++e) d += (double)(q[(size_t)r * Q + h * HD + e] * scale) * at(kp, base + (size_t)g * HD + e);
                sc[t] = d; m = std::fmax(m, d);
            }
            double l = 0.0;
            std::fill(o.begin(), o.end(), 0.0);
            for (int t = 0; t < n; ++t) {
                const void *vp = t < prefix ? vc : vs;
                const size_t base = t < prefix ? (size_t)t * KV : ((size_t)r * suf_rows + (t - prefix)) * KV;
                const double p = std::exp(sc[t] - m);
                l += p;
                for (int e = 0; e < HD; ++e) o[e] += p * at(vp, base + (size_t)g * HD + e);
            }
            for (int e = 0; e < HD; ++e) {
                const size_t i = (size_t)r * Q + h * HD + e;
                const double got = (double)bf16_to_f32(ohi[i]) + (double)bf16_to_f32(olo[i]);
                worst = std::fmax(worst, std::fabs(got - o[e] / l) / (0.05 + std::fabs(o[e] / l)));
            }
        }
    const bool ok = worst <= 1e-4;
    std::printf("k_bd_attn<%d, %d> rows %d heads %d gqa %d prefix %d slot %d: worst %.3g (allowed 1e-4)%s\n", KVBF16, HD, R, heads, gqa, prefix, slot,
                worst, ok ? "" : "  FAIL");
    if (!ok) ++failures;
    std::free(q); std::free(kc); std::free(vc); std::free(ks); std::free(vs); std::free(ohi); std::free(olo); std::free(bp);
}

int main() {
    attn_case<1, 128>(2, 2, 1, 37, 0, 4);          // fewer rows than slots: most lane groups have nothing to do
    attn_case<1, 128>(3, 4, 2, 300, 5, 9);         // grouped heads, more than one pass of 256 rows
    attn_case<1, 64>(2, 4, 4, 130, 2, 3);
    attn_case<0, 128>(2, 2, 2, 70, 1, 2);          // fp32 cache: 32 lanes per cache row
    attn_case<0, 64>(1, 2, 1, 0, 0, 1);            // no prefix, a single position
    attn_case<1, 128>(1, 1, 1, 1029, 3, 8);        // a count that ends inside a pass
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
