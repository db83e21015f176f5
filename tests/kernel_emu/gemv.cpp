// The matrix-vector kernel of the one-kernel-per-product path (kernel_gemv.inc: k_gemv with the four weight decoders,
// cut out of hipdec_kernels.h and hipdec_common.h by the test) run on the CPU for every weight format and every fused
// prologue / epilogue (RMSNorm on the way in; RoPE + cache append, residual, activation . up, logits on the way out)
// against plain fp64 restatements.  The 4-bit and e4m3 decoders are the ones the persistent kernels use as well.
#include "emu.h"
#include "kernel_gemv.inc"
#include <cstdio>
#include <random>

static std::mt19937 rng(17);
static float urand(float a) { return std::uniform_real_distribution<float>(-a, a)(rng); }
static int failures = 0;

struct Weights { std::vector<uint8_t> bytes; std::vector<uint8_t> scales; std::vector<double> value; };
static Weights make_weights(int wt, int rows, int K) {
    Weights w;
    w.value.resize((size_t)rows * K);
    const int G = K / 128;
    if (wt == WT_F32) { w.bytes.resize((size_t)rows * K * 4); for (size_t i = 0; i < (size_t)rows * K; ++i) { const float v = urand(0.3f); ((float *)w.bytes.data())[i] = v; w.value[i] = v; } }
    else if (wt == WT_BF16) { w.bytes.resize((size_t)rows * K * 2); for (size_t i = 0; i < (size_t)rows * K; ++i) { const uint16_t h = f32_to_bf16_rne(urand(0.3f)); ((uint16_t *)w.bytes.data())[i] = h; w.value[i] = bf16_to_f32(h); } }
    else if (wt == WT_FP8) {
        w.bytes.resize((size_t)rows * K); w.scales.resize((size_t)rows * 4);
        for (int r = 0; r < rows; ++r) {
            const float sc = 0.001f + 0.002f * std::fabs(urand(1.0f));
            ((float *)w.scales.data())[r] = sc;
            for (int k = 0; k < K; ++k) { uint8_t b = (uint8_t)(rng() & 255); if ((b & 0x7f) == 0x7f) b &= 0x7e; w.bytes[(size_t)r * K + k] = b; w.value[(size_t)r * K + k] = (double)emu::e4m3_to_float(b) * sc; }
        }
    } else {
        w.bytes.assign((size_t)rows * K / 2, 0); w.scales.resize((size_t)rows * G * 2);
        for (int r = 0; r < rows; ++r)
            for (int k = 0; k < K; ++k) {
                if (k % 128 == 0) ((uint16_t *)w.scales.data())[(size_t)r * G + k / 128] = f32_to_bf16_rne(0.01f + 0.02f * std::fabs(urand(1.0f)));
                const int nib = (int)(rng() & 15);
                w.bytes[((size_t)r * K + k) / 2] |= (uint8_t)(nib << (4 * (k & 1)));     // element 2i = low nibble of byte i, offset binary
                w.value[(size_t)r * K + k] = (double)(nib - 8) * (double)bf16_to_f32(((uint16_t *)w.scales.data())[(size_t)r * G + k / 128]);
            }
    }
    return w;
}

template <int WT, int EPI, int KVBF16>
static void gemv_case(int rows, int K, int q_dim, int kv_dim, int hd, int pos, int act, unsigned blocks) {
    constexpr bool NORM = (EPI == EPI_QKV || EPI == EPI_W13 || EPI == EPI_HEAD);
    const Weights w = make_weights(WT, rows, K);
    void *W = std::malloc(w.bytes.size()); std::memcpy(W, w.bytes.data(), w.bytes.size());
    void *S = w.scales.empty() ? nullptr : std::malloc(w.scales.size());
    if (S) std::memcpy(S, w.scales.data(), w.scales.size());
    float *in = (float *)std::malloc((size_t)K * 4), *gamma = (float *)std::malloc((size_t)K * 4), *resid = (float *)std::malloc((size_t)rows * 4);
    const int n_out = EPI == EPI_QKV ? q_dim : EPI == EPI_W13 ? rows / 2 : rows;
    float *out = (float *)std::malloc((size_t)n_out * 4);
    for (int i = 0; i < K; ++i) { in[i] = urand(2.0f); gamma[i] = urand(1.5f); }
    for (int i = 0; i < rows; ++i) resid[i] = urand(3.0f);
    for (int i = 0; i < n_out; ++i) out[i] = std::nanf("");
    const size_t esz = KVBF16 ? 2 : 4, cache_elems = (size_t)(pos + 1) * (kv_dim ? kv_dim : 1);
    void *kc = std::calloc(cache_elems, esz), *vc = std::calloc(cache_elems, esz);
    const int hp = hd / 2;
    float *rc = (float *)std::malloc((size_t)(pos + 1) * (hp ? hp : 1) * 4), *rs = (float *)std::malloc((size_t)(pos + 1) * (hp ? hp : 1) * 4);
    for (int p = 0; p <= pos; ++p) for (int i = 0; i < hp; ++i) { const double a = p * std::pow(10000.0, -2.0 * i / hd); rc[p * hp + i] = (float)std::cos(a); rs[p * hp + i] = (float)std::sin(a); }
    StepParams *sp = (StepParams *)std::calloc(1, sizeof(StepParams));
    sp->pos = pos;
    const float alpha = 0.41f;
    GemvArgs a{W, S, in, gamma, resid, out, kc, vc, rc, rs, sp, rows, K, q_dim, kv_dim, hd, alpha, act};
    emu::launch_fn([&] { k_gemv<WT, EPI, KVBF16>(a); }, dim3{blocks, 1, 1}, 256, (size_t)K * 4);

    std::vector<double> x(K), y(rows);
    double inv = 1.0;
    if (NORM) { double ss = 0; for (int i = 0; i < K; ++i) ss += (double)in[i] * in[i]; inv = 1.0 / std::sqrt(ss / K + 1e-5); }
    for (int i = 0; i < K; ++i) x[i] = NORM ? (double)in[i] * inv * gamma[i] : (double)in[i];
    for (int r = 0; r < rows; ++r) { double s = 0; for (int k = 0; k < K; ++k) s += w.value[(size_t)r * K + k] * x[k]; y[r] = s; }
    double worst = 0, scale_of = 0;
    for (int r = 0; r < rows; ++r) scale_of = std::fmax(scale_of, std::fabs(y[r]));
    auto cmp = [&](double got, double want, double extra_rel = 0.0) { worst = std::fmax(worst, (std::fabs(got - want) - extra_rel * std::fabs(want)) / (scale_of + 1e-30)); };
    auto cache_at = [&](const void *c, size_t i) -> double { return KVBF16 ? (double)bf16_to_f32(((const uint16_t *)c)[i]) : (double)((const float *)c)[i]; };
    if (EPI == EPI_QKV) {
        for (int row0 = 0; row0 < rows; row0 += 2) {
            double e = y[row0], o = y[row0 + 1];
            if (row0 < q_dim + kv_dim) {
                const int rr = row0 < q_dim ? row0 : row0 - q_dim, pi = (rr % hd) >> 1;
                const double c = rc[(size_t)pos * hp + pi], s = rs[(size_t)pos * hp + pi];
                const double e2 = e * c - o * s, o2 = o * c + e * s;
                e = e2; o = o2;
            }
            const double cache_rel = KVBF16 ? 1.0 / 256 : 0.0;
            if (row0 < q_dim) { cmp(out[row0], e); cmp(out[row0 + 1], o); }
            else if (row0 < q_dim + kv_dim) { const size_t i = (size_t)pos * kv_dim + (row0 - q_dim); cmp(cache_at(kc, i), e, cache_rel); cmp(cache_at(kc, i + 1), o, cache_rel); }
            else { const size_t i = (size_t)pos * kv_dim + (row0 - q_dim - kv_dim); cmp(cache_at(vc, i), e, cache_rel); cmp(cache_at(vc, i + 1), o, cache_rel); }
        }
    } else if (EPI == EPI_WO || EPI == EPI_W2) {
        for (int r = 0; r < rows; ++r) cmp(out[r], resid[r] + alpha * y[r]);
    } else if (EPI == EPI_W13) {
        scale_of = 0;
        std::vector<double> gte(rows / 2);
        for (int h = 0; h < rows / 2; ++h) {
            const double h1 = y[2 * h], h3 = y[2 * h + 1];
            if (act == 1) { const double l = h1 > 0 ? h1 : 0.5 * h1; gte[h] = l * l * h3; } else gte[h] = h1 / (1.0 + std::exp(-h1)) * h3;
            scale_of = std::fmax(scale_of, std::fabs(gte[h]));
        }
        for (int h = 0; h < rows / 2; ++h) cmp(out[h], gte[h]);
    } else {
        for (int r = 0; r < rows; ++r) cmp(out[r], y[r]);
    }
    const bool ok = worst <= 2e-5;
    std::printf("k_gemv<format %d, epilogue %d, bf16 cache %d> rows %d K %d: worst %.3g of the largest value (allowed 2e-5)%s\n", WT, EPI, KVBF16, rows, K, worst,
                ok ? "" : "  FAIL");
    if (!ok) ++failures;
    std::free(W); std::free(S); std::free(in); std::free(gamma); std::free(resid); std::free(out); std::free(kc); std::free(vc); std::free(rc); std::free(rs); std::free(sp);
}

template <int WT>
static void all_epilogues() {
    gemv_case<WT, EPI_QKV, 1>(128 + 2 * 64, 384, 128, 64, 64, 9, 0, 3);     // q 128, k 64, v 64 rows; head dimension 64
    gemv_case<WT, EPI_QKV, 0>(256 + 2 * 128, 256, 256, 128, 128, 3, 0, 2);
    gemv_case<WT, EPI_WO, 0>(97, 384, 0, 0, 0, 0, 0, 3);                    // an odd row count re-reads its last row
    gemv_case<WT, EPI_W13, 0>(2 * 70, 256, 0, 0, 0, 0, 0, 2);
    gemv_case<WT, EPI_W13, 0>(2 * 70, 256, 0, 0, 0, 0, 1, 2);
    gemv_case<WT, EPI_W2, 0>(64, 1152, 0, 0, 0, 0, 0, 5);
    gemv_case<WT, EPI_HEAD, 0>(301, 128, 0, 0, 0, 0, 0, 4);
}

int main() {
    all_epilogues<WT_F32>();
    all_epilogues<WT_BF16>();
    all_epilogues<WT_FP8>();
    all_epilogues<WT_INT4>();
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
