// The element-wise kernels between the products of the prefill / multi-row step (kernels_epi.inc: their own source, cut
// out of hipdec_prefill.h and hipdec_batch.h by the test) run on the CPU on seeded random operands against plain fp64
// restatements: split planes summed, residual + norm input + chunk sums of squares (k_pf_resid), activation . up
// (k_pf_gate_epi), RoPE + cache append of the multi-row step (k_bd_qkv_epi), and the logits' row factor
// (k_bd_sum_planes).  Every operand lives in a heap block of its exact size (AddressSanitizer sees any access outside).
#include "emu.h"
#include "kernels_epi.inc"
#include <cstdio>
#include <random>

static std::mt19937 rng(7);
static float urand(float a) { return std::uniform_real_distribution<float>(-a, a)(rng); }
template <class T> static T *alloc(size_t n) { return (T *)std::malloc(n * sizeof(T) ? n * sizeof(T) : 1); }
static int failures = 0;
static void check(const char *what, double worst, double tol, long extra_bad = 0) {
    const bool ok = worst <= tol && extra_bad == 0;
    std::printf("%-60s worst %.3g (allowed %.3g)%s\n", what, worst, tol, ok ? "" : "  FAIL");
    if (!ok) ++failures;
}
static double pair_value(uint16_t hi, uint16_t lo) { return (double)bf16_to_f32(hi) + (double)bf16_to_f32(lo); }

static void resid_case(int T, int D, int splits, bool with_scale, bool with_gamma) {
    const int nch = (D + PF_CHUNK - 1) / PF_CHUNK;
    const size_t plane = (size_t)T * D;
    float *P = alloc<float>(splits * plane), *ws = with_scale ? alloc<float>(D) : nullptr, *res = alloc<float>(plane), *out = alloc<float>(plane);
    float *gamma = with_gamma ? alloc<float>(D) : nullptr, *ssq = alloc<float>((size_t)T * nch);
    uint16_t *hi = alloc<uint16_t>(plane), *lo = alloc<uint16_t>(plane);
    for (size_t i = 0; i < splits * plane; ++i) P[i] = urand(2.0f);
    for (size_t i = 0; i < plane; ++i) { res[i] = urand(3.0f); out[i] = std::nanf(""); hi[i] = lo[i] = 0x7fc0; }
    for (int d = 0; d < D; ++d) { if (ws) ws[d] = 0.5f + std::fabs(urand(1.0f)); if (gamma) gamma[d] = urand(2.0f); }
    for (int i = 0; i < T * nch; ++i) ssq[i] = std::nanf("");
    const float alpha = 0.37f;
    emu::launch_fn([&] { k_pf_resid(P, splits, plane, ws, res, alpha, out, gamma, hi, lo, ssq, D, nch, 0); }, dim3{(unsigned)((nch + 3) / 4), (unsigned)T, 1}, 256, 0);
    double worst = 0, worst_pair = 0, worst_ssq = 0;
    for (int t = 0; t < T; ++t) {
        std::vector<double> ss(nch, 0.0);
        for (int d = 0; d < D; ++d) {
            double s = 0;
            for (int z = 0; z < splits; ++z) s += P[z * plane + (size_t)t * D + d];
            const double v = res[(size_t)t * D + d] + alpha * s * (ws ? ws[d] : 1.0);
            worst = std::fmax(worst, std::fabs(out[(size_t)t * D + d] - v) / (1.0 + std::fabs(v)));
            // the pair holds the kernel's own fp32 row times gamma to 16 bits (the row itself is checked against fp64 above)
            if (gamma) {
                const double want = (double)out[(size_t)t * D + d] * gamma[d];
                worst_pair = std::fmax(worst_pair, std::fabs(pair_value(hi[(size_t)t * D + d], lo[(size_t)t * D + d]) - want) / (1e-30 + std::fabs(want)));
            }
            ss[d / PF_CHUNK] += v * v;
        }
        for (int c = 0; c < nch; ++c) worst_ssq = std::fmax(worst_ssq, std::fabs(ssq[t * nch + c] - ss[c]) / (1.0 + ss[c]));
    }
    char name[128];
    std::snprintf(name, sizeof name, "k_pf_resid T %d D %d splits %d scale %d gamma %d: rows", T, D, splits, (int)with_scale, (int)with_gamma);
    check(name, worst, 2e-6);
    if (gamma) check("    hi + lo = row * gamma", worst_pair, 3e-5);
    check("    chunk sums of squares", worst_ssq, 1e-5);
    std::free(P); std::free(ws); std::free(res); std::free(out); std::free(gamma); std::free(ssq); std::free(hi); std::free(lo);
}

static double row_inv(const std::vector<double> &row, int D) { double s = 0; for (double v : row) s += v * v; return 1.0 / std::sqrt(s / D + 1e-5); }

static void gate_case(int T, int D, int H, int splits, bool with_scale, int act) {
    const int nch = (D + PF_CHUNK - 1) / PF_CHUNK;
    const size_t plane = (size_t)T * 2 * H;
    float *P = alloc<float>(splits * plane), *ws = with_scale ? alloc<float>(2 * H) : nullptr, *ssq = alloc<float>((size_t)T * nch);
    uint16_t *hi = alloc<uint16_t>((size_t)T * H), *lo = alloc<uint16_t>((size_t)T * H);
    for (size_t i = 0; i < splits * plane; ++i) P[i] = urand(1.5f);
    for (int i = 0; i < 2 * H && ws; ++i) ws[i] = 0.5f + std::fabs(urand(1.0f));
    std::vector<double> inv(T);
    for (int t = 0; t < T; ++t) { double s = 0; for (int c = 0; c < nch; ++c) { ssq[t * nch + c] = 10.0f + std::fabs(urand(30.0f)); s += ssq[t * nch + c]; } inv[t] = 1.0 / std::sqrt(s / D + 1e-5); }
    emu::launch_fn([&] { k_pf_gate_epi(P, splits, plane, ws, hi, lo, ssq, nch, D, T, H, act, 0); }, dim3{(unsigned)((H / 4 + 255) / 256), (unsigned)T, 1}, 256, 0);
    double worst = 0;
    for (int t = 0; t < T; ++t)
        for (int j = 0; j < H; ++j) {
            double h1 = 0, h3 = 0;
            for (int z = 0; z < splits; ++z) { h1 += P[z * plane + (size_t)t * 2 * H + 2 * j]; h3 += P[z * plane + (size_t)t * 2 * H + 2 * j + 1]; }
            if (ws) { h1 *= ws[2 * j]; h3 *= ws[2 * j + 1]; }
            h1 *= inv[t]; h3 *= inv[t];
            double gte;
            if (act == 1) { const double lr = h1 > 0 ? h1 : 0.5 * h1; gte = lr * lr * h3; }
            else gte = h1 / (1.0 + std::exp(-h1)) * h3;
            // fp32 sums of up to a dozen planes (absolute part) and the 16-bit pair (relative part)
            worst = std::fmax(worst, std::fabs(pair_value(hi[(size_t)t * H + j], lo[(size_t)t * H + j]) - gte) / (2e-2 + std::fabs(gte)));
        }
    char name[128];
    std::snprintf(name, sizeof name, "k_pf_gate_epi T %d D %d H %d splits %d scale %d act %d", T, D, H, splits, (int)with_scale, act);
    check(name, worst, 1e-4);
    std::free(P); std::free(ws); std::free(ssq); std::free(hi); std::free(lo);
}

template <int KVBF16>
static void bd_qkv_case(int R, int D, int Q, int KV, int hd, int splits, bool with_scale, int pos, int slot, int suf_rows) {
    const int nch = (D + PF_CHUNK - 1) / PF_CHUNK, N = Q + 2 * KV;
    const size_t plane = (size_t)R * N;
    float *P = alloc<float>(splits * plane), *ws = with_scale ? alloc<float>(N) : nullptr, *ssq = alloc<float>((size_t)R * nch), *q = alloc<float>((size_t)R * Q);
    const size_t cache_elems = (size_t)R * suf_rows * KV;
    void *kc = std::malloc(cache_elems * (KVBF16 ? 2 : 4)), *vc = std::malloc(cache_elems * (KVBF16 ? 2 : 4));
    std::memset(kc, 0, cache_elems * (KVBF16 ? 2 : 4)); std::memset(vc, 0, cache_elems * (KVBF16 ? 2 : 4));
    float *rc = alloc<float>((size_t)(pos + 1) * (hd / 2)), *rs = alloc<float>((size_t)(pos + 1) * (hd / 2));
    for (int p = 0; p <= pos; ++p) for (int i = 0; i < hd / 2; ++i) { const double a = p * std::pow(10000.0, -2.0 * i / hd); rc[p * (hd / 2) + i] = (float)std::cos(a); rs[p * (hd / 2) + i] = (float)std::sin(a); }
    for (size_t i = 0; i < splits * plane; ++i) P[i] = urand(1.5f);
    for (int i = 0; i < N && ws; ++i) ws[i] = 0.5f + std::fabs(urand(1.0f));
    std::vector<double> inv(R);
    for (int t = 0; t < R; ++t) { double s = 0; for (int c = 0; c < nch; ++c) { ssq[t * nch + c] = 10.0f + std::fabs(urand(30.0f)); s += ssq[t * nch + c]; } inv[t] = 1.0 / std::sqrt(s / D + 1e-5); }
    for (size_t i = 0; i < (size_t)R * Q; ++i) q[i] = std::nanf("");
    BatchParams *bp = alloc<BatchParams>(1);
    *bp = BatchParams{pos, slot, pos - slot, 0, 1.0f, 0.0f};
    const size_t items = (size_t)R * (N / 2);
    emu::launch_fn([&] { k_bd_qkv_epi<KVBF16>(P, splits, plane, ws, q, kc, vc, (size_t)suf_rows, rc, rs, bp, ssq, nch, D, R, Q, KV, hd); },
                   dim3{(unsigned)((items + 255) / 256), 1, 1}, 256, 0);
    double worst_q = 0, worst_kv = 0;
    long stray = 0;
    for (int t = 0; t < R; ++t)
        for (int row0 = 0; row0 < N; row0 += 2) {
            double s0 = 0, s1 = 0;
            for (int z = 0; z < splits; ++z) { s0 += P[z * plane + (size_t)t * N + row0]; s1 += P[z * plane + (size_t)t * N + row0 + 1]; }
            if (ws) { s0 *= ws[row0]; s1 *= ws[row0 + 1]; }
            s0 *= inv[t]; s1 *= inv[t];
            if (row0 < Q + KV) {
                const int rr = row0 < Q ? row0 : row0 - Q, pi2 = (rr % hd) >> 1;
                const double c = rc[(size_t)pos * (hd / 2) + pi2], s = rs[(size_t)pos * (hd / 2) + pi2];
                const double e = s0 * c - s1 * s, o = s1 * c + s0 * s;
                s0 = e; s1 = o;
            }
            if (row0 < Q) {
                worst_q = std::fmax(worst_q, std::fmax(std::fabs(q[(size_t)t * Q + row0] - s0), std::fabs(q[(size_t)t * Q + row0 + 1] - s1)) / (1.0 + std::fabs(s0) + std::fabs(s1)));
            } else {
                const bool isk = row0 < Q + KV;
                const int rr = isk ? row0 - Q : row0 - Q - KV;
                const size_t at = ((size_t)t * suf_rows + slot) * KV + rr;
                double g0, g1;
                if (KVBF16) { g0 = bf16_to_f32(((uint16_t *)(isk ? kc : vc))[at]); g1 = bf16_to_f32(((uint16_t *)(isk ? kc : vc))[at + 1]); }
                else { g0 = ((float *)(isk ? kc : vc))[at]; g1 = ((float *)(isk ? kc : vc))[at + 1]; }
                const double tol = KVBF16 ? 1.0 / 256 : 0.0;     // (bf16 cache: half a unit in the last of 8 bits, relative)
                worst_kv = std::fmax(worst_kv, std::fmax((std::fabs(g0 - s0) - tol * std::fabs(s0)) / (1.0 + std::fabs(s0)), (std::fabs(g1 - s1) - tol * std::fabs(s1)) / (1.0 + std::fabs(s1))));
            }
        }
    // nothing but slot `slot` of every row's suffix cache may have been written
    for (int t = 0; t < R; ++t)
        for (int sr = 0; sr < suf_rows; ++sr)
            if (sr != slot)
                for (int c = 0; c < KV; ++c) {
                    const size_t at = ((size_t)t * suf_rows + sr) * KV + c;
                    if (KVBF16 ? (((uint16_t *)kc)[at] || ((uint16_t *)vc)[at]) : (((float *)kc)[at] != 0.0f || ((float *)vc)[at] != 0.0f)) ++stray;
                }
    char name[160];
    std::snprintf(name, sizeof name, "k_bd_qkv_epi<%d> R %d Q %d KV %d hd %d splits %d scale %d pos %d slot %d: q", KVBF16, R, Q, KV, hd, splits, (int)with_scale, pos, slot);
    check(name, worst_q, 3e-6);
    check("    k / v rows appended at the slot, other slots untouched", worst_kv, 3e-6, stray);
    std::free(P); std::free(ws); std::free(ssq); std::free(q); std::free(kc); std::free(vc); std::free(rc); std::free(rs); std::free(bp);
}

static void sum_planes_case(int R, int D, int V, int splits) {
    const int nch = (D + PF_CHUNK - 1) / PF_CHUNK;
    const size_t n = (size_t)R * V;
    float *P = alloc<float>(splits * n), *out = alloc<float>(n), *ssq = alloc<float>((size_t)R * nch);
    for (size_t i = 0; i < splits * n; ++i) P[i] = urand(2.0f);
    for (size_t i = 0; i < n; ++i) out[i] = std::nanf("");
    std::vector<double> inv(R);
    for (int t = 0; t < R; ++t) { double s = 0; for (int c = 0; c < nch; ++c) { ssq[t * nch + c] = 10.0f + std::fabs(urand(30.0f)); s += ssq[t * nch + c]; } inv[t] = 1.0 / std::sqrt(s / D + 1e-5); }
    emu::launch_fn([&] { k_bd_sum_planes(P, splits, n, out, n, ssq, nch, D, V); }, dim3{(unsigned)((n + 255) / 256), 1, 1}, 256, 0);
    double worst = 0;
    for (size_t i = 0; i < n; ++i) {
        double s = 0;
        for (int z = 0; z < splits; ++z) s += P[z * n + i];
        s *= inv[i / V];
        worst = std::fmax(worst, std::fabs(out[i] - s) / (1.0 + std::fabs(s)));
    }
    char name[128];
    std::snprintf(name, sizeof name, "k_bd_sum_planes R %d D %d V %d splits %d", R, D, V, splits);
    check(name, worst, 3e-6);
    std::free(P); std::free(out); std::free(ssq);
}

template <int EWT>
static void embed_case(int T, int D, int vocab) {
    const int nch = (D + PF_CHUNK - 1) / PF_CHUNK;
    void *embed = std::malloc((size_t)vocab * D * (EWT == WT_F32 ? 4 : 2));
    for (size_t i = 0; i < (size_t)vocab * D; ++i) { const float v = urand(2.0f); if (EWT == WT_F32) ((float *)embed)[i] = v; else ((uint16_t *)embed)[i] = f32_to_bf16_rne(v); }
    uint32_t *ids = alloc<uint32_t>(T);
    for (int t = 0; t < T; ++t) ids[t] = (uint32_t)(rng() % vocab);
    ids[0] = (uint32_t)(vocab - 1);                                                   // the table's last row
    float *x = alloc<float>((size_t)T * D), *gamma = alloc<float>(D), *ssq = alloc<float>((size_t)T * nch);
    uint16_t *hi = alloc<uint16_t>((size_t)T * D), *lo = alloc<uint16_t>((size_t)T * D);
    for (int d = 0; d < D; ++d) gamma[d] = urand(2.0f);
    for (size_t i = 0; i < (size_t)T * D; ++i) x[i] = std::nanf("");
    emu::launch_fn([&] { k_pf_embed<EWT>(embed, ids, x, gamma, hi, lo, ssq, D, 0); }, dim3{(unsigned)nch, (unsigned)T, 1}, PF_CHUNK, 0);
    double worst_pair = 0, worst_ssq = 0;
    long bad = 0;
    for (int t = 0; t < T; ++t) {
        std::vector<double> ss(nch, 0.0);
        for (int d = 0; d < D; ++d) {
            const size_t at = (size_t)ids[t] * D + d;
            const float v = EWT == WT_F32 ? ((float *)embed)[at] : bf16_to_f32(((uint16_t *)embed)[at]);
            if (!(x[(size_t)t * D + d] == v)) ++bad;
            const double want = (double)(v * gamma[d]);
            worst_pair = std::fmax(worst_pair, std::fabs(pair_value(hi[(size_t)t * D + d], lo[(size_t)t * D + d]) - want) / (1e-30 + std::fabs(want)));
            ss[d / PF_CHUNK] += (double)v * v;
        }
        for (int c = 0; c < nch; ++c) worst_ssq = std::fmax(worst_ssq, std::fabs(ssq[t * nch + c] - ss[c]) / (1.0 + ss[c]));
    }
    char name[128];
    std::snprintf(name, sizeof name, "k_pf_embed<%d> T %d D %d: rows copied exactly, hi + lo = row * gamma", EWT, T, D);
    check(name, worst_pair, 3e-5, bad);
    check("    chunk sums of squares", worst_ssq, 1e-5);
    std::free(embed); std::free(ids); std::free(x); std::free(gamma); std::free(ssq); std::free(hi); std::free(lo);
}

template <int KVBF16>
static void pf_qkv_case(int T, int D, int Q, int KV, int hd, int splits, bool with_scale, int pos0) {
    const int nch = (D + PF_CHUNK - 1) / PF_CHUNK, N = Q + 2 * KV, seq = pos0 + T;
    const size_t plane = (size_t)T * N;
    float *P = alloc<float>(splits * plane), *ws = with_scale ? alloc<float>(N) : nullptr, *ssq = alloc<float>((size_t)T * nch), *q = alloc<float>((size_t)T * Q);
    const size_t cache_elems = (size_t)seq * KV;
    void *kc = std::calloc(cache_elems, KVBF16 ? 2 : 4), *vc = std::calloc(cache_elems, KVBF16 ? 2 : 4);
    float *rc = alloc<float>((size_t)seq * (hd / 2)), *rs = alloc<float>((size_t)seq * (hd / 2));
    for (int p = 0; p < seq; ++p) for (int i = 0; i < hd / 2; ++i) { const double a = p * std::pow(10000.0, -2.0 * i / hd); rc[p * (hd / 2) + i] = (float)std::cos(a); rs[p * (hd / 2) + i] = (float)std::sin(a); }
    for (size_t i = 0; i < splits * plane; ++i) P[i] = urand(1.5f);
    for (int i = 0; i < N && ws; ++i) ws[i] = 0.5f + std::fabs(urand(1.0f));
    std::vector<double> inv(T);
    for (int t = 0; t < T; ++t) { double s = 0; for (int c = 0; c < nch; ++c) { ssq[t * nch + c] = 10.0f + std::fabs(urand(30.0f)); s += ssq[t * nch + c]; } inv[t] = 1.0 / std::sqrt(s / D + 1e-5); }
    for (size_t i = 0; i < (size_t)T * Q; ++i) q[i] = std::nanf("");
    emu::launch_fn([&] { k_pf_qkv_epi<KVBF16>(P, splits, plane, ws, q, kc, vc, rc, rs, ssq, nch, D, T, Q, KV, hd, pos0); },
                   dim3{(unsigned)((N / 4 + 255) / 256), (unsigned)T, 1}, 256, 0);
    double worst_q = 0, worst_kv = 0;
    long stray = 0;
    for (int t = 0; t < T; ++t)
        for (int row0 = 0; row0 < N; row0 += 2) {
            double s0 = 0, s1 = 0;
            for (int z = 0; z < splits; ++z) { s0 += P[z * plane + (size_t)t * N + row0]; s1 += P[z * plane + (size_t)t * N + row0 + 1]; }
            if (ws) { s0 *= ws[row0]; s1 *= ws[row0 + 1]; }
            s0 *= inv[t]; s1 *= inv[t];
            const int pos = pos0 + t;
            if (row0 < Q + KV) {
                const int rr = row0 < Q ? row0 : row0 - Q, pi2 = (rr % hd) >> 1;
                const double c = rc[(size_t)pos * (hd / 2) + pi2], s = rs[(size_t)pos * (hd / 2) + pi2];
                const double e = s0 * c - s1 * s, o = s1 * c + s0 * s;
                s0 = e; s1 = o;
            }
            if (row0 < Q) worst_q = std::fmax(worst_q, std::fmax(std::fabs(q[(size_t)t * Q + row0] - s0), std::fabs(q[(size_t)t * Q + row0 + 1] - s1)) / (1.0 + std::fabs(s0) + std::fabs(s1)));
            else {
                const bool isk = row0 < Q + KV;
                const size_t at = (size_t)pos * KV + (isk ? row0 - Q : row0 - Q - KV);
                double g0, g1;
                if (KVBF16) { g0 = bf16_to_f32(((uint16_t *)(isk ? kc : vc))[at]); g1 = bf16_to_f32(((uint16_t *)(isk ? kc : vc))[at + 1]); }
                else { g0 = ((float *)(isk ? kc : vc))[at]; g1 = ((float *)(isk ? kc : vc))[at + 1]; }
                const double tol = KVBF16 ? 1.0 / 256 : 0.0;
                worst_kv = std::fmax(worst_kv, std::fmax((std::fabs(g0 - s0) - tol * std::fabs(s0)) / (1.0 + std::fabs(s0)), (std::fabs(g1 - s1) - tol * std::fabs(s1)) / (1.0 + std::fabs(s1))));
            }
        }
    for (size_t i = 0; i < (size_t)pos0 * KV; ++i)                                    // rows in front of the chunk stay as they were
        if (KVBF16 ? (((uint16_t *)kc)[i] || ((uint16_t *)vc)[i]) : (((float *)kc)[i] != 0.0f || ((float *)vc)[i] != 0.0f)) ++stray;
    char name[160];
    std::snprintf(name, sizeof name, "k_pf_qkv_epi<%d> T %d Q %d KV %d hd %d splits %d scale %d first position %d: q", KVBF16, T, Q, KV, hd, splits, (int)with_scale, pos0);
    check(name, worst_q, 3e-6);
    check("    k / v rows written at their positions, earlier rows untouched", worst_kv, 3e-6, stray);
    std::free(P); std::free(ws); std::free(ssq); std::free(q); std::free(kc); std::free(vc); std::free(rc); std::free(rs);
}

int main() {
    embed_case<WT_F32>(3, 640, 50);
    embed_case<WT_BF16>(5, 1000, 33);              // a last chunk that is not full
    for (int splits : {1, 4, 5, 9}) pf_qkv_case<1>(5, 512, 256, 128, 64, splits, splits == 4, 7);
    pf_qkv_case<0>(3, 384, 384, 128, 128, 6, true, 0);
    pf_qkv_case<1>(2, 256, 1280, 256, 128, 2, false, 300);     // more than one workgroup per row
    // split counts on both sides of the four- and eight-plane request rounds of the plane sums
    for (int splits : {1, 3, 4, 5, 8, 9, 11, 17, 22}) resid_case(3, 640, splits, splits % 2 == 0, true);
    resid_case(1, 256, 2, false, false);
    resid_case(5, 1000, 7, true, true);            // a last chunk that is not full
    for (int splits : {1, 4, 5, 8, 9}) gate_case(3, 512, 344, splits, splits == 5, splits % 2);
    gate_case(2, 384, 1028, 3, true, 0);           // more than one workgroup per row
    for (int splits : {1, 4, 5, 11}) bd_qkv_case<1>(3, 512, 256, 128, 64, splits, splits == 4, 37, 5, 9);
    bd_qkv_case<0>(5, 384, 384, 128, 128, 6, true, 12, 0, 4);
    bd_qkv_case<1>(8, 256, 256, 256, 128, 8, false, 600, 88, 100);
    for (int splits : {1, 2, 4, 6, 8, 13}) sum_planes_case(3, 512, 1000, splits);
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
