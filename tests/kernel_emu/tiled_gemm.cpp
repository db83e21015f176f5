// The tiled prefill GEMM kernel (kernel_tiled.inc: k_pf_gemm with its helpers, cut out of hipdec_prefill.h by the
// test) run on the CPU for bf16, e4m3 and 4-bit weights and the three activation formats (bf16 pair, bf16 hi part
// only, one fp16 number) under the launch plan given on the command line, against a plain fp64 product of the stored
// operands.  Every operand lives in a heap block of its exact size (AddressSanitizer sees any access outside).
// usage: tiled_gemm weight_format(1 bf16, 2 e4m3, 3 4-bit) activation_format(0 pair, 1 bf16, 2 fp16) T N K steps_per_split gx gy gz seed
#include "emu.h"
#define PF_BM 128
#define PF_BN_OF(WT) ((WT) == WT_FP8 ? 256 : 128)
#define PF_BK 32
#define PF_BKL 64
#define PF_LDS_STRIDE 72
typedef float pf_f32x16 __attribute__((ext_vector_type(16)));
#include "kernel_tiled.inc"
#include <cstdio>
#include <random>

int main(int argc, char **argv) {
    if (argc != 11) { std::fprintf(stderr, "usage: tiled_gemm wt act T N K steps_per_split gx gy gz seed\n"); return 2; }
    const int wt = atoi(argv[1]), act = atoi(argv[2]), T = atoi(argv[3]), N = atoi(argv[4]), K = atoi(argv[5]), sps = atoi(argv[6]);
    const dim3 grid{(unsigned)atoi(argv[7]), (unsigned)atoi(argv[8]), (unsigned)atoi(argv[9])};
    if (wt < 1 || wt > 3 || act < 0 || act > 2 || T < 1 || K % 32 || (wt == 3 && K % 128)) { std::fprintf(stderr, "not a launch of this kernel\n"); return 2; }
    const int kgrp = K / 128, splits = (int)grid.z;
    std::mt19937 rng((unsigned)atoi(argv[10]));
    std::uniform_real_distribution<float> ud(-1.0f, 1.0f);
    const size_t wbytes = wt == 1 ? (size_t)N * K * 2 : wt == 2 ? (size_t)N * K : (size_t)N * K / 2;
    uint16_t *Ahi = (uint16_t *)std::malloc((size_t)T * K * 2), *Alo = (uint16_t *)std::malloc((size_t)T * K * 2);
    uint8_t *W = (uint8_t *)std::calloc(wbytes, 1);
    uint16_t *S = wt == 3 ? (uint16_t *)std::malloc((size_t)N * kgrp * 2) : nullptr;
    float *P = (float *)std::malloc((size_t)splits * T * N * 4);
    std::vector<double> a((size_t)T * K), wv((size_t)N * K);
    for (size_t i = 0; i < (size_t)T * K; ++i) {
        const float v = ud(rng) * 3.0f;
        if (act == 2) { const _Float16 h = (_Float16)v; std::memcpy(&Ahi[i], &h, 2); Alo[i] = 0; a[i] = (double)(float)h; }
        else {
            Ahi[i] = f32_to_bf16_rne(v); Alo[i] = f32_to_bf16_rne(v - bf16_to_f32(Ahi[i]));
            a[i] = (double)bf16_to_f32(Ahi[i]) + (act == 0 ? (double)bf16_to_f32(Alo[i]) : 0.0);
        }
    }
    if (wt == 3) for (size_t i = 0; i < (size_t)N * kgrp; ++i) S[i] = f32_to_bf16_rne(0.01f + 0.02f * std::fabs(ud(rng)));
    for (size_t i = 0; i < (size_t)N * K; ++i) {
        const int n = (int)(i / K), k = (int)(i % K);
        if (wt == 1) { const uint16_t h = f32_to_bf16_rne(ud(rng) * 0.3f); ((uint16_t *)W)[i] = h; wv[i] = bf16_to_f32(h); }
        else if (wt == 2) { uint8_t b = (uint8_t)(rng() & 255); if ((b & 0x7f) == 0x7f) b &= 0x7e; W[i] = b; wv[i] = emu::e4m3_to_float(b); }
        else { const int nib = (int)(rng() & 15); W[i / 2] |= (uint8_t)(nib << (4 * (k & 1))); wv[i] = (double)(nib - 8) * (double)bf16_to_f32(S[(size_t)n * kgrp + k / 128]); }
    }
    for (size_t i = 0; i < (size_t)splits * T * N; ++i) P[i] = std::nanf("");
    PfGemm g{Ahi, Alo, W, S, P, T, N, K, sps};
#define GO(WTX) do { if (act == 2) emu::launch(k_pf_gemm<WTX, PF_ACT_F16>, grid, 256, 0, g); else if (act == 1) emu::launch(k_pf_gemm<WTX, PF_ACT_BF16>, grid, 256, 0, g); \
                     else emu::launch(k_pf_gemm<WTX, PF_ACT_PAIR>, grid, 256, 0, g); } while (0)
    if (wt == 1) GO(WT_BF16); else if (wt == 2) GO(WT_FP8); else GO(WT_INT4);
    double worst = 0.0, big = 0.0;
    long unwritten = 0;
    for (int t = 0; t < T; ++t)
        for (int n = 0; n < N; ++n) {
            double ref = 0.0;
            for (int k = 0; k < K; ++k) ref += a[(size_t)t * K + k] * wv[(size_t)n * K + k];
            double got = 0.0;
            for (int z = 0; z < splits; ++z) { const float p = P[((size_t)z * T + t) * N + n]; if (p != p) ++unwritten; got += p; }
            worst = std::fmax(worst, std::fabs(got - ref));
            big = std::fmax(big, std::fabs(ref));
        }
    std::printf("weights %d activations %d T %d N %d K %d: %d splits, max |kernel - fp64| = %.3g, largest value %.3g, result elements not written %ld\n", wt, act, T,
                N, K, splits, worst, big, unwritten);
    std::free(Ahi); std::free(Alo); std::free(W); std::free(S); std::free(P);
    return (unwritten == 0 && worst <= 2e-5 * big) ? 0 : 1;
}
