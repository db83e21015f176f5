// The 4-bit few-row GEMM kernel's own source (kernel_i4.inc: cut out of hipdec_prefill.h by the test) run on the
// CPU under the launch plan given on the command line, on seeded random operands, against a plain fp64 product.
// Every operand lives in a heap block of its exact size, so with -fsanitize=address an access outside any of them
// (weights, scales, activation planes, result planes, LDS) ends the program with a report.
// usage: few_row_i4 T N K steps_per_split gx gy gz threads lds_bytes seed
#include "emu.h"
#define PF_BK 32
#define PF_SK_PAD 8
#include "pfgemm_struct.inc"
#include "kernel_i4.inc"
#include <cstdio>
#include <random>

static uint16_t to_bf16(float v) { uint32_t u; std::memcpy(&u, &v, 4); u += 0x7fff + ((u >> 16) & 1); return (uint16_t)(u >> 16); }

int main(int argc, char **argv) {
    if (argc != 11) { std::fprintf(stderr, "usage: few_row_i4 T N K steps_per_split gx gy gz threads lds_bytes seed\n"); return 2; }
    const int T = atoi(argv[1]), N = atoi(argv[2]), K = atoi(argv[3]), sps = atoi(argv[4]);
    const dim3 grid{(unsigned)atoi(argv[5]), (unsigned)atoi(argv[6]), (unsigned)atoi(argv[7])};
    const unsigned threads = (unsigned)atoi(argv[8]);
    const size_t lds_bytes = (size_t)atoll(argv[9]);
    if (threads != 512 || T < 1 || T > 32 || K % 128 || grid.z != 1) { std::fprintf(stderr, "not a launch of this kernel\n"); return 2; }
    const int kgrp = K / 128, splits = (int)grid.y;
    std::mt19937 rng((unsigned)atoi(argv[10]));
    std::uniform_real_distribution<float> ud(-1.0f, 1.0f);
    uint16_t *Ahi = (uint16_t *)std::malloc((size_t)T * K * 2), *Alo = (uint16_t *)std::malloc((size_t)T * K * 2);
    uint8_t *W = (uint8_t *)std::malloc((size_t)N * K / 2);
    uint16_t *S = (uint16_t *)std::malloc((size_t)N * kgrp * 2);
    float *P = (float *)std::malloc((size_t)splits * T * N * 4);
    std::vector<double> act((size_t)T * K);
    for (size_t i = 0; i < (size_t)T * K; ++i) {
        const float v = ud(rng) * 3.0f;
        Ahi[i] = to_bf16(v);
        Alo[i] = to_bf16(v - emu::bf16_to_float(Ahi[i]));
        act[i] = (double)emu::bf16_to_float(Ahi[i]) + (double)emu::bf16_to_float(Alo[i]);
    }
    for (size_t i = 0; i < (size_t)N * K / 2; ++i) W[i] = (uint8_t)(rng() & 255);
    for (size_t i = 0; i < (size_t)N * kgrp; ++i) S[i] = to_bf16(0.01f + 0.02f * std::fabs(ud(rng)));
    for (size_t i = 0; i < (size_t)splits * T * N; ++i) P[i] = std::nanf("");

    PfGemm g{Ahi, Alo, W, S, P, T, N, K, sps};
    if (T <= 8) emu::launch(k_pf_gemm_skinny_i4<1, true, 1, 8>, grid, threads, lds_bytes, g);
    else if (T <= 16) emu::launch(k_pf_gemm_skinny_i4<1, false, 1, 8>, grid, threads, lds_bytes, g);
    else emu::launch(k_pf_gemm_skinny_i4<2, false, 1, 8>, grid, threads, lds_bytes, g);

    // storage format: element 2i of a row is the low nibble of byte i, offset binary (q + 8); one bf16 scale per
    // row and 128 elements
    double worst = 0.0, big = 0.0;
    long unwritten = 0;
    for (int t = 0; t < T; ++t)
        for (int n = 0; n < N; ++n) {
            double ref = 0.0;
            for (int k = 0; k < K; ++k) {
                const int nib = (W[((size_t)n * K + k) / 2] >> (4 * (k & 1))) & 15;
                ref += act[(size_t)t * K + k] * (double)(nib - 8) * (double)emu::bf16_to_float(S[(size_t)n * kgrp + k / 128]);
            }
            double got = 0.0;
            for (int z = 0; z < splits; ++z) {
                const float p = P[((size_t)z * T + t) * N + n];
                if (p != p) ++unwritten;
                got += p;
            }
            worst = std::fmax(worst, std::fabs(got - ref));
            big = std::fmax(big, std::fabs(ref));
        }
    std::printf("T %d N %d K %d: %d splits, max |kernel - fp64| = %.3g, largest value %.3g, result elements not written %ld\n", T, N, K,
                splits, worst, big, unwritten);
    std::free(Ahi); std::free(Alo); std::free(W); std::free(S); std::free(P);
    return (unwritten == 0 && worst <= 2e-5 * big) ? 0 : 1;
}
