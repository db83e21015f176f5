// The general few-row GEMM kernel's own source (kernel_few.inc: cut out of hipdec_prefill.h by the test, with the
// helpers it calls) run on the CPU for one of the four weight formats under the launch plan given on the command
// line, on seeded random operands, against a plain fp64 product of the stored weights.  Every operand lives in a heap
// block of its exact size: with -fsanitize=address an access outside any of them ends the program with a report.
// usage: few_row_general weight_format(0 fp32, 1 bf16, 2 e4m3, 3 4-bit) T N K steps_per_split gx gy gz threads lds_bytes seed
#include "emu.h"
#define PF_BK 32
typedef float pf_f32x16 __attribute__((ext_vector_type(16)));
#include "pfgemm_struct.inc"
#include "kernel_few.inc"
#include <cstdio>
#include <random>

static uint16_t to_bf16(float v) { return f32_to_bf16_rne(v); }

int main(int argc, char **argv) {
    if (argc != 12) { std::fprintf(stderr, "usage: few_row_general wt T N K steps_per_split gx gy gz threads lds_bytes seed\n"); return 2; }
    const int wt = atoi(argv[1]), T = atoi(argv[2]), N = atoi(argv[3]), K = atoi(argv[4]), sps = atoi(argv[5]);
    const dim3 grid{(unsigned)atoi(argv[6]), (unsigned)atoi(argv[7]), (unsigned)atoi(argv[8])};
    const unsigned threads = (unsigned)atoi(argv[9]);
    const size_t lds_bytes = (size_t)atoll(argv[10]);
    if (wt < 0 || wt > 3 || threads != 256 || T < 1 || T > 32 || K % 32 || (wt == 3 && K % 128) || grid.z != 1) { std::fprintf(stderr, "not a launch of this kernel\n"); return 2; }
    const int kgrp = K / 128, splits = (int)grid.y;
    std::mt19937 rng((unsigned)atoi(argv[11]));
    std::uniform_real_distribution<float> ud(-1.0f, 1.0f);
    const size_t wbytes = wt == 0 ? (size_t)N * K * 4 : wt == 1 ? (size_t)N * K * 2 : wt == 2 ? (size_t)N * K : (size_t)N * K / 2;
    uint16_t *Ahi = (uint16_t *)std::malloc((size_t)T * K * 2), *Alo = (uint16_t *)std::malloc((size_t)T * K * 2);
    uint8_t *W = (uint8_t *)std::malloc(wbytes);
    uint16_t *S = wt == 3 ? (uint16_t *)std::malloc((size_t)N * kgrp * 2) : nullptr;
    float *P = (float *)std::malloc((size_t)splits * T * N * 4);
    std::vector<double> act((size_t)T * K), wv((size_t)N * K);
    for (size_t i = 0; i < (size_t)T * K; ++i) {
        const float v = ud(rng) * 3.0f;
        Ahi[i] = to_bf16(v);
        Alo[i] = to_bf16(v - bf16_to_f32(Ahi[i]));
        act[i] = (double)bf16_to_f32(Ahi[i]) + (double)bf16_to_f32(Alo[i]);
    }
    if (wt == 3) for (size_t i = 0; i < (size_t)N * kgrp; ++i) S[i] = to_bf16(0.01f + 0.02f * std::fabs(ud(rng)));
    for (size_t i = 0; i < (size_t)N * K; ++i) {
        const int n = (int)(i / K), k = (int)(i % K);
        if (wt == 0) { const float v = ud(rng) * 0.3f; ((float *)W)[i] = v; wv[i] = v; }
        else if (wt == 1) { const uint16_t h = to_bf16(ud(rng) * 0.3f); ((uint16_t *)W)[i] = h; wv[i] = bf16_to_f32(h); }
        else if (wt == 2) { uint8_t b = (uint8_t)(rng() & 255); if ((b & 0x7f) == 0x7f) b &= 0x7e; W[i] = b; wv[i] = emu::e4m3_to_float(b); }
        else {
            // element 2i of a row is the low nibble of byte i, offset binary (q + 8); one bf16 scale per row and 128 elements
            const int nib = (int)(rng() & 15);
            uint8_t &byte = W[i / 2];
            byte = (k & 1) ? (uint8_t)((byte & 0x0f) | (nib << 4)) : (uint8_t)nib;
            wv[i] = (double)(nib - 8) * (double)bf16_to_f32(S[(size_t)n * kgrp + k / 128]);
        }
    }
    for (size_t i = 0; i < (size_t)splits * T * N; ++i) P[i] = std::nanf("");

    PfGemm g{Ahi, Alo, W, S, P, T, N, K, sps};
    if (wt == 0) emu::launch(k_pf_gemm_skinny<WT_F32>, grid, threads, lds_bytes, g);
    else if (wt == 1) emu::launch(k_pf_gemm_skinny<WT_BF16>, grid, threads, lds_bytes, g);
    else if (wt == 2) emu::launch(k_pf_gemm_skinny<WT_FP8>, grid, threads, lds_bytes, g);
    else emu::launch(k_pf_gemm_skinny<WT_INT4>, grid, threads, lds_bytes, g);

    double worst = 0.0, big = 0.0;
    long unwritten = 0;
    for (int t = 0; t < T; ++t)
        for (int n = 0; n < N; ++n) {
            double ref = 0.0;
            for (int k = 0; k < K; ++k) ref += act[(size_t)t * K + k] * wv[(size_t)n * K + k];
            double got = 0.0;
            for (int z = 0; z < splits; ++z) {
                const float p = P[((size_t)z * T + t) * N + n];
                if (p != p) ++unwritten;
                got += p;
            }
            worst = std::fmax(worst, std::fabs(got - ref));
            big = std::fmax(big, std::fabs(ref));
        }
    std::printf("format %d T %d N %d K %d: %d splits, max |kernel - fp64| = %.3g, largest value %.3g, result elements not written %ld\n", wt, T, N,
                K, splits, worst, big, unwritten);
    std::free(Ahi); std::free(Alo); std::free(W); std::free(S); std::free(P);
    // fp32 weights enter as (hi, lo) bf16 pairs: what is dropped is 2^-16 of a product
    return (unwritten == 0 && worst <= (wt == 0 ? 1e-4 : 2e-5) * big) ? 0 : 1;
}
