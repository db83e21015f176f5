// The e4m3 few-row GEMM kernel's own source (kernel_f8.inc: cut out of hipdec_prefill.h by the test) run on the CPU
// under the launch plan given on the command line, on seeded random operands, against a plain fp64 product (the
// per-row scale is applied by the kernel that sums the planes, so none is involved here).  Every operand lives in a
// heap block of its exact size: with -fsanitize=address an access outside any of them ends the program with a report.
// usage: few_row_f8 T N K steps_per_split gx gy gz threads lds_bytes seed
#include "emu.h"
#define PF_BK 32
#define PF_SK_PAD 8
typedef float pf_f32x4 __attribute__((ext_vector_type(4)));
#include "pfgemm_struct.inc"
#include "kernel_f8.inc"
#include <cstdio>
#include <random>

static uint16_t to_bf16(float v) { uint32_t u; std::memcpy(&u, &v, 4); u += 0x7fff + ((u >> 16) & 1); return (uint16_t)(u >> 16); }

int main(int argc, char **argv) {
    if (argc != 11) { std::fprintf(stderr, "usage: few_row_f8 T N K steps_per_split gx gy gz threads lds_bytes seed\n"); return 2; }
    const int T = atoi(argv[1]), N = atoi(argv[2]), K = atoi(argv[3]), sps = atoi(argv[4]);
    const dim3 grid{(unsigned)atoi(argv[5]), (unsigned)atoi(argv[6]), (unsigned)atoi(argv[7])};
    const unsigned threads = (unsigned)atoi(argv[8]);
    const size_t lds_bytes = (size_t)atoll(argv[9]);
    if (threads != 64 * EMU_F8_WAVES || T < 1 || T > 32 || K % 64 || grid.z != 1) { std::fprintf(stderr, "not a launch of this kernel\n"); return 2; }
    const int splits = (int)grid.y;
    std::mt19937 rng((unsigned)atoi(argv[10]));
    std::uniform_real_distribution<float> ud(-1.0f, 1.0f);
    uint16_t *Ahi = (uint16_t *)std::malloc((size_t)T * K * 2), *Alo = (uint16_t *)std::malloc((size_t)T * K * 2);
    uint8_t *W = (uint8_t *)std::malloc((size_t)N * K);
    float *P = (float *)std::malloc((size_t)splits * T * N * 4);
    std::vector<double> act((size_t)T * K);
    for (size_t i = 0; i < (size_t)T * K; ++i) {
        const float v = ud(rng) * 3.0f;
        Ahi[i] = to_bf16(v);
        Alo[i] = to_bf16(v - emu::bf16_to_float(Ahi[i]));
        act[i] = (double)emu::bf16_to_float(Ahi[i]) + (double)emu::bf16_to_float(Alo[i]);
    }
    for (size_t i = 0; i < (size_t)N * K; ++i) {
        uint8_t b = (uint8_t)(rng() & 255);
        if ((b & 0x7f) == 0x7f) b &= 0x7e;                   // (no NaN codes: stored weights never hold one)
        W[i] = b;
    }
    for (size_t i = 0; i < (size_t)splits * T * N; ++i) P[i] = std::nanf("");

    PfGemm g{Ahi, Alo, W, nullptr, P, T, N, K, sps};
    if (T <= 8) emu::launch(EMU_F8_KERNEL(1, true), grid, threads, lds_bytes, g);
    else if (T <= 16) emu::launch(EMU_F8_KERNEL(1, false), grid, threads, lds_bytes, g);
    else emu::launch(EMU_F8_KERNEL(2, false), grid, threads, lds_bytes, g);

    double worst = 0.0, big = 0.0;
    long unwritten = 0;
    for (int t = 0; t < T; ++t)
        for (int n = 0; n < N; ++n) {
            double ref = 0.0;
            for (int k = 0; k < K; ++k) ref += act[(size_t)t * K + k] * (double)emu::e4m3_to_float(W[(size_t)n * K + k]);
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
    std::free(Ahi); std::free(Alo); std::free(W); std::free(P);
    return (unwritten == 0 && worst <= 2e-5 * big) ? 0 : 1;
}
