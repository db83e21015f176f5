// The weight conversion kernel (kernel_convert.inc: k_convert_rows with the e4m3 encoder, cut out of hipdec_kernels.h
// and hipdec_common.h by the test) run on the CPU: stored e4m3 rows with their per-row scale and stored 4-bit rows
// with their bf16 group scales, bit for bit against the oracle's quantisers (oracle/rustane_oracle.c, linked in as the
// checker), including rows and groups of zeros, magnitudes from 1e-6 to 1e4 and the interleaving row map.
#include "emu.h"
#include "kernel_convert.inc"
#include <cstdio>
#include <random>

extern "C" void orc_quant_fp8_rows(const float *W, int O, int K, uint8_t *q, float *scale, float *dequant);
extern "C" void orc_quant_int4_g128(const float *W, int O, int K, int8_t *q, float *scale, float *dequant);

static std::mt19937 rng(5);
static int failures = 0;

static void convert_case(int rows, int K, int row_mul, int row_off) {
    float *src = (float *)std::malloc((size_t)rows * K * 4);
    for (int r = 0; r < rows; ++r) {
        const float mag = std::pow(10.0f, (float)((int)(rng() % 11) - 6));
        for (int k = 0; k < K; ++k) src[(size_t)r * K + k] = std::uniform_real_distribution<float>(-1.0f, 1.0f)(rng) * mag;
        if (r == 1) for (int k = 0; k < K; ++k) src[(size_t)r * K + k] = 0.0f;                       // a row of zeros
        if (r == 2) for (int k = 0; k < 128 && k < K; ++k) src[(size_t)r * K + k] = 0.0f;            // a group of zeros
        if (r == 3) for (int k = 0; k < K; ++k) src[(size_t)r * K + k] = (float)((k % 16) - 8) * 0.5f;  // exact halves: ties of the rounding
    }
    const size_t drows = (size_t)rows * row_mul;
    long bad = 0;
    {   // e4m3 with a scale per row
        uint8_t *dst = (uint8_t *)std::malloc(drows * K);
        float *sc = (float *)std::malloc(drows * 4);
        std::memset(dst, 0xAA, drows * K);
        emu::launch_fn([&] { k_convert_rows<WT_FP8>(src, dst, sc, K, row_mul, row_off); }, dim3{(unsigned)rows, 1, 1}, 256, 0);
        std::vector<uint8_t> q((size_t)rows * K);
        std::vector<float> s(rows);
        orc_quant_fp8_rows(src, rows, K, q.data(), s.data(), nullptr);
        for (int r = 0; r < rows; ++r) {
            const size_t d = (size_t)r * row_mul + row_off;
            if (std::memcmp(&sc[d], &s[r], 4)) ++bad;
            if (std::memcmp(dst + d * K, q.data() + (size_t)r * K, K)) ++bad;
        }
        std::free(dst); std::free(sc);
    }
    if (K % 128 == 0) {   // 4-bit, groups of 128 with a bf16 scale
        const int G = K / 128;
        uint8_t *dst = (uint8_t *)std::malloc(drows * K / 2);
        uint16_t *sc = (uint16_t *)std::malloc(drows * G * 2);
        emu::launch_fn([&] { k_convert_rows<WT_INT4>(src, dst, sc, K, row_mul, row_off); }, dim3{(unsigned)rows, 1, 1}, 256, 0);
        std::vector<int8_t> q((size_t)rows * K);
        std::vector<float> s((size_t)rows * G);
        orc_quant_int4_g128(src, rows, K, q.data(), s.data(), nullptr);
        for (int r = 0; r < rows; ++r) {
            const size_t d = (size_t)r * row_mul + row_off;
            for (int g = 0; g < G; ++g) if (bf16_to_f32(sc[d * G + g]) != s[(size_t)r * G + g]) ++bad;
            for (int k = 0; k < K; ++k) {
                const int nib = (dst[d * (K / 2) + k / 2] >> (4 * (k & 1))) & 15;          // element 2i = low nibble of byte i, offset binary
                if (nib - 8 != q[(size_t)r * K + k]) ++bad;
            }
        }
        std::free(dst); std::free(sc);
    }
    {   // bf16, round to nearest even
        uint16_t *dst = (uint16_t *)std::malloc(drows * K * 2);
        emu::launch_fn([&] { k_convert_rows<WT_BF16>(src, dst, nullptr, K, row_mul, row_off); }, dim3{(unsigned)rows, 1, 1}, 256, 0);
        for (int r = 0; r < rows; ++r)
            for (int k = 0; k < K; ++k) {
                const float v = src[(size_t)r * K + k], got = bf16_to_f32(dst[((size_t)r * row_mul + row_off) * K + k]);
                // the nearest bf16 number: within half a unit of 8 bits, and no other candidate is nearer
                if (std::fabs(got - v) > std::fabs(v) * (1.0f / 256.0f)) ++bad;
            }
        std::free(dst);
    }
    std::printf("k_convert_rows rows %d K %d row map %d r + %d: %ld mismatches%s\n", rows, K, row_mul, row_off, bad, bad ? "  FAIL" : "");
    if (bad) ++failures;
    std::free(src);
}

int main() {
    convert_case(6, 384, 1, 0);
    convert_case(5, 1152, 2, 1);      // the gate / up interleave: destination row 2 r + 1
    convert_case(4, 320, 1, 0);       // not a multiple of 128: e4m3 and bf16 only
    convert_case(7, 128, 2, 0);
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}
