// Shared device helpers for the gfx950 decode kernels: weight-stream decoders, wave reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

// ---------------------------------------------------------------- step parameters
// One small block of device memory carries everything that changes between two replays of a
// captured step: kernels read it instead of taking launch arguments, so one hipGraph serves
// every token.  The reference passes slot / attn_len / token as per-dispatch constants
// (crates/metal-decode/src/lib.rs:249-250, :647, :709, :743, :781).
struct StepParams {
    int tok;        // input token id
    int pos;        // slot = len before the step; attends over pos + 1 rows
    int step;       // index into the output token ring of a multi-step greedy run
    int top_k;      // head variant parameter
    float inv_t;    // block-stats 1/temperature
    float softcap;  // <= 0 disables
    int use_x_in;   // 1: the residual stream starts from x_in instead of an embedding row
    int block_idx;  // materialise: which 256-row block
};

enum { WT_F32 = 0, WT_BF16 = 1, WT_FP8 = 2, WT_INT4 = 3 };

__device__ __forceinline__ float bf16_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even fp32 -> bf16 bits (finite inputs)
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7f800000u) == 0x7f800000u) return (uint16_t)(u >> 16);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

// Sum over the 64 lanes of a wave with data-parallel-primitive moves (no LDS round trips);
// the total is valid in lane 63.  Fixed order: quads, halves of 8, rows of 16, then the rows.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_get(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v += dpp_get<0xB1, 0xf>(v);      // quad_perm [1,0,3,2]
    v += dpp_get<0x4E, 0xf>(v);      // quad_perm [2,3,0,1]
    v += dpp_get<0x141, 0xf>(v);     // row_half_mirror
    v += dpp_get<0x140, 0xf>(v);     // row_mirror: every lane of a row now holds the row's sum
    v += dpp_get<0x142, 0xa>(v);     // row_bcast:15 into rows 1 and 3
    v += dpp_get<0x143, 0xc>(v);     // row_bcast:31 into rows 2 and 3
    return v;
}
// sum over aligned groups of N lanes (8, 16 or 32); every lane of the group receives it
template <int N> __device__ __forceinline__ float group_sum_dpp(float v) {
    v += dpp_get<0xB1, 0xf>(v);
    v += dpp_get<0x4E, 0xf>(v);
    v += dpp_get<0x141, 0xf>(v);
    if (N >= 16) v += dpp_get<0x140, 0xf>(v);
    if (N >= 32) v += __shfl_xor(v, 16, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// (value desc, index asc) ordering used by every head kernel of the reference
// (crates/metal-decode/src/lib.rs:1553, :1612-1613, :1749)
__device__ __forceinline__ bool better(float v, uint32_t i, float bv, uint32_t bi) {
    return v > bv || (v == bv && i < bi);
}
__device__ __forceinline__ void wave_argbest(float &v, uint32_t &i) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ov = __shfl_xor(v, o, WAVE);
        uint32_t oi = (uint32_t)__shfl_xor((int)i, o, WAVE);
        if (better(ov, oi, v, i)) { v = ov; i = oi; }
    }
}

// 16-byte load of data that is used once per step (the weight stream of the persistent decode
// kernel): the non-temporal hint keeps it from displacing what the caches should hold (600M step
// 0.730 -> 0.708 ms, 5B 3.10 -> 2.89 ms).  Not for the multi-row streaming GEMM, where neighbouring
// lanes' 32-byte pieces share cache lines across instructions: there the hint costs 15 %.
typedef uint32_t stream_u4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld_stream_u4(const void *p) {
    const stream_u4 v = __builtin_nontemporal_load((const __attribute__((address_space(1))) stream_u4 *)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// ---------------------------------------------------------------- weight stream decoders
// Every weight matrix is stored out-major: row = output channel, reduction axis contiguous, so
// one 128-bit load gives a lane EPL consecutive reduction elements of one output row.
template <int WT> struct WS;

template <> struct WS<WT_F32> {
    static constexpr int EPL = 4;                       // elements per 16-byte load
    static __device__ __forceinline__ size_t row_bytes(int K) { return (size_t)K * 4; }
    static __device__ __forceinline__ void decode(const uint4 &w, float *f) {
        f[0] = __uint_as_float(w.x); f[1] = __uint_as_float(w.y);
        f[2] = __uint_as_float(w.z); f[3] = __uint_as_float(w.w);
    }
};
template <> struct WS<WT_BF16> {
    static constexpr int EPL = 8;
    static __device__ __forceinline__ size_t row_bytes(int K) { return (size_t)K * 2; }
    static __device__ __forceinline__ void decode(const uint4 &w, float *f) {
        f[0] = __uint_as_float(w.x << 16); f[1] = __uint_as_float(w.x & 0xffff0000u);
        f[2] = __uint_as_float(w.y << 16); f[3] = __uint_as_float(w.y & 0xffff0000u);
        f[4] = __uint_as_float(w.z << 16); f[5] = __uint_as_float(w.z & 0xffff0000u);
        f[6] = __uint_as_float(w.w << 16); f[7] = __uint_as_float(w.w & 0xffff0000u);
    }
};
template <> struct WS<WT_FP8> {
    static constexpr int EPL = 16;
    static __device__ __forceinline__ size_t row_bytes(int K) { return (size_t)K; }
    static __device__ __forceinline__ void decode(const uint4 &w, float *f) {
        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(u[i], false);   // bytes 0,1 (OCP e4m3 on gfx950)
            auto hi = __builtin_amdgcn_cvt_pk_f32_fp8(u[i], true);    // bytes 2,3
            f[4 * i + 0] = lo[0]; f[4 * i + 1] = lo[1];
            f[4 * i + 2] = hi[0]; f[4 * i + 3] = hi[1];
        }
    }
};
template <> struct WS<WT_INT4> {
    static constexpr int EPL = 32;
    static __device__ __forceinline__ size_t row_bytes(int K) { return (size_t)K / 2; }
    // Nibbles are offset-binary (q + 8); element 2j is the low nibble of byte j.  Flipping bit 3 of
    // every nibble turns them into two's complement, which v_cvt_off_f32_i4 converts to q / 16 in one
    // instruction (byte selects address the nibbles, no extract / convert / subtract chain), so the
    // decoded values are q / 16 and the caller multiplies its group scale by SCALE_MUL = 16: both
    // are exact power-of-two scalings, the products and sums are bit-identical to using q.
    static constexpr float SCALE_MUL = 16.0f;
    static __device__ __forceinline__ void decode(const uint4 &w, float *f) {
        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t lo = u[i] ^ 0x88888888u;
            uint32_t hi = lo >> 4;
            asm volatile("" : "+v"(hi));      // keeps `hi` a register of its own (otherwise its bytes are re-extracted from `lo` with one bit-field op each)
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                // (written as byte extractions so that they fold into the instruction's byte select)
                f[8 * i + 2 * b] = __builtin_amdgcn_cvt_off_f32_i4(b == 0 ? (int)lo : (int)((lo >> (8 * b)) & 0xffu));
                f[8 * i + 2 * b + 1] = __builtin_amdgcn_cvt_off_f32_i4((int)((hi >> (8 * b)) & 0xffu));
            }
        }
    }
};

// software OCP e4m3fn encoder, round to nearest even, saturating (used once, at weight load)
__device__ __forceinline__ uint8_t f32_to_e4m3(float f) {
    uint32_t u = __float_as_uint(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    float a = fabsf(f);
    if (a != a) return sign | 0x7f;
    if (a >= 464.0f) return sign | 0x7e;
    if (a < 0.0009765625f) return sign;
    int e;
    float mant = frexpf(a, &e);
    int ex = e - 1;
    if (ex < -6) {
        int qi = (int)rintf(a * 512.0f);
        if (qi >= 8) return sign | 0x08;
        return sign | (uint8_t)qi;
    }
    int mi = (int)rintf((2.0f * mant - 1.0f) * 8.0f);
    if (mi == 8) { mi = 0; ex += 1; }
    if (ex > 8 || (ex == 8 && mi > 6)) return sign | 0x7e;
    return sign | (uint8_t)(((ex + 7) << 3) | mi);
}
