// Finishing the sampled decode step on the GPU.
//
// The reference stops the device work of a sampled step at the per-block top-k candidates or the
// per-block softmax statistics, reads them back and draws the token on the CPU
// (engine/src/inference.rs:586-618), one host round trip per token (two with top_k == 0).  The
// kernels below do that host work on the device with the host's arithmetic, operation for
// operation, so the drawn token feeds the next step without leaving the GPU and a run of steps is
// enqueued back to back:
//   candidate merge            engine/src/decode.rs:218-253 (value desc, index asc; drops
//                              idx == u32::MAX and non-finite values)
//   draw over the candidates   engine/src/inference.rs:823-849
//   block draw from statistics engine/src/inference.rs:851-891
//   draw inside the block      engine/src/inference.rs:893-921 (+ block_idx * 256, :613)
//   uniform numbers            engine/src/inference.rs:759-768 (64-bit LCG, top 24 bits)
//   softcap of the candidates  engine/src/decode.rs:155-159 (cap * tanhf(v / cap) on the host)
// Sums run sequentially in one thread in the host's order; every float operation is written with
// a single-rounding intrinsic (or compiled with contraction off) so that the compiler cannot fuse
// a multiply into an add.
#pragma once
#include "hipdec_batch.h"
#include "hipdec_kernels.h"

// ---------------------------------------------------------------- expf with the host's bits
// exp(x) for float x the way the GNU C library's expf computes it on a host with fused
// multiply-add (x86-64 glibc >= 2.27 selects that variant at load time): in double,
// z = x * 32/ln2, k = nearest integer (by adding and subtracting 1.5 * 2^52), r = x * 32/ln2 - k as
// ONE fused operation, 2^(k/32) from a 32-entry table whose exponent field is advanced by k / 32,
// a cubic in r, one rounding to float.  The table holds 2^(i/32) rounded to double with i << 47
// subtracted from the bit pattern.  The tests compare this function on the host with the C
// library for every float below zero and up to 89, and the device against the host through
// checksums over the same ranges.
__host__ __device__ __forceinline__ uint64_t sample_exp2_tab(unsigned i) {
    constexpr uint64_t tab[32] = {
        0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
        0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
        0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
        0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
        0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
        0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
        0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
        0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};
    return tab[i & 31u];
}

__host__ __device__ inline float expf_as_host(float x) {
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0, shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0, c1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0,
                 c2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    const uint32_t xb = __builtin_bit_cast(uint32_t, x);
    const uint32_t abstop = (xb >> 20) & 0x7ffu;
    if (abstop >= 0x42bu) {                                  // |x| >= 88 or not finite
        if (xb == 0xff800000u) return 0.0f;                  // -inf
        if (abstop >= 0x7f8u) return x + x;                  // +inf, nan
        if (x > 0x1.62e42ep6f) return __builtin_inff();      // overflow
        if (x < -0x1.9fe368p6f) return 0.0f;                 // below the smallest subnormal
    }
    const double xd = (double)x;
    const double z = inv_ln2_n * xd;
    double kd = z + shift;
    const uint64_t ki = __builtin_bit_cast(uint64_t, kd);
    kd -= shift;
    const double r = __builtin_fma(inv_ln2_n, xd, -kd);
    const uint64_t t = sample_exp2_tab((unsigned)ki) + (ki << 47);
    const double s = __builtin_bit_cast(double, t);
    const double p = __builtin_fma(c0, r, c1);
    const double r2 = r * r;
    double y = __builtin_fma(c2, r, 1.0);
    y = __builtin_fma(p, r2, y);
    y = y * s;
    return (float)y;
}

// ---------------------------------------------------------------- tanhf with the host's bits
// The GNU C library's float tanh (through glibc 2.40) is the classic single-precision routine:
// tanh(x) = 1 - 2/(expm1(2|x|) + 2) for |x| >= 1, -t/(t + 2) with t = expm1(-2|x|) below, x(1 + x)
// for tiny x and 1 - 1e-30 from 22 up, on top of the single-precision expm1 (argument reduction by
// ln2 in two pieces, a degree-5 polynomial in x^2/2, reconstruction by exponent arithmetic).  It is
// plain float arithmetic with no fused operations, which is how both functions are written here;
// the tests compare them with the C library for all 2^32 floats on the host and the device
// against the host through checksums.
__host__ __device__ inline float expm1f_as_host(float x) {
#pragma clang fp contract(off)
    const float one = 1.0f, huge = 1.0e+30f, tiny = 1.0e-30f, o_threshold = 8.8721679688e+01f,
                ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f,
                q1 = -3.3333335072e-02f, q2 = 1.5873016091e-03f, q3 = -7.9365076090e-05f, q4 = 4.0082177293e-06f,
                q5 = -2.0109921195e-07f;
    float y, hi, lo, c = 0.0f, t, e;
    int k;
    uint32_t hx = __builtin_bit_cast(uint32_t, x);
    const bool neg = (hx & 0x80000000u) != 0;
    hx &= 0x7fffffffu;
    if (hx >= 0x4195b844u) {                                     // |x| >= 27 ln2
        if (hx >= 0x42b17218u) {                                 // |x| >= 88.72...
            if (hx > 0x7f800000u) return x + x;
            if (hx == 0x7f800000u) return neg ? -1.0f : x;
            if (x > o_threshold) return huge * huge;
        }
        if (neg && x + tiny < 0.0f) return tiny - one;
    }
    if (hx > 0x3eb17218u) {                                      // |x| > 0.5 ln2
        if (hx < 0x3f851592u) {                                  // and < 1.5 ln2
            if (!neg) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int)(invln2 * x + (neg ? -0.5f : 0.5f));
            t = (float)k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {                               // |x| < 2^-25
        return x;
    } else {
        k = 0;
    }
    const float hfx = 0.5f * x;
    const float hxs = x * hfx;
    const float r1 = one + hxs * (q1 + hxs * (q2 + hxs * (q3 + hxs * (q4 + hxs * q5))));
    t = 3.0f - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0f - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = x * (e - c) - c;
    e -= hxs;
    if (k == -1) return 0.5f * (x - e) - 0.5f;
    if (k == 1) {
        if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
        return one + 2.0f * (x - e);
    }
    const uint32_t kexp = (uint32_t)k << 23;
    if (k <= -2 || k > 56) {
        y = one - (e - x);
        y = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, y) + kexp);
        return y - one;
    }
    if (k < 23) {
        t = __builtin_bit_cast(float, 0x3f800000u - (0x1000000u >> k));      // 1 - 2^-k
        y = t - (e - x);
        y = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, y) + kexp);
    } else {
        t = __builtin_bit_cast(float, (uint32_t)(0x7f - k) << 23);            // 2^-k
        y = x - (e + t);
        y += one;
        y = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, y) + kexp);
    }
    return y;
}

__host__ __device__ inline float tanhf_as_host(float x) {
#pragma clang fp contract(off)
    const float one = 1.0f, two = 2.0f, tiny = 1.0e-30f;
    const uint32_t xb = __builtin_bit_cast(uint32_t, x);
    const bool neg = (xb & 0x80000000u) != 0;
    const uint32_t ix = xb & 0x7fffffffu;
    const float ax = __builtin_bit_cast(float, ix);
    float z;
    if (ix >= 0x7f800000u) return neg ? one / x - one : one / x + one;        // +-1 for inf, nan for nan
    if (ix < 0x41b00000u) {                                      // |x| < 22
        if (ix == 0) return x;
        if (ix < 0x24000000u) return x * (one + x);              // |x| < 2^-55
        if (ix >= 0x3f800000u) {
            const float t = expm1f_as_host(two * ax);
            z = one - two / (t + two);
        } else {
            const float t = expm1f_as_host(-two * ax);
            z = -t / (t + two);
        }
    } else {
        z = one - tiny;
    }
    return neg ? -z : z;
}

// which host function a verification call addresses
enum { HOSTMATH_EXPF = 0, HOSTMATH_TANHF = 1 };
__host__ __device__ __forceinline__ float hostmath_eval(int fn, float x) {
    return fn == HOSTMATH_TANHF ? tanhf_as_host(x) : expf_as_host(x);
}

// order-independent checksum of a restated function over `count` consecutive float bit patterns
__host__ __device__ __forceinline__ uint64_t hostmath_mix(int fn, uint32_t in_bits) {
    const uint32_t out = __builtin_bit_cast(uint32_t, hostmath_eval(fn, __builtin_bit_cast(float, in_bits)));
    return ((uint64_t)out + 1ull) * (0x9e3779b97f4a7c15ull ^ ((uint64_t)in_bits << 17));
}

__global__ __launch_bounds__(256) void k_hostmath_checksum(int fn, uint32_t first_bits, uint64_t count,
                                                           unsigned long long *__restrict__ out) {
    uint64_t acc = 0;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (uint64_t)gridDim.x * blockDim.x)
        acc += hostmath_mix(fn, first_bits + (uint32_t)i);
    atomicAdd(out, (unsigned long long)acc);
}

__global__ void k_hostmath_eval(int fn, const float *__restrict__ in, float *__restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = hostmath_eval(fn, in[i]);
}

// ---------------------------------------------------------------- run state
struct SampleParams {        // device-resident; written by the host before a run
    float temperature;
    float softcap;           // top-k: applied to the merged candidates; block path: to the chosen block's logits
    int top_k;
    int step;                // ring slot of the step that is running
    int ring_cap;            // steps the ring holds
    unsigned done;           // rows that have finished the running step
};

__device__ __forceinline__ bool sample_finite(float v) { return (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u; }

// engine/src/inference.rs:759-768
__device__ __forceinline__ float sample_next_f32(uint64_t &s) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return __fdiv_rn((float)(s >> 40), 16777216.0f);
}

// f32::total_cmp as an integer key; the last maximal element (Iterator::max_by, inference.rs:778-783)
__device__ __forceinline__ int sample_total_key(float f) {
    const int b = __float_as_int(f);
    return b ^ (int)(((unsigned)(b >> 31)) >> 1);
}

// what every row does once its token is drawn: publish it, and the last row to arrive moves the
// run to its next step (rows read the run state only before they arrive here)
__device__ __forceinline__ void sample_finish(uint32_t tok, uint64_t s, int row, int rows, int step, SampleParams *ss,
                                              uint64_t *rng, uint32_t *tok_out, uint32_t *ring, BatchParams *bp) {
    tok_out[row] = tok;
    if (step >= 0 && step < ss->ring_cap) ring[(size_t)step * rows + row] = tok;
    rng[row] = s;
    __threadfence();
    const unsigned arrived = atomicAdd(&ss->done, 1u);
    if (arrived == (unsigned)rows - 1u) {
        ss->done = 0;
        ss->step = step + 1;
        if (bp) { bp->pos = bp->pos + 1; bp->slot = bp->slot + 1; }
    }
}

// One workgroup per row.  vals/idxs: [rows][blocks * top_k], each block's list already in
// (value desc, index asc) order.  A thread owns blocks tid, tid + 256, ... (up to 4) and offers
// the best of their heads; top_k rounds of a workgroup-wide selection give the merged list.
#define SAMPLE_MAX_BLOCKS 1024
__global__ __launch_bounds__(256) void k_sample_topk(const float *__restrict__ vals, const uint32_t *__restrict__ idxs,
                                                     int blocks, SampleParams *ss, uint64_t *rng, uint32_t *tok_out,
                                                     uint32_t *ring, BatchParams *bp) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    __shared__ float mv[32];
    __shared__ float w[32];
    __shared__ uint32_t mi[32];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.x, rows = gridDim.x;
    const int k = ss->top_k, step = ss->step;
    const float temperature = ss->temperature, cap = ss->softcap;
    const float *v = vals + (size_t)row * blocks * k;
    const uint32_t *ix = idxs + (size_t)row * blocks * k;
    int ptr[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int b = tid + 256 * j;
        ptr[j] = k;
        if (b < blocks) {
            int p = 0;
            while (p < k && (ix[b * k + p] == 0xffffffffu || !sample_finite(v[b * k + p]))) ++p;
            ptr[j] = p;
        }
    }
    int n = 0;
    for (int rank = 0; rank < k; ++rank) {
        float cv = -INFINITY; uint32_t ci = 0xffffffffu;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int b = tid + 256 * j;
            if (b < blocks && ptr[j] < k) {
                const float hv = v[b * k + ptr[j]];
                const uint32_t hi = ix[b * k + ptr[j]];
                if (better(hv, hi, cv, ci)) { cv = hv; ci = hi; }
            }
        }
        float bv = cv; uint32_t bi = ci;
        wave_argbest(bv, bi);
        if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
        __syncthreads();
        bv = sv[0]; bi = si[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        __syncthreads();
        if (bi == 0xffffffffu) break;                          // uniform: every list is used up
        if (tid == 0) { mv[rank] = bv; mi[rank] = bi; }
        n = rank + 1;
        if (ci == bi) {                                        // the owner moves that list on
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int b = tid + 256 * j;
                if (b < blocks && ptr[j] < k && ix[b * k + ptr[j]] == bi) {
                    int p = ptr[j] + 1;
                    while (p < k && (ix[b * k + p] == 0xffffffffu || !sample_finite(v[b * k + p]))) ++p;
                    ptr[j] = p;
                }
            }
        }
    }
    if (tid != 0) return;
    if (cap > 0.0f)                                            // decode.rs:155-159
        for (int i = 0; i < n; ++i) mv[i] = __fmul_rn(cap, tanhf_as_host(__fdiv_rn(mv[i], cap)));
    uint64_t s = rng[row];
    uint32_t tok = 0;
    if (n > 0) {
        tok = mi[0];
        if (temperature > 0.0f && n > 1) {
            float mx = -INFINITY;
            for (int i = 0; i < n; ++i) mx = fmaxf(mx, mv[i]);
            float sum = 0.0f;
            for (int i = 0; i < n; ++i) {
                w[i] = expf_as_host(__fdiv_rn(__fsub_rn(mv[i], mx), temperature));
                sum = __fadd_rn(sum, w[i]);
            }
            if (sample_finite(sum) && sum > 0.0f) {
                float draw = __fmul_rn(sample_next_f32(s), sum);
                tok = mi[n - 1];
                for (int i = 0; i < n; ++i) {
                    draw = __fsub_rn(draw, w[i]);
                    if (draw <= 0.0f) { tok = mi[i]; break; }
                }
            }
        }
    }
    sample_finish(tok, s, row, rows, step, ss, rng, tok_out, ring, bp);
}

// One workgroup per row: the block from the statistics, then the token inside the block.
// logits: [rows][V] raw; maxes/sums: [rows][blocks].
__global__ __launch_bounds__(256) void k_sample_fullvocab(const float *__restrict__ logits, int V,
                                                          const float *__restrict__ maxes, const float *__restrict__ sums,
                                                          int blocks, SampleParams *ss, uint64_t *rng, uint32_t *tok_out,
                                                          uint32_t *ring, BatchParams *bp) {
    __shared__ float sw[SAMPLE_MAX_BLOCKS];
    __shared__ float sl[256];
    __shared__ float sr[4];
    __shared__ int s_blk;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.x, rows = gridDim.x;
    const int step = ss->step;
    const float temperature = ss->temperature, cap = ss->softcap;
    const float *mx_b = maxes + (size_t)row * blocks, *sm_b = sums + (size_t)row * blocks;
    // inference.rs:851-891
    float g = -INFINITY;
    for (int b = tid; b < blocks; b += 256)
        if (sample_finite(mx_b[b])) g = fmaxf(g, mx_b[b]);
    g = wave_max(g);
    if (lane == 0) sr[wave] = g;
    __syncthreads();
    g = fmaxf(fmaxf(sr[0], sr[1]), fmaxf(sr[2], sr[3]));
    const bool have = sample_finite(g);
    if (have)
        for (int b = tid; b < blocks; b += 256) {
            const float m = mx_b[b], sm = sm_b[b];
            sw[b] = (sample_finite(m) && sample_finite(sm) && sm > 0.0f) ? __fmul_rn(expf_as_host(__fsub_rn(m, g)), sm) : 0.0f;
        }
    __syncthreads();
    uint64_t s = 0;
    if (tid == 0) {
        s = rng[row];
        int blk = 0;
        if (have) {
            float total = 0.0f;
            for (int b = 0; b < blocks; ++b) total = __fadd_rn(total, sw[b]);
            if (sample_finite(total) && total > 0.0f) {
                float draw = __fmul_rn(sample_next_f32(s), total);
                blk = blocks - 1;
                for (int b = 0; b < blocks; ++b) {
                    draw = __fsub_rn(draw, sw[b]);
                    if (draw <= 0.0f) { blk = b; break; }
                }
            }
        }
        s_blk = blk;
    }
    __syncthreads();
    // inference.rs:893-921 over the softcapped logits of the block (lib.rs:1702-1723)
    const int start = s_blk * 256;
    const int valid = min(256, V - start);
    float val = -INFINITY;
    if (tid < valid) val = softcap_dev(logits[(size_t)row * V + start + tid], cap);
    sl[tid] = val;
    float mx = wave_max(val);
    __syncthreads();                                           // sr is free again, sl is complete
    if (lane == 0) sr[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(sr[0], sr[1]), fmaxf(sr[2], sr[3]));
    sw[tid] = tid < valid ? expf_as_host(__fdiv_rn(__fsub_rn(val, mx), temperature)) : 0.0f;
    __syncthreads();
    if (tid != 0) return;
    float sum = 0.0f;
    for (int i = 0; i < valid; ++i) sum = __fadd_rn(sum, sw[i]);
    int pick;
    if (!sample_finite(sum) || sum <= 0.0f) {
        pick = 0;
        int best = sample_total_key(sl[0]);
        for (int i = 1; i < valid; ++i) {
            const int key = sample_total_key(sl[i]);
            if (key >= best) { best = key; pick = i; }
        }
    } else {
        float draw = __fmul_rn(sample_next_f32(s), sum);
        pick = valid - 1;
        for (int i = 0; i < valid; ++i) {
            draw = __fsub_rn(draw, sw[i]);
            if (draw <= 0.0f) { pick = i; break; }
        }
    }
    sample_finish((uint32_t)(start + pick), s, row, rows, step, ss, rng, tok_out, ring, bp);
}
