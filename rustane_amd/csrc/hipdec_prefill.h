// Prompt prefill for gfx950: all prompt rows of a chunk go through each layer together.
//
// The reference prefills on the Apple Neural Engine (engine/src/inference.rs:136-144, the graphs of
// engine/src/kernels/sdpa_fwd.rs, dyn_matmul.rs, ffn_fused.rs); this file is the same arithmetic
// (crates/engine/src/layer.rs:1287-1431) laid out for matrix cores:
//
//  * the four projections of a layer are GEMMs  P[t][n] = sum_k A[t][k] * W[n][k]  on the bf16 MFMA
//    (32x32x16).  Activations stay fp32-grade: every activation is carried as the sum of two bf16
//    numbers (hi = rne(v), lo = rne(v - hi), 16 mantissa bits together) and each weight tile is
//    multiplied by both, so the products lose nothing against the fp32 token path beyond the
//    accumulation order.  8-bit weights are widened to bf16 (exact) on their way into LDS and their
//    per-row scale is applied to the finished sum;
//  * a GEMM may be split along K over blockIdx.z; the partial planes are summed in a fixed order by
//    the element-wise kernel that consumes them (RoPE + cache write, residual + RMSNorm, gate);
//  * attention runs on the fp32 MFMA (32x32x2): one wave per (head, 32 query rows) walks the key
//    tiles with an online softmax, scores kept transposed so that the probabilities are already in
//    operand layout for the P.V product.
#pragma once
#include "hipdec_kernels.h"

typedef __bf16 pf_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pf_f32x16 __attribute__((ext_vector_type(16)));

#define PF_BM 128           // prompt rows per GEMM workgroup tile
// weight rows (output channels) per GEMM workgroup tile (a wave owns half of them as 32-wide
// matrix-core tiles): the widest that still leaves two workgroups per CU.  e4m3 tiles need half the
// staging registers of bf16 ones, so they can be 256 wide (5B, 512 rows: 25.2 -> 19.5 ms); bf16 at
// 256 spills 11 registers at two workgroups per CU (48 ms) and is slower at one (39.7 - 43.9 ms
// against 40 ms at 128); 4-bit tiles carry a second accumulator set and stay at one workgroup per CU.
#define PF_BN_OF(WT) ((WT) == WT_FP8 ? 256 : 128)
#define PF_BK 32            // reduction elements per step of the streaming (few-row) GEMM; K must be a multiple
#define PF_BKL 64           // reduction elements per step of the tiled GEMM
#define PF_LDS_STRIDE 72    // bf16 elements per LDS tile row (144 bytes: 16-byte aligned; 16 consecutive rows
                            // start 36 banks apart, so a 128-bit operand read by 16 lanes touches every bank once)

// f16 != 0: the activation as ONE fp16 number in hi (11 mantissa bits, saturating at the fp16 range; lo unused)
__device__ __forceinline__ void pf_split(float v, uint16_t &hi, uint16_t &lo, int f16 = 0) {
    if (f16) {
        const _Float16 h = (_Float16)fminf(fmaxf(v, -65504.0f), 65504.0f);
        hi = __builtin_bit_cast(uint16_t, h);
        lo = 0;
        return;
    }
    hi = f32_to_bf16_rne(v);
    lo = f32_to_bf16_rne(v - bf16_to_f32(hi));
}

typedef __bf16 pf_bf16x2 __attribute__((ext_vector_type(2)));
typedef float pf_f32x2 __attribute__((ext_vector_type(2)));
// two floats as packed bf16 (round to nearest even, in hardware), and as a (hi, lo) pair of such words
__device__ __forceinline__ uint32_t pf_pack_bf16(float a, float b) {
    const pf_f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, pf_bf16x2));
}
__device__ __forceinline__ void pf_split2(float a, float b, uint32_t &hi, uint32_t &lo) {
    hi = pf_pack_bf16(a, b);
    lo = pf_pack_bf16(a - __uint_as_float(hi << 16), b - __uint_as_float(hi & 0xffff0000u));
}

__device__ __forceinline__ float pf_block_sum(float v, float *red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nw; ++w) t += red[w];
    return t;
}

// RMSNorm (cpu/rmsnorm.rs:149-183) is split so that no kernel has to wait for a whole row: the
// kernel that produces a residual row writes x * gamma as the hi/lo pair and, per 256-element
// chunk, the sum of squares; the kernel that consumes the following GEMM multiplies its sums by
// inv[t] = 1 / sqrt(sum_chunks / D + eps), which commutes with the product.
#define PF_CHUNK 256
__device__ __forceinline__ float pf_row_inv(const float *__restrict__ ssq, int t, int nch, int D) {
    float s = 0.0f;
    for (int c = 0; c < nch; c += 8) {                   // eight loads in flight, added in chunk order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = ssq[t * nch + min(c + u, nch - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (c + u < nch) s += v[u];
    }
    return 1.0f / sqrtf(s * (1.0f / (float)D) + 1e-5f);
}

// The same for a wave whose lanes all work on row t, in two halves: lane c requests chunk sum c (one load,
// issued beside the kernel's own loads instead of nch dependent ones per thread), and once those have
// come back the wave adds them up with shuffles.
__device__ __forceinline__ float pf_row_part(const float *__restrict__ ssq, int t, int nch) {
    float s = 0.0f;
    for (int c = threadIdx.x & 63; c < nch; c += 64) s += ssq[t * nch + c];
    return s;
}
__device__ __forceinline__ float pf_row_finish(float part, int D) {
    return 1.0f / sqrtf(wave_sum(part) * (1.0f / (float)D) + 1e-5f);
}

// s[0..W) += sum over the split planes of the W floats at offset o, in plane order.  U planes are
// requested at a time (past the last plane the last one is requested again and not added): a loop
// of one load and one add per plane is a chain of `splits` round trips to the L2, which is what
// these small kernels' run time consists of.
template <int W, int U>
__device__ __forceinline__ void pf_sum_planes_u(const float *__restrict__ P, int splits, size_t plane, size_t o, float *s) {
    typedef float vt __attribute__((ext_vector_type(W)));
    for (int z = 0; z < splits; z += U) {
        vt p[U];
#pragma unroll
        for (int u = 0; u < U; ++u) p[u] = *(const vt *)(P + (size_t)min(z + u, splits - 1) * plane + o);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (z + u < splits) {
#pragma unroll
                for (int e = 0; e < W; ++e) s[e] += p[u][e];
            }
        }
    }
}
template <int W>
__device__ __forceinline__ void pf_sum_planes(const float *__restrict__ P, int splits, size_t plane, size_t o, float *s) {
    if (splits > 4) pf_sum_planes_u<W, 8>(P, splits, plane, o, s);
    else pf_sum_planes_u<W, 4>(P, splits, plane, o, s);
}

// x[t] = embed[ids[t]] (cpu/embedding.rs:8-16); hi/lo = x * gamma1 of the first layer; chunk sums of squares.
// grid (chunks, rows)
template <int EWT>
__global__ __launch_bounds__(PF_CHUNK) void k_pf_embed(const void *__restrict__ embed, const uint32_t *__restrict__ ids,
                                                       float *__restrict__ x, const float *__restrict__ gamma,
                                                       uint16_t *__restrict__ hi, uint16_t *__restrict__ lo,
                                                       float *__restrict__ ssq, int D, int f16) {
    __shared__ float red[8];
    const int t = blockIdx.y, d = blockIdx.x * PF_CHUNK + threadIdx.x;
    float v = 0.0f;
    if (d < D) {
        const size_t tok = ids[t];
        v = EWT == WT_F32 ? ((const float *)embed)[tok * D + d] : bf16_to_f32(((const uint16_t *)embed)[tok * D + d]);
        x[(size_t)t * D + d] = v;
        pf_split(v * gamma[d], hi[(size_t)t * D + d], lo[(size_t)t * D + d], f16);
    }
    const float ss = pf_block_sum(v * v, red);
    if (threadIdx.x == 0) ssq[t * gridDim.x + blockIdx.x] = ss;
}

// out[t][d] = resid[t][d] + alpha * scale[d] * sum_z P[z][t][d]   (layer.rs:1397-1405, :1300);
// hi/lo = out * gamma for the next GEMM (gamma == nullptr: none); chunk sums of squares.  grid (chunks, rows)
__global__ __launch_bounds__(256) void k_pf_resid(const float *__restrict__ P, int splits, size_t plane,
                                                 const float *__restrict__ wscale, const float *__restrict__ resid,
                                                 float alpha, float *__restrict__ out, const float *__restrict__ gamma,
                                                 uint16_t *__restrict__ hi, uint16_t *__restrict__ lo,
                                                 float *__restrict__ ssq, int D, int nch, int f16) {
    // a wave per 256-element chunk, four neighbouring elements per lane (D is a multiple of 4); grid (ceil(nch / 4), rows)
    const int t = blockIdx.y, chunk = blockIdx.x * 4 + (threadIdx.x >> 6), d = chunk * PF_CHUNK + 4 * (threadIdx.x & 63);
    if (chunk >= nch) return;
    float ss = 0.0f;
    if (d < D) {
        const size_t o = (size_t)t * D + d;
        float sv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        pf_sum_planes<4>(P, splits, plane, o, sv);
        float4 s = make_float4(sv[0], sv[1], sv[2], sv[3]);
        if (wscale) {
            const float4 ws = *(const float4 *)(wscale + d);
            s.x *= ws.x; s.y *= ws.y; s.z *= ws.z; s.w *= ws.w;
        }
        const float4 rs = *(const float4 *)(resid + o);
        const float4 v = make_float4(rs.x + alpha * s.x, rs.y + alpha * s.y, rs.z + alpha * s.z, rs.w + alpha * s.w);
        *(float4 *)(out + o) = v;
        if (gamma) {
            const float4 gm = *(const float4 *)(gamma + d);
            uint16_t h0, l0, h1, l1, h2, l2, h3, l3;
            pf_split(v.x * gm.x, h0, l0, f16); pf_split(v.y * gm.y, h1, l1, f16);
            pf_split(v.z * gm.z, h2, l2, f16); pf_split(v.w * gm.w, h3, l3, f16);
            *(uint2 *)(hi + o) = make_uint2((uint32_t)h0 | ((uint32_t)h1 << 16), (uint32_t)h2 | ((uint32_t)h3 << 16));
            *(uint2 *)(lo + o) = make_uint2((uint32_t)l0 | ((uint32_t)l1 << 16), (uint32_t)l2 | ((uint32_t)l3 << 16));
        }
        ss = (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) ssq[t * nch + chunk] = ss;
}

// q/k/v rows of the chunk: sum the split planes, scale (8-bit weights), RoPE on interleaved pairs
// (kernels/sdpa_fwd.rs:18-33, :258-321), q kept as fp32, k and v written into the caches at
// positions pos0 + t in cache precision.  One thread per (row, two channel pairs): the q, k and v
// sections are multiples of 4 channels wide, so the two pairs lie in the same section and head.
template <int KVBF16>
__global__ __launch_bounds__(256) void k_pf_qkv_epi(const float *__restrict__ P, int splits, size_t plane,
                                                    const float *__restrict__ wscale, float *__restrict__ q,
                                                    void *__restrict__ kc, void *__restrict__ vc,
                                                    const float *__restrict__ rope_cos, const float *__restrict__ rope_sin,
                                                    const float *__restrict__ ssq, int nch, int D,
                                                    int T, int Q, int KV, int hd, int pos0) {
    // grid (ceil(N / 4 / 256), rows): no division to find the row, and one row factor per workgroup
    const int N = Q + 2 * KV, t = blockIdx.y, row0 = 4 * (int)(blockIdx.x * blockDim.x + threadIdx.x);
    const float part = pf_row_part(ssq, t, nch);
    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (row0 < N) {
        pf_sum_planes<4>(P, splits, plane, (size_t)t * N + row0, s);
    }
    const float inv = pf_row_finish(part, D);
    if (row0 >= N) return;
    if (wscale) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] *= wscale[row0 + e];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] *= inv;
    const int pos = pos0 + t;
    if (row0 < Q + KV) {
        const int rr = row0 < Q ? row0 : row0 - Q;
        const int pi2 = (rr & (hd - 1)) >> 1;          // (hd is 64 or 128)
        const float2 c = *(const float2 *)(rope_cos + (size_t)pos * (hd / 2) + pi2);
        const float2 sn = *(const float2 *)(rope_sin + (size_t)pos * (hd / 2) + pi2);
        const float e0 = s[0] * c.x - s[1] * sn.x, o0 = s[1] * c.x + s[0] * sn.x;
        const float e1 = s[2] * c.y - s[3] * sn.y, o1 = s[3] * c.y + s[2] * sn.y;
        s[0] = e0; s[1] = o0; s[2] = e1; s[3] = o1;
    }
    if (row0 < Q) {
        *(float4 *)(q + (size_t)t * Q + row0) = make_float4(s[0], s[1], s[2], s[3]);
    } else {
        const bool isk = row0 < Q + KV;
        const int rr = isk ? row0 - Q : row0 - Q - KV;
        void *cache = isk ? kc : vc;
        if (KVBF16) {
            uint16_t *cp = (uint16_t *)cache + (size_t)pos * KV + rr;
            *(uint2 *)cp = make_uint2((uint32_t)f32_to_bf16_rne(s[0]) | ((uint32_t)f32_to_bf16_rne(s[1]) << 16),
                                      (uint32_t)f32_to_bf16_rne(s[2]) | ((uint32_t)f32_to_bf16_rne(s[3]) << 16));
        } else {
            *(float4 *)((float *)cache + (size_t)pos * KV + rr) = make_float4(s[0], s[1], s[2], s[3]);
        }
    }
}

// gate[t][j] = act(h1) * h3 with h1 = row 2j and h3 = row 2j+1 of the interleaved gate/up product
// (kernels/ffn_fused.rs:114-150), written as the hi/lo pair the down projection reads.  One thread
// per four gate elements of a row (H % 4 == 0): 32 bytes of each plane in, 8 + 8 bytes out, the row
// factor computed once.
__global__ __launch_bounds__(256) void k_pf_gate_epi(const float *__restrict__ P, int splits, size_t plane,
                                                     const float *__restrict__ wscale, uint16_t *__restrict__ hi,
                                                     uint16_t *__restrict__ lo, const float *__restrict__ ssq, int nch,
                                                     int D, int T, int H, int act, int f16) {
    // grid (ceil(H / 4 / 256), rows)
    const int t = blockIdx.y, j = 4 * (int)(blockIdx.x * blockDim.x + threadIdx.x);
    const float part = pf_row_part(ssq, t, nch);
    float h[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (j < H) {
        // (two requests of 16 bytes per plane, four planes at a time)
        pf_sum_planes_u<4, 4>(P, splits, plane, (size_t)t * 2 * H + 2 * j, h);
        pf_sum_planes_u<4, 4>(P, splits, plane, (size_t)t * 2 * H + 2 * j + 4, h + 4);
    }
    const float inv = pf_row_finish(part, D);
    if (j >= H) return;
    if (wscale) {
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] *= wscale[2 * j + e];
    }
    uint16_t oh[4], ol[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float h1 = h[2 * e] * inv, h3 = h[2 * e + 1] * inv;
        float g;
        if (act == 1) { const float lr = h1 > 0.0f ? h1 : 0.5f * h1; g = lr * lr * h3; }
        else { const float sig = 1.0f / (1.0f + expf(-h1)); g = h1 * sig * h3; }
        pf_split(g, oh[e], ol[e], f16);
    }
    const size_t o = (size_t)t * H + j;
    *(uint2 *)(hi + o) = make_uint2((uint32_t)oh[0] | ((uint32_t)oh[1] << 16), (uint32_t)oh[2] | ((uint32_t)oh[3] << 16));
    *(uint2 *)(lo + o) = make_uint2((uint32_t)ol[0] | ((uint32_t)ol[1] << 16), (uint32_t)ol[2] | ((uint32_t)ol[3] << 16));
}

// ---------------------------------------------------------------- GEMM on the bf16 matrix cores
struct PfGemm {
    const uint16_t *Ahi, *Alo;   // activations [T][K], hi and lo parts
    const void *W;               // weights [N][K]: bf16, e4m3, or 4-bit (two per byte)
    const uint16_t *S;           // 4-bit weights: bf16 scale per row and 128 reduction elements, [N][K/128]
    float *P;                    // partial planes [splits][T][N]
    int T, N, K;
    int steps_per_split;         // reduction steps (PF_BKL tiled, PF_BK streaming) each K split covers
};

__device__ __forceinline__ pf_bf16x8 pf_frag(const uint16_t *p) {
    const uint4 v = *(const uint4 *)p;
    return __builtin_bit_cast(pf_bf16x8, v);
}

// 256 threads = 4 waves in a 2 x 2 arrangement; each wave owns 64 rows x PF_BN / 2 channels =
// 2 x (PF_BN / 64) MFMA tiles.  Operand layout of v_mfma_f32_32x32x16_bf16: lane l supplies row
// (l % 32), reduction elements 8 * (l / 32) .. + 7 of both operands; result register i of lane l is
// C[8 * (i / 4) + 4 * (l / 32) + i % 4][l % 32].
// ACT: how the activations arrive.  PF_ACT_PAIR: two bf16 numbers (hi, lo), each weight tile multiplies both;
// PF_ACT_BF16: the hi parts only (8 mantissa bits, half the matrix work); PF_ACT_F16: one fp16 number in
// hi (11 mantissa bits, half the matrix work): the weight tile is widened to fp16 on its way into LDS
// (exact for bf16, e4m3 and 4-bit values down to 2^-24) and the product runs on the fp16 matrix instruction.
enum { PF_ACT_PAIR = 0, PF_ACT_BF16 = 1, PF_ACT_F16 = 2 };
typedef _Float16 pf_f16x8 __attribute__((ext_vector_type(8)));
typedef __fp16 pf_h2 __attribute__((ext_vector_type(2)));
// two fp32 values that are exactly representable -> packed fp16 (the rounding mode never applies)
__device__ __forceinline__ uint32_t pf_pack_f16(float a, float b) {
    const pf_h2 h = __builtin_amdgcn_cvt_pkrtz(a, b);
    return __builtin_bit_cast(uint32_t, h);
}
// a 32-bit word holding two bf16 numbers -> the same two numbers as fp16
__device__ __forceinline__ uint32_t pf_bf16x2_to_f16x2(uint32_t w) {
    return pf_pack_f16(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u));
}
__device__ __forceinline__ pf_f32x16 pf_mma(const uint4 &a, const uint4 &b, pf_f32x16 c, bool f16) {
    if (f16) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_f16x8, a), __builtin_bit_cast(pf_f16x8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, a), __builtin_bit_cast(pf_bf16x8, b), c, 0, 0, 0);
}
template <int WT, int ACT = PF_ACT_PAIR>
__global__ __launch_bounds__(256, WT == WT_INT4 ? 1 : 2) void k_pf_gemm(PfGemm g) {
    constexpr bool LO = ACT == PF_ACT_PAIR;
    constexpr bool F16 = ACT == PF_ACT_F16;
    constexpr int PF_BN = PF_BN_OF(WT);
    __shared__ __align__(16) uint16_t sAh[PF_BM * PF_LDS_STRIDE];
    __shared__ __align__(16) uint16_t sAl[PF_BM * PF_LDS_STRIDE];
    __shared__ __align__(16) uint16_t sW[PF_BN * PF_LDS_STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int n0 = blockIdx.x * PF_BN, t0 = blockIdx.y * PF_BM, z = blockIdx.z;
    const int nsteps = (g.K + PF_BKL - 1) / PF_BKL;
    const int s_begin = z * g.steps_per_split, s_end = min(nsteps, s_begin + g.steps_per_split);

    constexpr int NT = PF_BN / 64;             // 32-channel tiles per wave (a wave owns PF_BN / 2 channels)
    constexpr int WCH = PF_BN / 32;            // 16-byte chunks of the bf16 weight tile per thread
    pf_f32x16 acc[2][NT];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.0f;
    // 4-bit weights enter the matrix cores as the exact integers -8..7; the products of one scale
    // group (128 reduction elements = two steps) are summed separately and scaled once, in fp32,
    // like the per-piece scale of the decode GEMV
    pf_f32x16 accg[WT == WT_INT4 ? 2 : 1][WT == WT_INT4 ? NT : 1];
    if (WT == WT_INT4) {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < NT; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) accg[a % (WT == WT_INT4 ? 2 : 1)][b % (WT == WT_INT4 ? NT : 1)][i] = 0.0f;
    }

    // global -> register staging ahead of the multiply.  Activation tiles: 128 rows x 8 chunks of
    // 8 elements, four chunks per thread for hi and for lo.  Weight tile of PF_BN rows: bf16 8 chunks
    // per row, e4m3 4 chunks of 16 elements, 4-bit 2 chunks of 32.  Rows past the end re-read the
    // last valid row (their results are not stored); chunks past K are zero.
    struct Stage { uint4 ah[4], al[4], w[WCH]; };
    const uint4 zero4 = make_uint4(0, 0, 0, 0);
    auto gload = [&](Stage &s, int step) {
        const int k0 = step * PF_BKL;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = tid + 256 * j, row = c >> 3, k = k0 + (c & 7) * 8;
            const size_t ta = (size_t)min(t0 + row, g.T - 1);
            s.ah[j] = zero4; s.al[j] = zero4;
            if (k < g.K) {
                s.ah[j] = *(const uint4 *)(g.Ahi + ta * g.K + k);
                if (LO) s.al[j] = *(const uint4 *)(g.Alo + ta * g.K + k);
            }
        }
#pragma unroll
        for (int j = 0; j < WCH; ++j) s.w[j] = zero4;
        if (WT == WT_BF16) {
#pragma unroll
            for (int j = 0; j < WCH; ++j) {
                const int c = tid + 256 * j, row = c >> 3, k = k0 + (c & 7) * 8;
                const size_t na = (size_t)min(n0 + row, g.N - 1);
                if (k < g.K) s.w[j] = *(const uint4 *)((const uint16_t *)g.W + na * g.K + k);
            }
        }
        if (WT == WT_FP8) {
#pragma unroll
            for (int j = 0; j < WCH / 2; ++j) {
                const int c = tid + 256 * j, row = c >> 2, k = k0 + (c & 3) * 16;
                const size_t na = (size_t)min(n0 + row, g.N - 1);
                if (k < g.K) s.w[j] = *(const uint4 *)((const uint8_t *)g.W + na * g.K + k);
            }
        }
        if (WT == WT_INT4) {       // PF_BN rows x 2 halves of 32 elements (16 bytes)
#pragma unroll
            for (int j = 0; j < WCH / 4; ++j) {
                const int c = tid + 256 * j, row = c >> 1, k = k0 + (c & 1) * 32;
                const size_t na = (size_t)min(n0 + row, g.N - 1);
                if (k < g.K) s.w[j] = *(const uint4 *)((const uint8_t *)g.W + na * (size_t)(g.K / 2) + k / 2);
            }
        }
    };
    auto lstore = [&](const Stage &s) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = tid + 256 * j, row = c >> 3, kc = c & 7;
            *(uint4 *)(sAh + row * PF_LDS_STRIDE + kc * 8) = s.ah[j];
            if (LO) *(uint4 *)(sAl + row * PF_LDS_STRIDE + kc * 8) = s.al[j];
        }
        if (WT == WT_BF16) {
#pragma unroll
            for (int j = 0; j < WCH; ++j) {
                const int c = tid + 256 * j, row = c >> 3, kc = c & 7;
                uint4 v = s.w[j];
                if (F16) v = make_uint4(pf_bf16x2_to_f16x2(v.x), pf_bf16x2_to_f16x2(v.y), pf_bf16x2_to_f16x2(v.z), pf_bf16x2_to_f16x2(v.w));
                *(uint4 *)(sW + row * PF_LDS_STRIDE + kc * 8) = v;
            }
        }
        if (WT == WT_FP8) {
#pragma unroll
            for (int j = 0; j < WCH / 2; ++j) {
                const int c = tid + 256 * j, row = c >> 2, q = c & 3;
                const uint32_t u[4] = {s.w[j].x, s.w[j].y, s.w[j].z, s.w[j].w};
                uint32_t o[8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    auto lo2 = __builtin_amdgcn_cvt_pk_f32_fp8(u[i], false);
                    auto hi2 = __builtin_amdgcn_cvt_pk_f32_fp8(u[i], true);
                    // e4m3 values are exact in bf16 (keep the upper halves of the fp32 patterns) and in fp16
                    if (F16) {
                        o[2 * i] = pf_pack_f16(lo2[0], lo2[1]);
                        o[2 * i + 1] = pf_pack_f16(hi2[0], hi2[1]);
                    } else {
                        o[2 * i] = (__float_as_uint(lo2[0]) >> 16) | (__float_as_uint(lo2[1]) & 0xffff0000u);
                        o[2 * i + 1] = (__float_as_uint(hi2[0]) >> 16) | (__float_as_uint(hi2[1]) & 0xffff0000u);
                    }
                }
                uint16_t *dst = sW + row * PF_LDS_STRIDE + q * 16;
                *(uint4 *)dst = make_uint4(o[0], o[1], o[2], o[3]);
                *(uint4 *)(dst + 8) = make_uint4(o[4], o[5], o[6], o[7]);
            }
        }
        if (WT == WT_INT4) {
            // nibble n (offset-binary, element 2j = low nibble of byte j) -> bf16 bits of the integer n - 8:
            // 2^23 + n is exact in fp32, subtracting 2^23 + 8 leaves n - 8, whose upper 16 bits are its bf16 form
#pragma unroll
            for (int j = 0; j < WCH / 4; ++j) {
                const int c = tid + 256 * j, row = c >> 1, half = c & 1;
                const uint32_t u[4] = {s.w[j].x, s.w[j].y, s.w[j].z, s.w[j].w};
                uint16_t *dst = sW + row * PF_LDS_STRIDE + half * 32;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    uint32_t o[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float f0 = __uint_as_float(0x4B000000u | ((u[i] >> (8 * e)) & 0xfu)) - 8388616.0f;
                        const float f1 = __uint_as_float(0x4B000000u | ((u[i] >> (8 * e + 4)) & 0xfu)) - 8388616.0f;
                        o[e] = F16 ? pf_pack_f16(f0, f1) : (__float_as_uint(f0) >> 16) | (__float_as_uint(f1) & 0xffff0000u);
                    }
                    *(uint4 *)(dst + 8 * i) = make_uint4(o[0], o[1], o[2], o[3]);
                }
            }
        }
    };
    auto multiply = [&]() {
        const int r = lane & 31, kq = 8 * (lane >> 5);
#pragma unroll
        for (int j = 0; j < PF_BKL / 16; ++j) {
            uint4 ah[2], al[2];
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                ah[mt] = *(const uint4 *)(sAh + (64 * wm + 32 * mt + r) * PF_LDS_STRIDE + 16 * j + kq);
                if (LO) al[mt] = *(const uint4 *)(sAl + (64 * wm + 32 * mt + r) * PF_LDS_STRIDE + 16 * j + kq);
            }
            // two workgroups per CU: one weight fragment at a time keeps the kernel within 128 registers
            // (the other workgroup covers the LDS latency); alone on the CU, all fragments are requested first
            constexpr bool PRELOAD = (WT == WT_INT4);
            uint4 bpre[PRELOAD ? NT : 1];
            if (PRELOAD) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    bpre[PRELOAD ? nt : 0] = *(const uint4 *)(sW + (32 * NT * wn + 32 * nt + r) * PF_LDS_STRIDE + 16 * j + kq);
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint4 bf = PRELOAD ? bpre[PRELOAD ? nt : 0]
                                         : *(const uint4 *)(sW + (32 * NT * wn + 32 * nt + r) * PF_LDS_STRIDE + 16 * j + kq);
#pragma unroll
                for (int mt = 0; mt < 2; ++mt) {
                    if (WT == WT_INT4) {
                        pf_f32x16 &t = accg[mt % (WT == WT_INT4 ? 2 : 1)][nt % (WT == WT_INT4 ? NT : 1)];
                        t = pf_mma(ah[mt], bf, t, F16);
                        if (LO) t = pf_mma(al[mt], bf, t, F16);
                    } else {
                        acc[mt][nt] = pf_mma(ah[mt], bf, acc[mt][nt], F16);
                        if (LO) acc[mt][nt] = pf_mma(al[mt], bf, acc[mt][nt], F16);
                    }
                }
            }
        }
    };
    // 4-bit weights: the group that steps (i, i + 1) of this split make up, scaled into the result.
    // Result register columns are weight rows (lane % 32), so the scale is one value per lane and tile.
    auto scale_group = [&](int step) {
        if (WT != WT_INT4) return;
        const int grp = step / (128 / PF_BKL), kg = g.K / 128;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const size_t na = (size_t)min(n0 + 32 * NT * wn + 32 * nt + (lane & 31), g.N - 1);
            const float sc = __uint_as_float((uint32_t)g.S[na * kg + grp] << 16);
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                pf_f32x16 &t = accg[mt % (WT == WT_INT4 ? 2 : 1)][nt % (WT == WT_INT4 ? NT : 1)];
#pragma unroll
                for (int i = 0; i < 16; ++i) { acc[mt][nt][i] = fmaf(t[i], sc, acc[mt][nt][i]); t[i] = 0.0f; }
            }
        }
    };

    const int n = s_end - s_begin;
    if constexpr (WT != WT_INT4) {
    // one step of operand loads in flight in registers: 48 registers fewer than two, which lets two
    // workgroups share a CU (one multiplies while the other stages)
    Stage S0;
    if (n > 0) gload(S0, s_begin);
    for (int i = 0; i < n; ++i) {
        __syncthreads();                       // the previous step's operand reads are done
        lstore(S0);
        __syncthreads();
        if (i + 1 < n) gload(S0, s_begin + i + 1);
        multiply();
    }
    } else {
    // alone on the CU (the second accumulator set of the 4-bit path): two steps in flight
    Stage S0, S1;
    if (n > 0) gload(S0, s_begin);
    if (n > 1) gload(S1, s_begin + 1);
    for (int i = 0; i < n; i += 2) {
        __syncthreads();                       // the previous step's operand reads are done
        lstore(S0);
        __syncthreads();
        if (i + 2 < n) gload(S0, s_begin + i + 2);   // two steps in flight while this one multiplies
        multiply();
        if (i + 1 < n) {
            __syncthreads();
            lstore(S1);
            __syncthreads();
            if (i + 3 < n) gload(S1, s_begin + i + 3);
            multiply();
        }
        scale_group(s_begin + i);              // (splits of 4-bit weights start on a group boundary)
    }
    }

    float *Pz = g.P + (size_t)z * g.T * g.N;
    const int r = lane & 31, gq = lane >> 5;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int n = n0 + 32 * NT * wn + 32 * nt + r;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int t = t0 + 64 * wm + 32 * mt + 8 * (i >> 2) + 4 * gq + (i & 3);
                if (t < g.T && n < g.N) Pz[(size_t)t * g.N + n] = acc[mt][nt][i];
            }
        }
}

// ---------------------------------------------------------------- tiled GEMM, operands loaded straight into LDS
// The kernel above moves every operand global -> registers -> LDS, which costs it 48 staging registers
// (so its tile cannot grow), a round of LDS store instructions per step, and leaves one step of loads
// in flight.  For bf16 weights no conversion is needed on the way, so this variant lets the memory
// system write the tiles into LDS itself (`global_load_lds_dwordx4`: every lane names a 16-byte chunk in
// global memory, the wave's 64 chunks land side by side at an LDS address the wave gives).  No staging
// registers: the workgroup tile is 128 rows x 256 channels, eight waves of 64 x 64 each (two per SIMD: one
// multiplies while the other reads operands and computes addresses; four waves of 64 x 128 with one
// wave per SIMD ran 10 % slower), two (pair) or three (single) LDS stages of 64 / 48 KB, a step's loads
// issued one or two steps before its multiply and waited for with `s_waitcnt vmcnt(n)`, one workgroup
// per CU.  Stand-alone, 1024 x 22016 x 4096 / 1024 x 4096 x 11008 / 1024 x 6144 x 4096, pair: 351 / 172 /
// 119 us against 429 / 219 / 152 us for the kernel above; single bf16: 234 / 113 / 80 us against 278 / 144 / 81.
// LDS layout: tile rows without padding -- the hardware writes a wave's chunks contiguously -- with the
// chunks of a row permuted by an XOR of the row index, so that the rows of an operand read spread over
// all banks; the lane that loads slot s of row R fetches the chunk that belongs there from global.
#define PF_DL_BM 128
#define PF_DL_BN 256
#define PF_DL_WAVES 8      // waves per workgroup the host launches (64 x 64 of the tile each)
// One load-to-LDS instruction of a wave: lane l's 16 bytes at gptr land at LDS byte address lds_base + 16 l
// (lds_base wave-uniform, in M0).  Written as assembly on purpose: through the builtin the compiler knows
// the instruction writes LDS, and across the loop's back edge it can no longer tell the stage being read
// from the stage being filled, so it waits for ALL of these loads (vmcnt(0)) before the first operand read
// of every other step -- which serialises the pipeline.  Here every wait for them is stated by hand
// (pf_vmcnt); the counter is shared with the compiler's own loads, whose waits can only get stricter
// by loads it does not know of (they complete in order).
__device__ __forceinline__ void pf_dl_load16(const uint16_t *gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :: "v"(gptr), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ uint32_t pf_lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}
// s_waitcnt vmcnt(n) alone (n < 64): bits 3:0 and 15:14 hold the count, the other counters stay at their maximum
__device__ __forceinline__ constexpr int pf_vmcnt(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }
// Workgroup barrier for the LDS stages.  A release fence on local memory would also wait for every
// outstanding load-to-LDS (they are LDS writes), the next stage's included, which is exactly the
// overlap this kernel is built for; the waits are stated by hand instead (vmcnt(n) by the caller for
// the stage it is about to read, lgkmcnt(0) here for its own LDS reads), and the "memory" clobber keeps
// the compiler from moving LDS accesses across the barrier.
__device__ __forceinline__ void pf_lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// BK: reduction elements per stage (32 or 64); STAGES: stages in LDS.  Step i's loads are issued
// STAGES - 1 steps before they are read: after the barrier of step i - (STAGES - 1), i.e. once every wave
// is done with the stage they overwrite, so a step needs ONE barrier.
// WAVES: 4 (each wave 64 x 128 of the tile) or 8 (64 x 64: two waves per SIMD cover each other's operand
// reads and address arithmetic); WGS: workgroups per CU the registers and LDS are budgeted for.
template <bool LO, int BK, int STAGES, int WAVES, int WGS>
__global__ __launch_bounds__(64 * WAVES, WGS) void k_pf_gemm_dl(PfGemm g) {
    constexpr int NTW = 8 / (WAVES / 2);                      // 32-channel tiles per wave
    constexpr int CPR = BK / 8;                               // 16-byte chunks per tile row
    constexpr int RPB = 256 / (BK * 2);                       // tile rows per 256 bytes of LDS (64 banks of 4 bytes)
    constexpr int A_EL = PF_DL_BM * BK, W_EL = PF_DL_BN * BK;
    constexpr int W_AT = A_EL * (LO ? 2 : 1);                 // element offset of the weight tile inside a stage
    constexpr int ST_EL = W_AT + W_EL;
    constexpr int NA = PF_DL_BM * CPR / (64 * WAVES), NW = PF_DL_BN * CPR / (64 * WAVES);   // load instructions per wave: activation tile, weight tile
    constexpr int LOADS = NA * (LO ? 2 : 1) + NW;             // per wave and stage
    static_assert(STAGES >= 2 && STAGES <= 6 && LOADS * (STAGES - 1) < 64, "vmcnt holds 6 bits");
    __shared__ __align__(16) uint16_t sbuf[STAGES * ST_EL];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / (WAVES / 2), wn = wave % (WAVES / 2);
    const int n0 = blockIdx.x * PF_DL_BN, t0 = blockIdx.y * PF_DL_BM, z = blockIdx.z;
    const int nsteps = g.K / BK;
    const int s_begin = z * g.steps_per_split, s_end = min(nsteps, s_begin + g.steps_per_split);

    pf_f32x16 acc[2][NTW];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < NTW; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.0f;

    // Load instruction q of a tile covers the LDS chunk positions 64 q .. 64 q + 63; wave w issues
    // q = w, w + WAVES, ...  The global element offset of this lane's chunk is fixed over the K loop (rows past
    // the end re-read the last valid row; their results are not stored).  Chunk c of row R sits at slot
    // c ^ ((R / RPB) % CPR): a 128-bit operand read is served 16 lanes (16 consecutive tile rows) at a time
    // out of 64 banks, and with this the 16 chunks fall into 16 different 16-byte bank groups (measured:
    // swizzled by R % CPR, as 32 banks would want, half of the LDS cycles were bank conflicts).
    size_t a_off[NA], w_off[NW];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const int P = 64 * (wave + WAVES * i) + lane, row = P / CPR, c = (P % CPR) ^ ((row / RPB) % CPR);
        a_off[i] = (size_t)min(t0 + row, g.T - 1) * g.K + c * 8;
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        const int P = 64 * (wave + WAVES * i) + lane, row = P / CPR, c = (P % CPR) ^ ((row / RPB) % CPR);
        w_off[i] = (size_t)min(n0 + row, g.N - 1) * g.K + c * 8;
    }
    const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)pf_lds_addr(sbuf)) + (uint32_t)wave * 1024u;   // bytes
    auto issue = [&](int slot, int step) {
        const size_t k0 = (size_t)step * BK;
        const uint32_t base = lds0 + (uint32_t)slot * (2u * ST_EL);
#pragma unroll
        for (int i = 0; i < NA; ++i) pf_dl_load16(g.Ahi + a_off[i] + k0, base + 1024u * WAVES * i);
        if (LO) {
#pragma unroll
            for (int i = 0; i < NA; ++i) pf_dl_load16(g.Alo + a_off[i] + k0, base + 2u * A_EL + 1024u * WAVES * i);
        }
#pragma unroll
        for (int i = 0; i < NW; ++i) pf_dl_load16((const uint16_t *)g.W + w_off[i] + k0, base + 2u * W_AT + 1024u * WAVES * i);
    };
    const int r = lane & 31, gq = lane >> 5, sw = (r / RPB) % CPR;
    auto multiply = [&](const uint16_t *sb) {
#pragma unroll
        for (int j = 0; j < BK / 16; ++j) {
            const int slot = ((2 * j + gq) ^ sw) * 8;          // this lane's chunk of the sub-step, swizzled (the tile bases are multiples of 32 rows)
            uint4 ah[2], al[2];
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                const int R = 64 * wm + 32 * mt + r;
                ah[mt] = *(const uint4 *)(sb + R * BK + slot);
                if (LO) al[mt] = *(const uint4 *)(sb + A_EL + R * BK + slot);
            }
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
                const int R = 32 * NTW * wn + 32 * nt + r;
                const uint4 bf = *(const uint4 *)(sb + W_AT + R * BK + slot);
#pragma unroll
                for (int mt = 0; mt < 2; ++mt) {
                    acc[mt][nt] = pf_mma(ah[mt], bf, acc[mt][nt], false);
                    if (LO) acc[mt][nt] = pf_mma(al[mt], bf, acc[mt][nt], false);
                }
            }
        }
    };
    // wait until at most `stages` later stages of this wave's loads are outstanding
    auto wait_stages = [&](int stages) {
        switch (stages) {
            case 0: __builtin_amdgcn_s_waitcnt(pf_vmcnt(0)); break;
            case 1: __builtin_amdgcn_s_waitcnt(pf_vmcnt(LOADS)); break;
            case 2: __builtin_amdgcn_s_waitcnt(pf_vmcnt(STAGES > 2 ? 2 * LOADS : 0)); break;
            case 3: __builtin_amdgcn_s_waitcnt(pf_vmcnt(STAGES > 3 ? 3 * LOADS : 0)); break;
            default: __builtin_amdgcn_s_waitcnt(pf_vmcnt(STAGES > 4 ? 4 * LOADS : 0)); break;
        }
    };

    const int n = s_end - s_begin;
#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if (p < n) issue(p, s_begin + p);
    int slot = 0;
    for (int i = 0; i < n; ++i) {
        wait_stages(min(STAGES - 2, n - 1 - i));   // this wave's part of step i has landed
        pf_lds_barrier();                          // everyone's has, and everyone is done with step i - 1
        if (i + STAGES - 1 < n) issue(slot == 0 ? STAGES - 1 : slot - 1, s_begin + i + STAGES - 1);
        multiply(sbuf + slot * ST_EL);
        slot = slot + 1 == STAGES ? 0 : slot + 1;
    }

    float *Pz = g.P + (size_t)z * g.T * g.N;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            const int col = n0 + 32 * NTW * wn + 32 * nt + r;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int t = t0 + 64 * wm + 32 * mt + 8 * (i >> 2) + 4 * gq + (i & 3);
                if (t < g.T && col < g.N) Pz[(size_t)t * g.N + col] = acc[mt][nt][i];
            }
        }
}

// GEMM for at most 32 activation rows (multi-sample decode, short prompts): weight streaming, not
// matrix throughput, bounds it, so there is no LDS tile and no barrier in the loop.  A workgroup
// owns 32 weight rows; its four waves split the workgroup's K range and each lane streams its own
// weight row straight into MFMA operand registers, several steps of loads in flight.  The
// workgroup's slice of the few activation rows (hi and lo parts) is staged once in LDS while the
// first weight loads are in flight; rows past T read row T-1 and are not stored.  The four partial
// tiles are summed through LDS in wave order.
// 4-bit weights: a lane's 16 elements of a step are 8 bytes; the PF_SK_UNROLL = 4 steps issued together are
// exactly one scale group of 128 elements (the host makes every K split, and the kernel every wave's part,
// a whole number of groups), whose products are summed unscaled and enter the result times the row's scale.
// fp32 weights: a lane's 16 elements of a step are 64 bytes; each is split in registers into a (hi, lo) pair
// of bf16 numbers like the activations, and x w = xh wh + xl wh + xh wl on the matrix cores (the dropped
// xl wl and the weight's third part are 2^-16 of a product and less): fp32-grade, three instructions.
#define PF_SK_UNROLL 4     // 32-element steps whose loads are issued together
#define PF_SK_PAD 8        // bf16 elements of padding per staged activation row
template <int WT>
__global__ __launch_bounds__(256) void k_pf_gemm_skinny(PfGemm g) {
    __shared__ float red[4][16][64];
    extern __shared__ __align__(16) uint16_t s_act[];      // [2][T][krange + PF_SK_PAD]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, gq = lane >> 5;
    const int n0 = blockIdx.x * 32, z = blockIdx.y;
    const int nsteps = g.K / PF_BK;
    const int zb = z * g.steps_per_split, ze = min(nsteps, zb + g.steps_per_split);
    const int per_wave = WT == WT_INT4 ? (((ze - zb + 3) / 4 + PF_SK_UNROLL - 1) / PF_SK_UNROLL) * PF_SK_UNROLL : (ze - zb + 3) / 4;
    const int s_begin = min(ze, zb + wave * per_wave), s_end = min(ze, s_begin + per_wave);
    const size_t na = (size_t)min(n0 + r, g.N - 1);
    const int krange = (ze - zb) * PF_BK, astride = g.steps_per_split * PF_BK + PF_SK_PAD;
    const uint16_t *ah = s_act + min(r, g.T - 1) * astride + 16 * gq;
    const uint16_t *al = ah + g.T * astride;
    // bytes of a weight row, and of this lane's 16 elements of a step
    const char *wp = (const char *)g.W +
                     na * (WT == WT_F32 ? (size_t)g.K * 4 : WT == WT_BF16 ? (size_t)g.K * 2 : WT == WT_INT4 ? (size_t)g.K / 2 : (size_t)g.K) +
                     (WT == WT_F32 ? 64 : WT == WT_BF16 ? 32 : WT == WT_INT4 ? 8 : 16) * gq;
    constexpr int WREG = WT == WT_F32 ? 4 : 2;             // 16-byte registers per step and lane

    uint4 w[PF_SK_UNROLL][WREG];
    auto wload = [&](int s0) {
#pragma unroll
        for (int u = 0; u < PF_SK_UNROLL; ++u) {
            const int s = min(s0 + u, s_end - 1);             // a padded step re-reads the last one (and is skipped below)
            const size_t k0 = (size_t)s * PF_BK;
            if (WT == WT_F32) {
#pragma unroll
                for (int c = 0; c < WREG; ++c) w[u][c] = *(const uint4 *)(wp + k0 * 4 + 16 * c);
            } else if (WT == WT_BF16) {
                w[u][0] = *(const uint4 *)(wp + k0 * 2);
                w[u][1] = *(const uint4 *)(wp + k0 * 2 + 16);
            } else if (WT == WT_INT4) {
                const uint2 v = *(const uint2 *)(wp + k0 / 2);
                w[u][0] = make_uint4(v.x, v.y, 0u, 0u);
            } else {
                w[u][0] = *(const uint4 *)(wp + k0);
            }
        }
    };
    if (s_begin < s_end) wload(s_begin);
    // stage activation rows [0, T) x this workgroup's K range
    {
        const int cpr = krange / 8;                           // 16-byte chunks per row
        for (int c = tid; c < g.T * cpr; c += 256) {
            const int t = c / cpr, kc = c - t * cpr;
            const size_t src = (size_t)t * g.K + (size_t)zb * PF_BK + kc * 8;
            *(uint4 *)(s_act + t * astride + kc * 8) = *(const uint4 *)(g.Ahi + src);
            *(uint4 *)(s_act + (g.T + t) * astride + kc * 8) = *(const uint4 *)(g.Alo + src);
        }
    }
    __syncthreads();

    pf_f32x16 acc, accg;
#pragma unroll
    for (int i = 0; i < 16; ++i) { acc[i] = 0.0f; accg[i] = 0.0f; }
    for (int s0 = s_begin; s0 < s_end; s0 += PF_SK_UNROLL) {
        uint4 wc[PF_SK_UNROLL][WREG], xh[PF_SK_UNROLL][2], xl[PF_SK_UNROLL][2];
        float gscale = 0.0f;
        if (WT == WT_INT4) gscale = __uint_as_float((uint32_t)g.S[na * (size_t)(g.K / 128) + s0 / PF_SK_UNROLL] << 16);
#pragma unroll
        for (int u = 0; u < PF_SK_UNROLL; ++u)
#pragma unroll
            for (int c = 0; c < WREG; ++c) wc[u][c] = w[u][c];
        if (s0 + PF_SK_UNROLL < s_end) wload(s0 + PF_SK_UNROLL);   // next group in flight while this one multiplies
#pragma unroll
        for (int u = 0; u < PF_SK_UNROLL; ++u) {
            const int k0 = (min(s0 + u, s_end - 1) - zb) * PF_BK;
            xh[u][0] = *(const uint4 *)(ah + k0); xh[u][1] = *(const uint4 *)(ah + k0 + 8);
            xl[u][0] = *(const uint4 *)(al + k0); xl[u][1] = *(const uint4 *)(al + k0 + 8);
        }
#pragma unroll
        for (int u = 0; u < PF_SK_UNROLL; ++u) {
            if (s0 + u < s_end) {
                uint4 b0, b1, c0 = make_uint4(0u, 0u, 0u, 0u), c1 = c0;      // (c0, c1: the lo parts of fp32 weights)
                if (WT == WT_F32) {
                    uint32_t oh[8], ol[8];
#pragma unroll
                    for (int c = 0; c < WREG; ++c) {
                        const uint4 v = wc[u][WT == WT_F32 ? c : 0];
                        pf_split2(__uint_as_float(v.x), __uint_as_float(v.y), oh[2 * c], ol[2 * c]);
                        pf_split2(__uint_as_float(v.z), __uint_as_float(v.w), oh[2 * c + 1], ol[2 * c + 1]);
                    }
                    b0 = make_uint4(oh[0], oh[1], oh[2], oh[3]); b1 = make_uint4(oh[4], oh[5], oh[6], oh[7]);
                    c0 = make_uint4(ol[0], ol[1], ol[2], ol[3]); c1 = make_uint4(ol[4], ol[5], ol[6], ol[7]);
                } else if (WT == WT_BF16) { b0 = wc[u][0]; b1 = wc[u][1]; }
                else if (WT == WT_INT4) {
                    // nibble n (offset-binary, element 2j = low nibble of byte j) -> bf16 bits of the integer n - 8
                    const uint32_t q[2] = {wc[u][0].x, wc[u][0].y};
                    uint32_t o[8];
#pragma unroll
                    for (int i = 0; i < 2; ++i)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float f0 = __uint_as_float(0x4B000000u | ((q[i] >> (8 * e)) & 0xfu)) - 8388616.0f;
                            const float f1 = __uint_as_float(0x4B000000u | ((q[i] >> (8 * e + 4)) & 0xfu)) - 8388616.0f;
                            o[4 * i + e] = (__float_as_uint(f0) >> 16) | (__float_as_uint(f1) & 0xffff0000u);
                        }
                    b0 = make_uint4(o[0], o[1], o[2], o[3]); b1 = make_uint4(o[4], o[5], o[6], o[7]);
                } else {
                    const uint32_t q[4] = {wc[u][0].x, wc[u][0].y, wc[u][0].z, wc[u][0].w};
                    uint32_t o[8];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        auto lo2 = __builtin_amdgcn_cvt_pk_f32_fp8(q[i], false);
                        auto hi2 = __builtin_amdgcn_cvt_pk_f32_fp8(q[i], true);
                        o[2 * i] = (__float_as_uint(lo2[0]) >> 16) | (__float_as_uint(lo2[1]) & 0xffff0000u);
                        o[2 * i + 1] = (__float_as_uint(hi2[0]) >> 16) | (__float_as_uint(hi2[1]) & 0xffff0000u);
                    }
                    b0 = make_uint4(o[0], o[1], o[2], o[3]); b1 = make_uint4(o[4], o[5], o[6], o[7]);
                }
                const pf_bf16x8 B0 = __builtin_bit_cast(pf_bf16x8, b0), B1 = __builtin_bit_cast(pf_bf16x8, b1);
                pf_f32x16 &t = WT == WT_INT4 ? accg : acc;
                t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, xh[u][0]), B0, t, 0, 0, 0);
                t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, xl[u][0]), B0, t, 0, 0, 0);
                t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, xh[u][1]), B1, t, 0, 0, 0);
                t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, xl[u][1]), B1, t, 0, 0, 0);
                if (WT == WT_F32) {
                    t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, xh[u][0]), __builtin_bit_cast(pf_bf16x8, c0), t, 0, 0, 0);
                    t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, xh[u][1]), __builtin_bit_cast(pf_bf16x8, c1), t, 0, 0, 0);
                }
            }
        }
        if (WT == WT_INT4) {       // result columns are weight rows (lane % 32): one scale per lane and group
#pragma unroll
            for (int i = 0; i < 16; ++i) { acc[i] = fmaf(accg[i], gscale, acc[i]); accg[i] = 0.0f; }
        }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) red[wave][i][lane] = acc[i];
    __syncthreads();
    // wave w finishes result registers 4w .. 4w+3 (rows 8w + 4*gq + 0..3)
    float *Pz = g.P + (size_t)z * g.T * g.N;
    const int n = n0 + r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = 4 * wave + j;
        const float v = ((red[0][i][lane] + red[1][i][lane]) + red[2][i][lane]) + red[3][i][lane];
        const int t = 8 * wave + 4 * gq + j;
        if (t < g.T && n < g.N) Pz[(size_t)t * g.N + n] = v;
    }
}

// The few-row GEMM for 4-bit weights.  In k_pf_gemm_skinny a lane's share of a step is 8 bytes of its own weight
// row, so one load instruction touches 32 rows for 16 bytes each, a workgroup streams 16 KB of weights against
// 32 KB of staged activations, and every nibble costs five to six vector instructions on its way to bf16: the
// 5B model's products of 8 rows ran at 0.7 - 1.6 TB/s (28 / 17 / 17 / 8 us for the gate-up, down, q/k/v and output
// projections).  Here
//  * the products are v_mfma_f32_16x16x32_bf16: lane (n = l % 16, kg = l / 16) holds weight row n and the 32
//    elements kg of a 128-element scale group -- ONE 16-byte load, and the four lanes of a row read 64
//    contiguous bytes; dword j of the load is the lane's 8 elements of matrix instruction j of the group;
//  * a wave owns NT tiles of 16 weight rows and walks the workgroup's whole K range, the WAVES waves share the
//    staged activations and nothing is reduced across waves;
//  * a nibble n' (offset binary) becomes the bf16 number 16 + n' with two instructions per PAIR: the nibbles
//    j and j + 4 of a dword are shifted into mantissa bits 3..6 of the two halves of 0x41804180 (one shift, one
//    and-or).  The activations are staged in the matching order (elements 0 4 1 5 2 6 3 7 of every eight), and
//    since 16 + n' = 24 + (n' - 8) every group's activations are also multiplied by a tile of -24s on the
//    matrix cores, which are idle otherwise: the two result tiles add up to the product with n' - 8 before the
//    group's scale is applied (all in fp32);
//  * PACK (at most 8 activation rows): the hi parts are rows 0..7 and the lo parts rows 8..15 of ONE operand
//    tile, so a weight fragment is multiplied once, not twice; the two halves of the result tile (lanes 32
//    apart) are added at the end, which is exact in the same sense as summing the two products' tiles;
//  * a workgroup lives for a few microseconds, all of them at the same time, so what it does before its first
//    matrix instruction is on the critical path of the launch: the staging loop has no integer division, no
//    sums and no cross-lane traffic, and the weights of the split's whole K range are requested before it (the
//    host keeps a split within PF_SQ_GU groups).
#define PF_SQ_GU 8                       // scale groups of a split: what a wave requests per tile, all at once
// a constant the compiler has to treat as a register's value (S: scalar register, V: vector register)
#ifndef PF_REG_CONST_S
#define PF_REG_CONST_S(var, lit) asm volatile("s_mov_b32 %0, " #lit : "=s"(var))
#define PF_REG_CONST_V(var, lit) asm volatile("v_mov_b32 %0, " #lit : "=v"(var))
#endif
typedef float pf_f32x4 __attribute__((ext_vector_type(4)));
template <int RT, bool PACK, int NT, int WAVES>   // RT tiles of 16 activation rows (T <= 16 RT; PACK: T <= 8, RT = 1); NT weight tiles per wave
__global__ __launch_bounds__(64 * WAVES) void k_pf_gemm_skinny_i4(PfGemm g) {
    static_assert(!PACK || RT == 1, "packed planes are one row tile");
    constexpr int NTHR = 64 * WAVES;
    extern __shared__ __align__(16) uint16_t s_act[];      // [2][T][astride] bf16
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kg = lane >> 4;
    const int n0 = blockIdx.x * (16 * NT * WAVES) + wave * (16 * NT), z = blockIdx.y;
    const int nsteps = g.K / PF_BK;
    const int zb = z * g.steps_per_split, ze = min(nsteps, zb + g.steps_per_split);
    const int g_begin = zb / 4, g_end = ze / 4;            // (the host makes every split a whole number of groups)
    const int krange = (ze - zb) * PF_BK, astride = g.steps_per_split * PF_BK + PF_SK_PAD;
    const int kgrp = g.K / 128;

    const char *wrow[NT];
    const uint16_t *srow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const size_t row = (size_t)min(n0 + 16 * nt + n, g.N - 1);
        wrow[nt] = (const char *)g.W + row * (size_t)(g.K / 2) + 16 * kg;
        srow[nt] = g.S + row * (size_t)kgrp;
    }
    // slot u holds the split's group u; sc0[q]: the four scales of slots 4q .. 4q+3
    uint4 w0[PF_SQ_GU][NT];
    uint2 sc0[PF_SQ_GU / 4][NT];
    auto wload = [&](const int u, const int gg) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) w0[u][nt] = *(const uint4 *)(wrow[nt] + (size_t)gg * 64);
    };
    // scales: a row's four from group gi on as one load (gi is a multiple of four groups from the split's first,
    // which is one from the row's first); where fewer than four are left in the row the load starts earlier and
    // is shifted
    auto sload = [&](const int q, const int gi) {
        if (kgrp >= 4) {
            const int gs = min(gi, kgrp - 4), sh = 16 * (gi - gs);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint2 v = *(const uint2 *)(srow[nt] + gs);
                const unsigned long long x = (((unsigned long long)v.y << 32) | v.x) >> sh;
                sc0[q][nt] = make_uint2((uint32_t)x, (uint32_t)(x >> 32));
            }
        } else {                                              // a reduction of fewer than four groups
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint32_t s0 = srow[nt][min(gi, kgrp - 1)], s1 = srow[nt][min(gi + 1, kgrp - 1)], s2 = srow[nt][min(gi + 2, kgrp - 1)];
                sc0[q][nt] = make_uint2(s0 | (s1 << 16), s2);
            }
        }
    };
    // The activation rows [0, T) x this workgroup's K range are requested first and the weights behind them, so
    // that staging waits for its own loads only.  Staged: every eight elements as 0 4 1 5 2 6 3 7.
    {
        constexpr int MAXIT = (1280 + NTHR - 1) / NTHR;        // 40 KB of staged rows: at most 1280 chunks of hi and lo
        const int cpr = krange / 8, items = g.T * cpr;         // (cpr is a multiple of 16, items at most 1280)
        const float rcp = 1.0f / (float)cpr;
        uint4 hh[MAXIT], ll[MAXIT];
        int dst[MAXIT];
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            if (it * NTHR < items) {
                const int cc = min(it * NTHR + tid, items - 1);
                // cc / cpr without the division: the quotient's fraction is a multiple of 1 / cpr >= 1 / 1280, the
                // half chunk added keeps it that far from the next integer, the rounding errors are below 1e-5
                const int t = (int)(((float)cc + 0.5f) * rcp), kc = cc - t * cpr;
                const size_t src = (size_t)t * g.K + (size_t)zb * PF_BK + kc * 8;
                hh[it] = *(const uint4 *)(g.Ahi + src); ll[it] = *(const uint4 *)(g.Alo + src);
                dst[it] = t * astride + kc * 8;
            }
        }
#pragma unroll
        for (int u = 0; u < PF_SQ_GU; ++u)
            if (g_begin + u < g_end) wload(u, g_begin + u);
#pragma unroll
        for (int q = 0; q < PF_SQ_GU / 4; ++q)
            if (g_begin + 4 * q < g_end) sload(q, g_begin + 4 * q);
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            if (it * NTHR < items && it * NTHR + tid < items) {
                const uint4 h = hh[it], l = ll[it];
                *(uint4 *)(s_act + dst[it]) =
                    make_uint4(__builtin_amdgcn_perm(h.z, h.x, 0x05040100u), __builtin_amdgcn_perm(h.z, h.x, 0x07060302u),
                               __builtin_amdgcn_perm(h.w, h.y, 0x05040100u), __builtin_amdgcn_perm(h.w, h.y, 0x07060302u));
                *(uint4 *)(s_act + g.T * astride + dst[it]) =
                    make_uint4(__builtin_amdgcn_perm(l.z, l.x, 0x05040100u), __builtin_amdgcn_perm(l.z, l.x, 0x07060302u),
                               __builtin_amdgcn_perm(l.w, l.y, 0x05040100u), __builtin_amdgcn_perm(l.w, l.y, 0x07060302u));
            }
        }
    }
    __syncthreads();

    const uint16_t *ah[RT], *al[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (PACK) {
            ah[rt] = s_act + (n < 8 ? min(n, g.T - 1) : g.T + min(n - 8, g.T - 1)) * astride + 32 * kg;
            al[rt] = ah[rt];
        } else {
            ah[rt] = s_act + min(16 * rt + n, g.T - 1) * astride + 32 * kg;
            al[rt] = ah[rt] + g.T * astride;
        }
    }
    // the unpacking constants live in registers: as literals each pair would cost an "and" and an "or"
    uint32_t nib_mask, nib_bias, m24;
    PF_REG_CONST_S(nib_mask, 0x00780078);
    PF_REG_CONST_V(nib_bias, 0x41804180);
    PF_REG_CONST_V(m24, 0xc1c0c1c0);                                   // two bf16 numbers -24
    const pf_bf16x8 BC = __builtin_bit_cast(pf_bf16x8, make_uint4(m24, m24, m24, m24));
    pf_f32x4 acc[RT][NT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = pf_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // group gl (counted from the split's first) out of slot u
    auto group = [&](const int u, const int gl) {
        pf_f32x4 ag[RT][NT], cg[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            cg[rt] = pf_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) ag[rt][nt] = pf_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint4 xh[RT], xl[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                xh[rt] = *(const uint4 *)(ah[rt] + gl * 128 + 8 * j);
                if (!PACK) xl[rt] = *(const uint4 *)(al[rt] + gl * 128 + 8 * j);
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                cg[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, xh[rt]), BC, cg[rt], 0, 0, 0);
                if (!PACK) cg[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, xl[rt]), BC, cg[rt], 0, 0, 0);
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint32_t q = j == 0 ? w0[u][nt].x : j == 1 ? w0[u][nt].y : j == 2 ? w0[u][nt].z : w0[u][nt].w;
                const uint4 b = make_uint4(((q << 3) & nib_mask) | nib_bias, ((q >> 1) & nib_mask) | nib_bias,
                                           ((q >> 5) & nib_mask) | nib_bias, ((q >> 9) & nib_mask) | nib_bias);
                const pf_bf16x8 B = __builtin_bit_cast(pf_bf16x8, b);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    ag[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, xh[rt]), B, ag[rt][nt], 0, 0, 0);
                    if (!PACK) ag[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, xl[rt]), B, ag[rt][nt], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint32_t sw = (u & 2) ? sc0[u >> 2][nt].y : sc0[u >> 2][nt].x;
                const float scale = __uint_as_float((u & 1) ? (sw & 0xffff0000u) : (sw << 16));
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[rt][nt][i] = fmaf(ag[rt][nt][i] + cg[rt][i], scale, acc[rt][nt][i]);
            }
    };
#pragma unroll
    for (int u = 0; u < PF_SQ_GU; ++u)
        if (g_begin + u < g_end) group(u, u);
    // lane (n, kg) holds rows 16 rt + 4 kg + i of column n of each tile (PACK: kg 0, 1 the hi parts' products of
    // rows 4 kg + i, kg 2, 3 the lo parts' of rows 4 (kg - 2) + i)
    float *Pz = g.P + (size_t)z * g.T * g.N;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int col = n0 + 16 * nt + n;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = acc[rt][nt][i];
                if (PACK) v += __shfl_xor(v, 32, 64);
                const int t = 16 * rt + 4 * kg + i;
                if ((!PACK || kg < 2) && t < g.T && col < g.N) Pz[(size_t)t * g.N + col] = v;
            }
        }
}

// The same few-row GEMM for e4m3 weights.  A lane's 16-byte load is 16 elements: lane (n, kg) holds weight row n and
// elements 16 kg .. + 16 of a 64-element block, the four lanes of a row read 64 contiguous bytes, and dwords 2 j,
// 2 j + 1 are the lane's 8 elements of matrix instruction j (j = 0, 1) of the block, widened to bf16 two at a time
// by v_cvt_scalef32_pk_bf16_fp8 (exact).  The activations are staged as they are; the per-row scale is applied by
// the kernel that sums the planes, as for k_pf_gemm_skinny.  A K split is a whole number of blocks, at most
// PF_S8_GU of them, all requested before the rows are staged; the staging loop has no integer division.
#define PF_S8_GU 8                       // 64-element blocks of a split: what a wave requests, all at once
typedef __bf16 pf_bf16x2v __attribute__((ext_vector_type(2)));
template <int RT, bool PACK, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void k_pf_gemm_skinny_f8(PfGemm g) {
    constexpr int NTHR = 64 * WAVES;
    static_assert(!PACK || RT == 1, "packed planes are one row tile");
    extern __shared__ __align__(16) uint16_t s_act[];      // [2][T][astride] bf16
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kg = lane >> 4;
    const int n0 = blockIdx.x * (16 * WAVES) + wave * 16, z = blockIdx.y;
    const int nsteps = g.K / PF_BK;
    const int zb = z * g.steps_per_split, ze = min(nsteps, zb + g.steps_per_split);
    const int b_begin = zb / 2, b_end = ze / 2;            // 64-element blocks (the host makes every split a whole number of them)
    const int krange = (ze - zb) * PF_BK, astride = g.steps_per_split * PF_BK + PF_SK_PAD;
    const char *wrow = (const char *)g.W + (size_t)min(n0 + n, g.N - 1) * (size_t)g.K + 16 * kg;
    // slot u holds the split's block u (the host keeps a split within PF_S8_GU blocks)
    uint4 w0[PF_S8_GU];
    // the activation rows are requested first and the weights behind them (staging waits for its own loads only)
    {
        constexpr int MAXIT = (1280 + NTHR - 1) / NTHR;        // 40 KB of staged rows: at most 1280 chunks of hi and lo
        const int cpr = krange / 8, items = g.T * cpr;         // (cpr is a multiple of 8, items at most 1280)
        const float rcp = 1.0f / (float)cpr;
        uint4 hh[MAXIT], ll[MAXIT];
        int dst[MAXIT];
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            if (it * NTHR < items) {
                const int cc = min(it * NTHR + tid, items - 1);
                // cc / cpr without the division: the quotient's fraction is a multiple of 1 / cpr >= 1 / 1280, the
                // half chunk added keeps it that far from the next integer, the rounding errors are below 1e-5
                const int t = (int)(((float)cc + 0.5f) * rcp), kc = cc - t * cpr;
                const size_t src = (size_t)t * g.K + (size_t)zb * PF_BK + kc * 8;
                hh[it] = *(const uint4 *)(g.Ahi + src); ll[it] = *(const uint4 *)(g.Alo + src);
                dst[it] = t * astride + kc * 8;
            }
        }
#pragma unroll
        for (int u = 0; u < PF_S8_GU; ++u)
            if (b_begin + u < b_end) w0[u] = *(const uint4 *)(wrow + (size_t)(b_begin + u) * 64);
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            if (it * NTHR < items && it * NTHR + tid < items) {
                *(uint4 *)(s_act + dst[it]) = hh[it];
                *(uint4 *)(s_act + g.T * astride + dst[it]) = ll[it];
            }
        }
    }
    __syncthreads();

    const uint16_t *ah[RT], *al[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (PACK) {
            ah[rt] = s_act + (n < 8 ? min(n, g.T - 1) : g.T + min(n - 8, g.T - 1)) * astride + 16 * kg;
            al[rt] = ah[rt];
        } else {
            ah[rt] = s_act + min(16 * rt + n, g.T - 1) * astride + 16 * kg;
            al[rt] = ah[rt] + g.T * astride;
        }
    }
    pf_f32x4 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc[rt] = pf_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < PF_S8_GU; ++u) {
        if (b_begin + u < b_end) {
            const int kl = u * 64;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t q0 = j == 0 ? w0[u].x : w0[u].z, q1 = j == 0 ? w0[u].y : w0[u].w;
                const uint4 b = make_uint4(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(q0, 1.0f, false)),
                                           __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(q0, 1.0f, true)),
                                           __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(q1, 1.0f, false)),
                                           __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(q1, 1.0f, true)));
                const pf_bf16x8 B = __builtin_bit_cast(pf_bf16x8, b);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const uint4 xh = *(const uint4 *)(ah[rt] + kl + 8 * j);
                    acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, xh), B, acc[rt], 0, 0, 0);
                    if (!PACK) {
                        const uint4 xl = *(const uint4 *)(al[rt] + kl + 8 * j);
                        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, xl), B, acc[rt], 0, 0, 0);
                    }
                }
            }
        }
    }
    float *Pz = g.P + (size_t)z * g.T * g.N;
    const int col = n0 + n;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = acc[rt][i];
            if (PACK) v += __shfl_xor(v, 32, 64);
            const int t = 16 * rt + 4 * kg + i;
            if ((!PACK || kg < 2) && t < g.T && col < g.N) Pz[(size_t)t * g.N + col] = v;
        }
}

// ---------------------------------------------------------------- causal attention over the chunk
// One workgroup of PF_ATT_WAVES waves per (32 query rows, head); wave w takes the key tiles w,
// w + PF_ATT_WAVES, ... with its own running maximum, sum and output tile, and the partial results
// are merged through LDS at the end (a single wave walking up to T/32 tiles one after the other is
// the critical path of the whole kernel under the causal mask).  S^T = K . Q^T, so lane
// (q = l % 32, g = l / 32) ends up with the scores of query q against keys 8 * (i / 4) + 4 * g + i % 4,
// i = 0..15 -- exactly the operand layout P needs in O += P . V.  Softmax statistics are per lane (+ one
// exchange with lane l ^ 32); the rescale factors of the O rows travel through LDS, and only in the
// tiles where some row's maximum grew; the causal mask is applied only in tiles that reach past the
// block's first query.  Scores carry a factor log2(e), so the exponentials are bare v_exp_f32.
// fp32 cache: both products on the fp32 MFMA (32x32x2: lane l supplies row l % 32 and reduction element
// l / 32 of both operands).  bf16 cache: both on the bf16 MFMA (32x32x16) -- keys and values are bf16
// numbers already; the scaled query rows and the probabilities enter as (hi, lo) bf16 pairs, like the
// activations of the GEMMs, so nothing is rounded to 8 bits.  The query pair tile is shared by the
// four waves and lives in LDS (chunks of a row permuted by the row index, so that 16 rows' reads of
// one chunk spread over all banks); in registers it cost 64 per lane and the loop spilled.
// (kernels/sdpa_fwd.rs:325-354: softmax(q . k^T / sqrt(hd) + causal mask) . v)
#define PF_ATT_WAVES 4
template <int KVBF16, int HD>
__global__ __launch_bounds__(64 * PF_ATT_WAVES) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_pf_attn(const float *__restrict__ q, const void *__restrict__ kc,
                                                const void *__restrict__ vc, uint16_t *__restrict__ ohi,
                                                uint16_t *__restrict__ olo, int T, int Q, int KV, int gqa, int pos0,
                                                int seq, float scale, int f16) {
    constexpr int HK = HD / 2;                 // reduction elements per lane group in S
    constexpr int NT = HD / 32;                // 32-wide column tiles of O
    constexpr int VS = HD + 8;                 // LDS row stride of the fp32 V tile (floats)
    constexpr int VSB = HD + 16;               // bf16 V tile: elements per LDS row (rows 4 apart fall 32 banks apart)
    constexpr int KESZ = KVBF16 ? 2 : 4;
    constexpr int CPR = HD * KESZ / 16;        // 16-byte chunks per cache row
    constexpr int KCH = HK * KESZ / 16;        // chunks of this lane's half row
    constexpr int VCH = 32 * CPR / 64;         // V-tile chunks per lane
    constexpr int QCH = HD / 8;                // 16-byte chunks of a bf16 query row
    // LDS.  fp32 cache: a V tile per wave, which also takes the wave's output tile for the merge.  bf16 cache:
    // the query pair tile and a V tile per wave; the merge (two output tiles at a time) reuses that space.
    constexpr int Q_BYTES = 2 * 32 * HD * 2, VB_BYTES = 32 * VSB * 2, MERGE_BYTES = 2 * 16 * NT * 64 * 4;
    constexpr int LOOP_BYTES = Q_BYTES + PF_ATT_WAVES * VB_BYTES;
    constexpr int LDS_BYTES = KVBF16 ? (LOOP_BYTES > MERGE_BYTES ? LOOP_BYTES : MERGE_BYTES) : PF_ATT_WAVES * 32 * VS * 4;
    __shared__ __align__(16) char smem[LDS_BYTES];
    __shared__ __align__(16) float sfacw[PF_ATT_WAVES][32], sfow[PF_ATT_WAVES][32];
    __shared__ float s_m[PF_ATT_WAVES][32], s_l[PF_ATT_WAVES][32];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, g = lane >> 5;
    float *sV = (float *)smem + wave * 32 * VS, *sfac = sfacw[wave];
    uint16_t *sQh = (uint16_t *)smem, *sQl = sQh + 32 * HD;
    uint16_t *sVb = (uint16_t *)(smem + (KVBF16 ? Q_BYTES + wave * VB_BYTES : 0));
    // LDS traffic inside the key loop stays within one wave (its own tile and factors): program order
    // is enough for the hardware, the fence keeps the compiler from reordering LDS accesses across it
    // (a fence over every address space also made it write the loaded V chunks to scratch and back)
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
    };
    // Which (query block, head) this workgroup takes.  Workgroups are dealt to the 8 XCDs round-robin by their
    // linear index, and each XCD has its own L2: with whole heads per XCD (heads a multiple of 8) a head's keys
    // and values are fetched into one L2 instead of all eight, and within an XCD the query blocks run from
    // the last (most keys) to the first, so the long ones do not end up as the tail of the launch.
    int qb = blockIdx.x, h = blockIdx.y;
    if ((gridDim.y & 7) == 0) {
        const int L = blockIdx.x + gridDim.x * blockIdx.y, xcd = L & 7, j = L >> 3;
        h = xcd * (gridDim.y >> 3) + j / gridDim.x;
        qb = gridDim.x - 1 - j % gridDim.x;
    }
    const int q0 = qb * 32, kvh = h / gqa;
    const int tq = min(q0 + r, T - 1);
    const int qpos = pos0 + q0 + r;            // position of this lane's query row
    const float sc2 = scale * 1.44269504088896341f;

    float qf[KVBF16 ? 1 : HK];
    int qoff[KVBF16 ? KCH : 1];                // element offsets of this lane's operand chunks inside its query row
    if constexpr (KVBF16 != 0) {
        // this lane's half of the query row in operand chunks of 8 elements; the four waves share the work
        const int rx = r & (QCH - 1);
#pragma unroll
        for (int c = 0; c < KCH; ++c) qoff[c] = r * HD + (((g * KCH + c) ^ rx) << 3);
        for (int c = wave; c < KCH; c += PF_ATT_WAVES) {
            const float *qp = q + (size_t)tq * Q + h * HD + HK * g + 8 * c;
            const float4 a = *(const float4 *)qp, b = *(const float4 *)(qp + 4);
            uint32_t wh[4], wl[4];
            pf_split2(a.x * sc2, a.y * sc2, wh[0], wl[0]);
            pf_split2(a.z * sc2, a.w * sc2, wh[1], wl[1]);
            pf_split2(b.x * sc2, b.y * sc2, wh[2], wl[2]);
            pf_split2(b.z * sc2, b.w * sc2, wh[3], wl[3]);
            const int o = r * HD + (((g * KCH + c) ^ rx) << 3);
            *(uint4 *)(sQh + o) = make_uint4(wh[0], wh[1], wh[2], wh[3]);
            *(uint4 *)(sQl + o) = make_uint4(wl[0], wl[1], wl[2], wl[3]);
        }
        __syncthreads();
    } else {
        const float *qp = q + (size_t)tq * Q + h * HD + HK * g;
#pragma unroll
        for (int s = 0; s < HK; s += 4) {
            const float4 v = *(const float4 *)(qp + s);
            qf[KVBF16 ? 0 : s] = v.x * sc2; qf[KVBF16 ? 0 : s + 1] = v.y * sc2;
            qf[KVBF16 ? 0 : s + 2] = v.z * sc2; qf[KVBF16 ? 0 : s + 3] = v.w * sc2;
        }
    }
    pf_f32x16 accO[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) accO[nt][i] = 0.0f;
    float m_run = -1e30f, l_run = 0.0f;

    const int last_pos = pos0 + min(q0 + 31, T - 1);
    const char *kbase = (const char *)kc + (size_t)kvh * HD * KESZ;
    const char *vbase = (const char *)vc + (size_t)kvh * HD * KESZ;
    const size_t rowb = (size_t)KV * KESZ;
    for (int kt0 = 32 * wave; kt0 <= last_pos; kt0 += 32 * PF_ATT_WAVES) {
        wave_sync();                           // the previous tile's reads of the V tile are done
        // this lane's key row (its half of the head dimension) and its share of the V tile
        uint4 kr[KCH], vr[VCH];
        {
            const int krow = min(kt0 + r, seq - 1);
            const char *kp = kbase + (size_t)krow * rowb + (size_t)g * HK * KESZ;
#pragma unroll
            for (int c = 0; c < KCH; ++c) kr[c] = *(const uint4 *)(kp + c * 16);
#pragma unroll
            for (int c = 0; c < VCH; ++c) {
                const int ch = lane + 64 * c, vrow = min(kt0 + ch / CPR, seq - 1), cc = ch % CPR;
                vr[c] = *(const uint4 *)(vbase + (size_t)vrow * rowb + cc * 16);
            }
        }
        // the V tile goes to LDS first, so that its registers are free during the products (and no fence
        // stands between its loads and its stores: across one the compiler parks the chunks in scratch)
        if constexpr (KVBF16 != 0) {
#pragma unroll
            for (int c = 0; c < VCH; ++c) {
                const int ch = lane + 64 * c, vrow = ch / CPR, cc = ch % CPR;
                *(uint4 *)(sVb + vrow * VSB + cc * 8) = vr[c];
            }
        } else {
#pragma unroll
            for (int c = 0; c < VCH; ++c) {
                const int ch = lane + 64 * c, vrow = ch / CPR, cc = ch % CPR;
                float vf[16 / KESZ];
                WS<KVBF16 ? WT_BF16 : WT_F32>::decode(vr[c], vf);
                float *dst = sV + vrow * VS + cc * (16 / KESZ);
#pragma unroll
                for (int e = 0; e < 16 / KESZ; e += 4) *(float4 *)(dst + e) = make_float4(vf[e], vf[e + 1], vf[e + 2], vf[e + 3]);
            }
        }
        pf_f32x16 accS;
#pragma unroll
        for (int i = 0; i < 16; ++i) accS[i] = 0.0f;
        if constexpr (KVBF16 != 0) {
            // chunk c of this lane's half key row is an operand as it is: reduction slot (g, e) of step c
            // is element g * HK + 8 c + e of the head dimension for the key and for the query alike
#pragma unroll
            for (int c = 0; c < KCH; ++c) {
                const uint4 qh = *(const uint4 *)(sQh + qoff[KVBF16 ? c : 0]), ql = *(const uint4 *)(sQl + qoff[KVBF16 ? c : 0]);
                accS = pf_mma(kr[c], qh, accS, false);
                accS = pf_mma(kr[c], ql, accS, false);
            }
        } else {
#pragma unroll
            for (int c = 0; c < KCH; ++c) {
                float kf[16 / KESZ];
                WS<KVBF16 ? WT_BF16 : WT_F32>::decode(kr[c], kf);
#pragma unroll
                for (int e = 0; e < 16 / KESZ; ++e)
                    accS = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[e], qf[KVBF16 ? 0 : c * (16 / KESZ) + e], accS, 0, 0, 0);
            }
        }
        // online softmax for query row r over this tile's 32 keys (16 here, 16 in lane r ^ 32); a tile that
        // ends at or before the block's first query needs no mask
        const bool full = kt0 + 31 <= pos0 + q0;
        float tmax = -1e30f;
        if (full) {
#pragma unroll
            for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, accS[i]);
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (kt0 + 8 * (i >> 2) + 4 * g + (i & 3) <= qpos) tmax = fmaxf(tmax, accS[i]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);
        const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
        const bool grew = __any(m_new > m_run) != 0;      // some row of this wave moved its maximum: the O rows need rescaling
        float psum = 0.0f;
        float p[16];
        if (full) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                p[i] = __builtin_amdgcn_exp2f(accS[i] - m_new);
                psum += p[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                p[i] = kt0 + 8 * (i >> 2) + 4 * g + (i & 3) <= qpos ? __builtin_amdgcn_exp2f(accS[i] - m_new) : 0.0f;
                psum += p[i];
            }
        }
        psum += __shfl_xor(psum, 32, 64);
        l_run = l_run * corr + psum;
        m_run = m_new;
        if (grew && g == 0) sfac[r] = corr;
        wave_sync();                           // V tile and rescale factors are in LDS
        if (grew) {
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4) {
                const float4 f = *(const float4 *)(sfac + 8 * j4 + 4 * g);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    accO[nt][4 * j4] *= f.x; accO[nt][4 * j4 + 1] *= f.y;
                    accO[nt][4 * j4 + 2] *= f.z; accO[nt][4 * j4 + 3] *= f.w;
                }
            }
        }
        if constexpr (KVBF16 != 0) {
            // two steps of 16 keys: reduction slot (g, e) of step t is key 16 t + 8 (e / 4) + 4 g + e % 4, the
            // key this lane's p[8 t + e] belongs to; the value operand gathers that key's column element
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                uint32_t ph[4], pl[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) pf_split2(p[8 * t + 2 * e], p[8 * t + 2 * e + 1], ph[e], pl[e]);
                const uint4 Ph = make_uint4(ph[0], ph[1], ph[2], ph[3]), Pl = make_uint4(pl[0], pl[1], pl[2], pl[3]);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    uint32_t vb[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int key = 16 * t + 8 * (e >> 1) + 4 * g + 2 * (e & 1);      // slots 2 e and 2 e + 1: this key and the next
                        vb[e] = (uint32_t)sVb[key * VSB + 32 * nt + r] | ((uint32_t)sVb[(key + 1) * VSB + 32 * nt + r] << 16);
                    }
                    const uint4 Vb = make_uint4(vb[0], vb[1], vb[2], vb[3]);
                    accO[nt] = pf_mma(Ph, Vb, accO[nt], false);
                    accO[nt] = pf_mma(Pl, Vb, accO[nt], false);
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                const int key = 8 * (s >> 2) + 4 * g + (s & 3);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    accO[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(p[s], sV[key * VS + 32 * nt + r], accO[nt], 0, 0, 0);
            }
        }
    }
    // merge the waves' partial results: O = sum_w e_w O_w / sum_w e_w l_w with e_w = 2^(m_w - max m)
    if constexpr (KVBF16 != 0) {
        // in registers, as a tree: waves 2 and 3 hand their tiles to waves 0 and 1, then wave 1 to wave 0 (every
        // wave holds its tile in the same layout, so a tile crosses LDS lane by lane)
        __syncthreads();                       // every wave is done with the query tile and its own V tile
        float *mb = (float *)smem;
        auto put = [&](int slot) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int i = 0; i < 16; ++i) mb[((slot * NT + nt) * 16 + i) * 64 + lane] = accO[nt][i];
            if (g == 0) { s_m[wave][r] = m_run; s_l[wave][r] = l_run; }
        };
        auto take = [&](int slot, int other) {
            const float mo = s_m[other][r], lo = s_l[other][r];
            const float M = fmaxf(m_run, mo);
            const float fs = __builtin_amdgcn_exp2f(m_run - M), fo = __builtin_amdgcn_exp2f(mo - M);
            l_run = fs * l_run + fo * lo;
            m_run = M;
            if (g == 0) { sfacw[wave][r] = fs; sfow[wave][r] = fo; }
            wave_sync();
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int qi = 8 * (i >> 2) + 4 * g + (i & 3);
                const float a = sfacw[wave][qi], b = sfow[wave][qi];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    accO[nt][i] = accO[nt][i] * a + mb[((slot * NT + nt) * 16 + i) * 64 + lane] * b;
            }
            wave_sync();                       // the factors are read before the next merge overwrites them
        };
        if (wave >= 2) put(wave - 2);
        __syncthreads();
        if (wave < 2) take(wave, wave + 2);
        __syncthreads();
        if (wave == 1) put(0);
        __syncthreads();
        if (wave == 0) {
            take(0, 1);
            if (g == 0) sfacw[0][r] = l_run > 0.0f ? 1.0f / l_run : 0.0f;
            wave_sync();
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int qi = 8 * (i >> 2) + 4 * g + (i & 3), t = q0 + qi;
                const float inv = sfacw[0][qi];
                if (t < T) {
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const size_t o = (size_t)t * Q + h * HD + 32 * nt + r;
                        pf_split(accO[nt][i] * inv, ohi[o], olo[o], f16);
                    }
                }
            }
        }
    } else {
        wave_sync();
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int qi = 8 * (i >> 2) + 4 * g + (i & 3);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) sV[qi * VS + 32 * nt + r] = accO[nt][i];
        }
        if (g == 0) { s_m[wave][r] = m_run; s_l[wave][r] = l_run; }
        __syncthreads();
        const float *sVall = (const float *)smem;
        for (int idx = threadIdx.x; idx < 32 * HD; idx += 64 * PF_ATT_WAVES) {
            const int qi = idx / HD, d = idx - qi * HD, t = q0 + qi;
            float M = -1e30f;
#pragma unroll
            for (int w = 0; w < PF_ATT_WAVES; ++w) M = fmaxf(M, s_m[w][qi]);
            float num = 0.0f, den = 0.0f;
#pragma unroll
            for (int w = 0; w < PF_ATT_WAVES; ++w) {
                const float e = __builtin_amdgcn_exp2f(s_m[w][qi] - M);
                den += e * s_l[w][qi];
                num += e * sVall[w * 32 * VS + qi * VS + d];
            }
            if (t < T) {
                const size_t o = (size_t)t * Q + h * HD + d;
                pf_split(den > 0.0f ? num / den : 0.0f, ohi[o], olo[o], f16);
            }
        }
    }
}
