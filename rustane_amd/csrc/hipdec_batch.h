// Multi-sample decode for gfx950: R continuations of one shared prompt prefix advance together, so
// each weight matrix is streamed once per step for all R rows.
//
// The reference runs its samples one after the other (engine/src/inference.rs:247-262: `samples`
// sequential runs, each re-seeding the KV cache from the shared prompt caches, :561).  Here the
// prompt's keys and values stay where the prefill put them (positions [0, prefix) of the model's
// caches, read by every row) and each row appends its own keys and values to a per-row suffix
// cache.  The projections reuse the prefill GEMM (hipdec_prefill.h) with T = R rows; this file
// adds what differs from prefill: all rows sit at the same position, attention reads prefix +
// own suffix, and the head kernels run once per row.
#pragma once
#include "hipdec_prefill.h"

struct BatchParams {         // device-resident, rewritten before every step (so one captured graph serves all steps)
    int pos;                 // position of the tokens of this step = prefix + slot
    int slot;                // index into the per-row suffix caches
    int prefix;              // shared prefix length
    int top_k;
    float inv_t, softcap;
};

// q/k/v rows of the step: sum the split planes, scale (8-bit weights), RoPE at the common position,
// q kept as fp32, k and v appended to the row's suffix cache in cache precision.
template <int KVBF16>
__global__ __launch_bounds__(256) void k_bd_qkv_epi(const float *__restrict__ P, int splits, size_t plane,
                                                    const float *__restrict__ wscale, float *__restrict__ q,
                                                    void *__restrict__ kc_suf, void *__restrict__ vc_suf, size_t suf_rows,
                                                    const float *__restrict__ rope_cos, const float *__restrict__ rope_sin,
                                                    const BatchParams *__restrict__ bp, const float *__restrict__ ssq,
                                                    int nch, int D, int R, int Q, int KV, int hd) {
    const int N = Q + 2 * KV, npairs = N >> 1;
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (size_t)R * npairs) return;
    const int t = (int)(gid / npairs), p = (int)(gid - (size_t)t * npairs), row0 = 2 * p;
    float sv[2] = {0.0f, 0.0f};
    pf_sum_planes<2>(P, splits, plane, (size_t)t * N + row0, sv);
    float s0 = sv[0], s1 = sv[1];
    if (wscale) { s0 *= wscale[row0]; s1 *= wscale[row0 + 1]; }
    const float inv = pf_row_inv(ssq, t, nch, D);
    s0 *= inv; s1 *= inv;
    const int pos = bp->pos;
    if (row0 < Q + KV) {
        const int rr = row0 < Q ? row0 : row0 - Q;
        const int pi2 = (rr % hd) >> 1;
        const float c = rope_cos[(size_t)pos * (hd / 2) + pi2], s = rope_sin[(size_t)pos * (hd / 2) + pi2];
        const float e = s0 * c - s1 * s, o = s1 * c + s0 * s;
        s0 = e; s1 = o;
    }
    if (row0 < Q) {
        *(float2 *)(q + (size_t)t * Q + row0) = make_float2(s0, s1);
    } else {
        const bool isk = row0 < Q + KV;
        const int rr = isk ? row0 - Q : row0 - Q - KV;
        void *cache = isk ? kc_suf : vc_suf;
        const size_t at = ((size_t)t * suf_rows + bp->slot) * KV + rr;
        if (KVBF16) {
            uint16_t *cp = (uint16_t *)cache + at;
            cp[0] = f32_to_bf16_rne(s0); cp[1] = f32_to_bf16_rne(s1);
        } else {
            float *cp = (float *)cache + at;
            cp[0] = s0; cp[1] = s1;
        }
    }
}

// One workgroup per (head, row): online softmax over the shared prefix rows and then the row's own
// suffix rows (same arithmetic as the single-row decode attention; crates/metal-decode/src/lib.rs:1426-1489),
// result as the hi/lo pair the output projection reads.
#define BD_ATT_THREADS 1024
template <int KVBF16, int HD>
__global__ __launch_bounds__(BD_ATT_THREADS) void k_bd_attn(const float *__restrict__ q, const void *__restrict__ kc,
                                                 const void *__restrict__ vc, const void *__restrict__ kc_suf,
                                                 const void *__restrict__ vc_suf, size_t suf_rows,
                                                 const BatchParams *__restrict__ bp, uint16_t *__restrict__ ohi,
                                                 uint16_t *__restrict__ olo, int Q, int KV, int gqa, float scale) {
    constexpr int ESZ = KVBF16 ? 2 : 4;
    constexpr int EPL = 16 / ESZ;          // elements per 16-byte load
    constexpr int LPR = HD / EPL;          // lanes per cache row
    constexpr int RPI = 64 / LPR;          // rows per wave instruction
    constexpr int SLOTS = (BD_ATT_THREADS / 64) * RPI;
    constexpr int UNR = 4;                 // cache rows in flight per thread
    __shared__ float sm[SLOTS][HD + 2];
    const int h = blockIdx.x, row = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane % LPR, r = lane / LPR;
    const int prefix = bp->prefix, n = prefix + bp->slot + 1;
    const int g = h / gqa;

    float qv[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) qv[e] = q[(size_t)row * Q + h * HD + sub * EPL + e] * scale;
    float m = -INFINITY, l = 0.0f, acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.0f;

    const size_t rowb = (size_t)KV * ESZ, hoff = ((size_t)g * HD + sub * EPL) * ESZ;
    const char *kb = (const char *)kc + hoff, *vb = (const char *)vc + hoff;
    const char *ksb = (const char *)kc_suf + (size_t)row * suf_rows * rowb + hoff;
    const char *vsb = (const char *)vc_suf + (size_t)row * suf_rows * rowb + hoff;
    for (int tb = wave * RPI + r; tb < n; tb += SLOTS * UNR) {
        uint4 kw[UNR], vw[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int t = tb + u * SLOTS;
            if (t < n) {
                const bool shared = t < prefix;
                const size_t at = (size_t)(shared ? t : t - prefix) * rowb;
                kw[u] = *(const uint4 *)((shared ? kb : ksb) + at);
                vw[u] = *(const uint4 *)((shared ? vb : vsb) + at);
            }
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            // the rows of one lane group are either all present or all past the end, so the
            // reduction below stays inside converged lanes
            if (tb + u * SLOTS < n) {
                float kf[EPL], vf[EPL];
                WS<KVBF16 ? WT_BF16 : WT_F32>::decode(kw[u], kf);
                WS<KVBF16 ? WT_BF16 : WT_F32>::decode(vw[u], vf);
                float d = 0.0f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) d = fmaf(qv[e], kf[e], d);
#pragma unroll
                for (int o = LPR >> 1; o > 0; o >>= 1) d += __shfl_xor(d, o, WAVE);
                const float mn = fmaxf(m, d);
                const float corr = __expf(m - mn), p = __expf(d - mn);
                l = l * corr + p;
#pragma unroll
                for (int e = 0; e < EPL; ++e) acc[e] = acc[e] * corr + p * vf[e];
                m = mn;
            }
        }
    }
    {
        const int slot = wave * RPI + r;
#pragma unroll
        for (int e = 0; e < EPL; ++e) sm[slot][sub * EPL + e] = acc[e];
        if (sub == 0) { sm[slot][HD] = m; sm[slot][HD + 1] = l; }
    }
    __syncthreads();
    if (tid < HD) {
        float M = -INFINITY;
#pragma unroll
        for (int k = 0; k < SLOTS; ++k) M = fmaxf(M, sm[k][HD]);
        float L = 0.0f, A = 0.0f;
        if (M > -INFINITY) {
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                const float w = __expf(sm[k][HD] - M);     // exp(-inf) = 0 for empty slots
                L += sm[k][HD + 1] * w;
                A += sm[k][tid] * w;
            }
        }
        const size_t o = (size_t)row * Q + h * HD + tid;
        pf_split(L > 0.0f ? A / L : 0.0f, ohi[o], olo[o]);
    }
}

// logits[r][v] = inv_rms[r] * sum_z P[z][r][v]   (the final RMSNorm's row factor, applied after the product)
__global__ __launch_bounds__(256) void k_bd_sum_planes(const float *__restrict__ P, int splits, size_t plane,
                                                       float *__restrict__ out, size_t n, const float *__restrict__ ssq,
                                                       int nch, int D, int V) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = 0.0f;
    pf_sum_planes<1>(P, splits, plane, i, &s);
    out[i] = s * pf_row_inv(ssq, (int)(i / V), nch, D);
}

// ---- head kernels, one grid row per sequence (same selection rules as the single-row kernels)
__global__ __launch_bounds__(1024) void k_bd_argmax(const float *__restrict__ logits, int V, uint32_t *__restrict__ out) {
    __shared__ float sv[16];
    __shared__ uint32_t si[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *lg = logits + (size_t)blockIdx.x * V;
    float bv = -INFINITY; uint32_t bi = 0xffffffffu;
    for (int i = tid; i < V; i += 1024) {
        const float v = lg[i];
        if (better(v, (uint32_t)i, bv, bi)) { bv = v; bi = (uint32_t)i; }
    }
    wave_argbest(bv, bi);
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 16; ++w) if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        out[blockIdx.x] = bi;
    }
}

__global__ __launch_bounds__(256) void k_bd_topk(const float *__restrict__ logits, int V, const BatchParams *__restrict__ bp,
                                                 float *__restrict__ out_vals, uint32_t *__restrict__ out_idxs) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int top_k = bp->top_k;
    const float *lg = logits + (size_t)blockIdx.y * V;
    const size_t obase = ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * top_k;
    const int row = blockIdx.x * 256 + tid;
    float cv = -INFINITY; uint32_t ci = 0xffffffffu;
    if (row < V) { cv = lg[row]; ci = (uint32_t)row; }
    for (int rank = 0; rank < top_k; ++rank) {
        float bv = cv; uint32_t bi = ci;
        wave_argbest(bv, bi);
        if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
        __syncthreads();
        bv = sv[0]; bi = si[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        if (tid == 0) { out_vals[obase + rank] = bv; out_idxs[obase + rank] = bi; }
        if (ci == bi) { cv = -INFINITY; ci = 0xffffffffu; }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void k_bd_block_stats(const float *__restrict__ logits, int V,
                                                        const BatchParams *__restrict__ bp, float *__restrict__ maxes,
                                                        float *__restrict__ sums) {
    __shared__ float sr[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *lg = logits + (size_t)blockIdx.y * V;
    const int row = blockIdx.x * 256 + tid;
    float val = -INFINITY;
    if (row < V) val = softcap_dev(lg[row], bp->softcap) * bp->inv_t;
    float mx = wave_max(val);
    if (lane == 0) sr[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(sr[0], sr[1]), fmaxf(sr[2], sr[3]));
    __syncthreads();
    float e = row < V ? expf(val - mx) : 0.0f;
    e = wave_sum(e);
    if (lane == 0) sr[wave] = e;
    __syncthreads();
    if (tid == 0) {
        const size_t o = (size_t)blockIdx.y * gridDim.x + blockIdx.x;
        maxes[o] = mx; sums[o] = (sr[0] + sr[1]) + (sr[2] + sr[3]);
    }
}
