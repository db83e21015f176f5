// Decode-step kernels for gfx950: row-per-wave GEMVs with fused prologues/epilogues, split-sequence
// attention over the HBM-resident KV cache, and the head reductions.
#pragma once
#include "hipdec_common.h"

enum { EPI_QKV = 0, EPI_WO = 1, EPI_W13 = 2, EPI_W2 = 3, EPI_HEAD = 4 };

// ---------------------------------------------------------------- embedding / input
// crates/metal-decode/src/lib.rs:1380-1390 embed_lookup (or the x_in upload of decode_token)
template <int WT>
__global__ void k_embed(const void *__restrict__ embed, const float *__restrict__ x_in,
                        const StepParams *__restrict__ sp, float *__restrict__ x, int D) {
    int d = blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= D) return;
    if (sp->use_x_in) { x[d] = x_in[d]; return; }
    size_t idx = (size_t)sp->tok * D + d;
    if (WT == WT_F32) x[d] = ((const float *)embed)[idx];
    else x[d] = bf16_to_f32(((const uint16_t *)embed)[idx]);
}

// ---------------------------------------------------------------- GEMV
struct GemvArgs {
    const void *W;          // out-major weights [rows][K]
    const void *scales;     // fp8: float[rows]; int4: bf16[rows][K/128]
    const float *in;        // input vector [K] (pre-norm residual stream when the prologue norms)
    const float *gamma;     // [K] when the prologue norms
    const float *resid;     // WO / W2: residual input [rows]
    float *out;             // QKV: q [q_dim]; WO/W2: x [rows]; W13: gate [rows/2]; HEAD: logits [rows]
    void *kc, *vc;          // QKV: this layer's caches [seq][kv_dim]
    const float *rope_cos, *rope_sin;   // [seq][hd/2]
    const StepParams *sp;
    int rows, K;
    int q_dim, kv_dim, hd;
    float alpha;
    int act;                // W13: 0 SwiGLU, 1 leaky_relu(x,0.5)^2
};

// R consecutive output rows per wave, the whole reduction axis inside the wave.  The input
// vector sits in LDS as fp32 (normalised on the way in when NORM), each lane streams 16-byte
// pieces of its rows, accumulates in fp32 and the wave reduces with cross-lane shuffles in a
// fixed order, so results are run-to-run identical.
template <int WT, int EPI, int KVBF16>
__global__ __launch_bounds__(256) void k_gemv(GemvArgs a) {
    constexpr int R = 2;
    constexpr int EPL = WS<WT>::EPL;
    constexpr bool NORM = (EPI == EPI_QKV || EPI == EPI_W13 || EPI == EPI_HEAD);
    extern __shared__ __align__(16) float xs[];
    __shared__ float red[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = a.K;

    // prologue: input vector -> LDS (RMSNorm: crates/metal-decode/src/lib.rs:1354-1378)
    if (NORM) {
        float ss = 0.0f;
        for (int i = tid; i < K; i += 256) { float v = a.in[i]; xs[i] = v; ss += v * v; }
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        float tot = red[0] + red[1] + red[2] + red[3];
        float inv = 1.0f / sqrtf(tot * (1.0f / (float)K) + 1e-5f);
        for (int i = tid; i < K; i += 256) xs[i] = xs[i] * inv * a.gamma[i];
    } else {
        for (int i = tid; i < K; i += 256) xs[i] = a.in[i];
    }
    __syncthreads();

    const int n_groups = (a.rows + R - 1) / R;
    const int waves_total = gridDim.x * 4;
    const size_t rb = WS<WT>::row_bytes(K);
    const int n_chunks = K / EPL;
    const int pos = a.sp->pos;

    for (int g = blockIdx.x * 4 + wave; g < n_groups; g += waves_total) {
        const int row0 = g * R;
        const char *wr[R];
        int rowi[R];
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            rowi[r] = min(row0 + r, a.rows - 1);          // an odd row count re-reads its last row
            wr[r] = (const char *)a.W + (size_t)rowi[r] * rb;
            acc[r] = 0.0f;
        }
#pragma unroll 4
        for (int c = lane; c < n_chunks; c += 64) {
            uint4 wv[R];
#pragma unroll
            for (int r = 0; r < R; ++r) wv[r] = *(const uint4 *)(wr[r] + (size_t)c * 16);
            float xv[EPL];
#pragma unroll
            for (int e = 0; e < EPL; e += 4) {
                float4 t = *(const float4 *)(xs + c * EPL + e);
                xv[e] = t.x; xv[e + 1] = t.y; xv[e + 2] = t.z; xv[e + 3] = t.w;
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float wf[EPL];
                WS<WT>::decode(wv[r], wf);
                float p = 0.0f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) p = fmaf(wf[e], xv[e], p);
                if (WT == WT_INT4) {
                    const uint16_t *sc = (const uint16_t *)a.scales + (size_t)rowi[r] * (K / 128);
                    p *= bf16_to_f32(sc[(c * EPL) / 128]) * WS<WT_INT4>::SCALE_MUL;
                }
                acc[r] += p;
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
        if (lane == 0) {
            if (WT == WT_FP8) {
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r] *= ((const float *)a.scales)[rowi[r]];
            }
            if (EPI == EPI_QKV) {
                // rows [0,Q) q, [Q,Q+KV) k, [Q+KV,Q+2KV) v; RoPE on the pair (row0,row0+1):
                // crates/metal-decode/src/lib.rs:1392-1408; append: :1410-1424
                const int Q = a.q_dim, KV = a.kv_dim, hp = a.hd / 2;
                if (row0 < Q + KV) {
                    int rr = row0 < Q ? row0 : row0 - Q;
                    int pi = (rr % a.hd) >> 1;
                    float c = a.rope_cos[(size_t)pos * hp + pi], s = a.rope_sin[(size_t)pos * hp + pi];
                    float e = acc[0] * c - acc[1] * s;
                    float o = acc[1] * c + acc[0] * s;
                    if (row0 < Q) { a.out[row0] = e; a.out[row0 + 1] = o; }
                    else if (KVBF16) {
                        uint16_t *kc = (uint16_t *)a.kc + (size_t)pos * KV + rr;
                        kc[0] = f32_to_bf16_rne(e); kc[1] = f32_to_bf16_rne(o);
                    } else {
                        float *kc = (float *)a.kc + (size_t)pos * KV + rr;
                        kc[0] = e; kc[1] = o;
                    }
                } else {
                    int rr = row0 - Q - KV;
                    if (KVBF16) {
                        uint16_t *vc = (uint16_t *)a.vc + (size_t)pos * KV + rr;
                        vc[0] = f32_to_bf16_rne(acc[0]); vc[1] = f32_to_bf16_rne(acc[1]);
                    } else {
                        float *vc = (float *)a.vc + (size_t)pos * KV + rr;
                        vc[0] = acc[0]; vc[1] = acc[1];
                    }
                }
            } else if (EPI == EPI_WO || EPI == EPI_W2) {
                // x + alpha*y: crates/metal-decode/src/lib.rs:1491-1502 and the w2 GEMV's
                // alpha/beta at :1189-1201
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (row0 + r < a.rows) a.out[row0 + r] = a.resid[row0 + r] + a.alpha * acc[r];
            } else if (EPI == EPI_W13) {
                // rows (2h, 2h+1) = (gate, up) of hidden unit h: lib.rs:1504-1513
                float h1 = acc[0], h3 = acc[1], gte;
                if (a.act == 1) { float l = h1 > 0.0f ? h1 : 0.5f * h1; gte = l * l * h3; }
                else { float sig = 1.0f / (1.0f + expf(-h1)); gte = h1 * sig * h3; }
                a.out[row0 >> 1] = gte;
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (row0 + r < a.rows) a.out[row0 + r] = acc[r];
            }
        }
    }
}

// ---------------------------------------------------------------- attention (one query row)
// grid (heads, NS): workgroup (h, s) covers cache rows [s*chunk, (s+1)*chunk) of head h with an
// online softmax, writes (max, sum, acc[HD]) and the last workgroup of a head to finish folds the
// NS partials in split order.  Replaces sdpa_causal, crates/metal-decode/src/lib.rs:1426-1489.
template <int KVBF16, int HD>
__global__ __launch_bounds__(256) void k_attn_decode(const float *__restrict__ q, const void *__restrict__ kc,
                                                     const void *__restrict__ vc, const StepParams *__restrict__ sp,
                                                     float *__restrict__ part, unsigned *__restrict__ counters,
                                                     float *__restrict__ att, int KV, int gqa, int NS, float scale) {
    constexpr int ESZ = KVBF16 ? 2 : 4;
    constexpr int EPL = 16 / ESZ;          // elements per 16-byte load
    constexpr int LPR = HD / EPL;          // lanes per cache row
    constexpr int RPI = 64 / LPR;          // rows per wave instruction
    constexpr int SLOTS = 4 * RPI;
    __shared__ float sm[SLOTS][HD + 2];
    __shared__ int s_last;
    const int h = blockIdx.x, s = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane % LPR, r = lane / LPR;
    const int n = sp->pos + 1;
    const int chunk = (n + NS - 1) / NS;
    const int t0 = s * chunk, t1 = min(n, t0 + chunk);
    const int g = h / gqa;

    float qv[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) qv[e] = q[h * HD + sub * EPL + e] * scale;
    float m = -INFINITY, l = 0.0f, acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.0f;

    const char *kb = (const char *)kc + ((size_t)g * HD + sub * EPL) * ESZ;
    const char *vb = (const char *)vc + ((size_t)g * HD + sub * EPL) * ESZ;
    const size_t rowb = (size_t)KV * ESZ;
    for (int t = t0 + wave * RPI + r; t < t1; t += SLOTS) {
        uint4 kw = *(const uint4 *)(kb + (size_t)t * rowb);
        uint4 vw = *(const uint4 *)(vb + (size_t)t * rowb);
        float kf[EPL], vf[EPL];
        WS<KVBF16 ? WT_BF16 : WT_F32>::decode(kw, kf);
        WS<KVBF16 ? WT_BF16 : WT_F32>::decode(vw, vf);
        float d = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) d = fmaf(qv[e], kf[e], d);
#pragma unroll
        for (int o = LPR >> 1; o > 0; o >>= 1) d += __shfl_xor(d, o, WAVE);
        float mn = fmaxf(m, d);
        float corr = __expf(m - mn), p = __expf(d - mn);
        l = l * corr + p;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[e] = acc[e] * corr + p * vf[e];
        m = mn;
    }
    // fold the SLOTS row-slots of this workgroup
    {
        int slot = wave * RPI + r;
#pragma unroll
        for (int e = 0; e < EPL; ++e) sm[slot][sub * EPL + e] = acc[e];
        if (sub == 0) { sm[slot][HD] = m; sm[slot][HD + 1] = l; }
    }
    __syncthreads();
    float *mypart = part + ((size_t)h * NS + s) * (HD + 2);
    if (tid < HD) {
        float M = -INFINITY;
#pragma unroll
        for (int k = 0; k < SLOTS; ++k) M = fmaxf(M, sm[k][HD]);
        float L = 0.0f, A = 0.0f;
        if (M > -INFINITY) {
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                float w = __expf(sm[k][HD] - M);     // exp(-inf) = 0 for empty slots
                L += sm[k][HD + 1] * w;
                A += sm[k][tid] * w;
            }
        }
        mypart[tid] = A;
        if (tid == 0) { mypart[HD] = M; mypart[HD + 1] = L; }
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        unsigned prev = atomicAdd(&counters[h], 1u);
        s_last = (prev == (unsigned)(NS - 1));
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    if (tid < HD) {
        const float *hp = part + (size_t)h * NS * (HD + 2);
        float M = -INFINITY;
        for (int k = 0; k < NS; ++k) M = fmaxf(M, __builtin_nontemporal_load(hp + k * (HD + 2) + HD));
        float L = 0.0f, A = 0.0f;
        for (int k = 0; k < NS; ++k) {
            float mk = __builtin_nontemporal_load(hp + k * (HD + 2) + HD);
            float w = mk > -INFINITY ? __expf(mk - M) : 0.0f;
            L += __builtin_nontemporal_load(hp + k * (HD + 2) + HD + 1) * w;
            A += __builtin_nontemporal_load(hp + k * (HD + 2) + tid) * w;
        }
        att[h * HD + tid] = L > 0.0f ? A / L : 0.0f;
    }
    if (tid == 0) counters[h] = 0u;
}

// ---------------------------------------------------------------- heads (on the raw logits)
// greedy: crates/metal-decode/src/lib.rs:1515-1565 + :1725-1760 collapsed into one scan;
// ties go to the lower index.  Also advances the device-side step state so that a run of
// greedy steps needs no host round trip.
__global__ __launch_bounds__(1024) void k_head_argmax(const float *__restrict__ logits, int V,
                                                      StepParams *__restrict__ sp, uint32_t *__restrict__ out_ring,
                                                      int ring_cap) {
    __shared__ float sv[16];
    __shared__ uint32_t si[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float bv = -INFINITY; uint32_t bi = 0xffffffffu;
    for (int i = tid; i < V; i += 1024) {
        float v = logits[i];
        if (better(v, (uint32_t)i, bv, bi)) { bv = v; bi = (uint32_t)i; }
    }
    wave_argbest(bv, bi);
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 16; ++w) if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        int st = sp->step;
        if (st >= 0 && st < ring_cap) out_ring[st] = bi;
        sp->tok = (int)bi;
        sp->pos = sp->pos + 1;
        sp->step = st + 1;
    }
}

// per-block top-k: crates/metal-decode/src/lib.rs:1567-1635
__global__ __launch_bounds__(256) void k_head_topk(const float *__restrict__ logits, int V,
                                                   const StepParams *__restrict__ sp,
                                                   float *__restrict__ out_vals, uint32_t *__restrict__ out_idxs) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int top_k = sp->top_k;
    const int row = blockIdx.x * 256 + tid;
    float cv = -INFINITY; uint32_t ci = 0xffffffffu;
    if (row < V) { cv = logits[row]; ci = (uint32_t)row; }
    for (int rank = 0; rank < top_k; ++rank) {
        float bv = cv; uint32_t bi = ci;
        wave_argbest(bv, bi);
        if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
        __syncthreads();
        bv = sv[0]; bi = si[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        if (tid == 0) { out_vals[blockIdx.x * top_k + rank] = bv; out_idxs[blockIdx.x * top_k + rank] = bi; }
        if (ci == bi) { cv = -INFINITY; ci = 0xffffffffu; }
        __syncthreads();
    }
}

__device__ __forceinline__ float softcap_dev(float x, float cap) { return cap > 0.0f ? cap * tanhf(x / cap) : x; }

// per-block softmax statistics: crates/metal-decode/src/lib.rs:1637-1700
__global__ __launch_bounds__(256) void k_head_block_stats(const float *__restrict__ logits, int V,
                                                          const StepParams *__restrict__ sp,
                                                          float *__restrict__ maxes, float *__restrict__ sums) {
    __shared__ float sr[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.x * 256 + tid;
    float val = -INFINITY;
    if (row < V) val = softcap_dev(logits[row], sp->softcap) * sp->inv_t;
    float mx = wave_max(val);
    if (lane == 0) sr[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(sr[0], sr[1]), fmaxf(sr[2], sr[3]));
    __syncthreads();
    float e = row < V ? expf(val - mx) : 0.0f;
    e = wave_sum(e);
    if (lane == 0) sr[wave] = e;
    __syncthreads();
    if (tid == 0) { maxes[blockIdx.x] = mx; sums[blockIdx.x] = (sr[0] + sr[1]) + (sr[2] + sr[3]); }
}

// softcapped copy of a logit range: the full-logits variant (engine/src/decode.rs:120-124) and
// logits_block_materialize (crates/metal-decode/src/lib.rs:1702-1723)
__global__ void k_softcap_copy(const float *__restrict__ logits, float *__restrict__ out, int start, int n, float cap) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = softcap_dev(logits[start + i], cap);
}

// bump the position after a step whose head does not do it itself
__global__ void k_advance(StepParams *sp) { sp->pos = sp->pos + 1; }

// plain device copy of a known size: the yardstick the memory-traffic counters are scaled by
__global__ __launch_bounds__(256) void k_calib_copy(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

// ---------------------------------------------------------------- weight load (one-time)
// [rows][cols] fp32 -> [cols][rows] fp32 through a 32x32 LDS tile
__global__ void k_transpose_f32(const float *__restrict__ in, float *__restrict__ out, int rows, int cols) {
    __shared__ float t[32][33];
    int bx = blockIdx.x * 32, by = blockIdx.y * 32;
    for (int j = threadIdx.y; j < 32; j += 8) {
        int r = by + j, c = bx + threadIdx.x;
        if (r < rows && c < cols) t[j][threadIdx.x] = in[(size_t)r * cols + c];
    }
    __syncthreads();
    for (int j = threadIdx.y; j < 32; j += 8) {
        int c = bx + j, r = by + threadIdx.x;
        if (r < rows && c < cols) out[(size_t)c * rows + r] = t[threadIdx.x][j];
    }
}

// one workgroup per source row of an out-major fp32 matrix [rows][K]; destination row =
// row*row_mul + row_off (interleaves gate/up rows, concatenates q/k/v)
template <int WT>
__global__ __launch_bounds__(256) void k_convert_rows(const float *__restrict__ src, void *__restrict__ dst,
                                                      void *__restrict__ scales, int K, int row_mul, int row_off) {
    __shared__ float red[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *s = src + (size_t)blockIdx.x * K;
    const size_t drow = (size_t)blockIdx.x * row_mul + row_off;
    if (WT == WT_F32) {
        float *d = (float *)dst + drow * K;
        for (int k = tid; k < K; k += 256) d[k] = s[k];
    } else if (WT == WT_BF16) {
        uint16_t *d = (uint16_t *)dst + drow * K;
        for (int k = tid; k < K; k += 256) d[k] = f32_to_bf16_rne(s[k]);
    } else if (WT == WT_FP8) {
        float am = 0.0f;
        for (int k = tid; k < K; k += 256) am = fmaxf(am, fabsf(s[k]));
        am = wave_max(am);
        if (lane == 0) red[wave] = am;
        __syncthreads();
        am = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        float sc = am > 0.0f ? am / 448.0f : 1.0f;
        if (tid == 0) ((float *)scales)[drow] = sc;
        uint8_t *d = (uint8_t *)dst + drow * K;
        for (int k = tid; k < K; k += 256) d[k] = f32_to_e4m3(s[k] / sc);
    } else {
        // groups of 128 along K; one wave per group, two elements per lane
        const int G = K / 128;
        uint8_t *d = (uint8_t *)dst + drow * (K / 2);
        uint16_t *sc = (uint16_t *)scales + drow * G;
        for (int g = wave; g < G; g += 4) {
            float a0 = s[g * 128 + 2 * lane], a1 = s[g * 128 + 2 * lane + 1];
            float am = wave_max(fmaxf(fabsf(a0), fabsf(a1)));
            uint16_t sb = am > 0.0f ? f32_to_bf16_rne(am / 7.0f) : (uint16_t)0x3f80;
            float scf = bf16_to_f32(sb);
            float r0 = fminf(fmaxf(rintf(a0 / scf), -8.0f), 7.0f);
            float r1 = fminf(fmaxf(rintf(a1 / scf), -8.0f), 7.0f);
            d[g * 64 + lane] = (uint8_t)(((int)r0 + 8) | (((int)r1 + 8) << 4));
            if (lane == 0) sc[g] = sb;
        }
    }
}

// inverse of k_convert_rows for verification: stored row -> fp32
template <int WT>
__global__ __launch_bounds__(256) void k_export_rows(const void *__restrict__ src, const void *__restrict__ scales,
                                                     float *__restrict__ dst, int K) {
    const size_t row = blockIdx.x;
    for (int k = threadIdx.x; k < K; k += 256) {
        float v;
        if (WT == WT_F32) v = ((const float *)src)[row * K + k];
        else if (WT == WT_BF16) v = bf16_to_f32(((const uint16_t *)src)[row * K + k]);
        else if (WT == WT_FP8) {
            uint32_t b = ((const uint8_t *)src)[row * K + k];
            auto p = __builtin_amdgcn_cvt_pk_f32_fp8(b, false);
            v = p[0] * ((const float *)scales)[row];
        } else {
            uint32_t b = ((const uint8_t *)src)[row * (K / 2) + k / 2];
            int nib = (k & 1) ? (b >> 4) : (b & 0xf);
            v = (float)(nib - 8) * bf16_to_f32(((const uint16_t *)scales)[row * (K / 128) + k / 128]);
        }
        dst[row * K + k] = v;
    }
}

// transposes a channel-first fp32 cache [kv_dim][seq] into the row-major device cache
// [seq][kv_dim] (crates/metal-decode/src/lib.rs:228-234); rows >= live_len become zero
template <int KVBF16>
__global__ void k_seed_cache(const float *__restrict__ cf, void *__restrict__ cache, int KV, int S, int live) {
    __shared__ float t[32][33];
    int bx = blockIdx.x * 32, by = blockIdx.y * 32;    // bx over pos, by over channel
    for (int j = threadIdx.y; j < 32; j += 8) {
        int d = by + j, p = bx + threadIdx.x;
        if (d < KV && p < S) t[j][threadIdx.x] = cf[(size_t)d * S + p];
    }
    __syncthreads();
    for (int j = threadIdx.y; j < 32; j += 8) {
        int p = bx + j, d = by + threadIdx.x;
        if (d < KV && p < S) {
            float v = p < live ? t[threadIdx.x][j] : 0.0f;
            if (KVBF16) ((uint16_t *)cache)[(size_t)p * KV + d] = f32_to_bf16_rne(v);
            else ((float *)cache)[(size_t)p * KV + d] = v;
        }
    }
}
