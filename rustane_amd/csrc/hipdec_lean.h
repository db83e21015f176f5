// The one-launch-per-token step of hipdec_mega.h for models whose phases are short: bf16 weights and
// every reduction length a multiple of 512 (the 600M-class shapes).
//
// There a phase of k_mega is a few microseconds, and what bounds it is neither the memory stream nor
// the arithmetic but the number of instructions the busiest wave issues between the arrival of a
// phase's input and the publication of its output: about a thousand per phase in the general kernel
// (runtime segment / piece bookkeeping, bounds checks, cursor updates, 8 unpacks + 8 multiply-adds per
// 16-byte weight load), one instruction every four to five clocks.  This kernel keeps k_mega's
// structure -- one resident workgroup per CU, stamped exchanges, two weight register sets requested a
// phase ahead, the same attention, fold and head code -- and rebuilds the matrix-vector phases so that
// the instruction count per phase is a few hundred:
//
//  * the unit of work is (row pair, chunk of 64 pieces = 512 reduction elements): one 16-byte load per
//    lane and row, no partial units, so no lane ever checks a bound;
//  * register slots are assigned at compile time (the chunks per row of the even phases are a template
//    constant), a load is `base + immediate`, and nothing walks a cursor per load;
//  * the products run on the matrix cores straight from the loaded registers (lean_tile_diag below): one instruction per weight register and input plane.
//
// Everything else (exchange protocol, epochs, abort flag, LDS layout, host-side sizing) is k_mega's, and
// the two kernels are interchangeable launch for launch.
#pragma once
#include "hipdec_mega.h"

// ---- bf16 weights on the matrix cores
// v_mfma_f32_16x16x32_bf16 takes from lane l eight bf16 numbers of row l % 16 of A and of column l % 16
// of B, reduction elements 8 (l / 16) ... + 8.  A weight load gives lane l the eight elements of piece l of
// a row chunk, and the staged vector read the same way gives lane l the inputs of piece l: used as they
// are, element (m, n) of the 16 x 16 result is the sum over g of <weights of piece 16 g + m, inputs of
// piece 16 g + n>, so the DIAGONAL holds 16 partial dot products whose sum is the dot product over the
// chunk's 64 pieces.  The input vector is staged as two bf16 planes (hi = rne(v), lo = rne(v - hi): 16
// mantissa bits) and each weight register multiplies both.  Lane 20 g + v (g, v < 4) holds diagonal
// element 4 g + v in component v of its result registers.
typedef __bf16 lean_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 lean_bf16x2 __attribute__((ext_vector_type(2)));
typedef float lean_f32x2 __attribute__((ext_vector_type(2)));
typedef float lean_f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint32_t lean_pack_bf16(float a, float b) {
    const lean_f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, lean_bf16x2));
}
// LEAN_PLANES bf16 planes of a staged vector: plane 0 = rne(v), plane 1 = rne(v - p0), plane 2 = rne(v - p0 - p1).
// Two planes carry 16 mantissa bits of every input (an error of 2^-17 per product); with three the inputs are
// exact to fp32's 24 bits, and the products, which the matrix cores add up in fp32, are what the fp32 vector path
// computes up to the order of summation.  Two planes kept every logit within 1e-4 of the oracle but not every
// greedy stream: with a bf16 cache, differences of 1e-5 flip a cached value's rounding now and then, and the
// 600M golden stream left the oracle's at its closest call (top-2 gap 2e-4 of the largest logit).
#ifndef LEAN_PLANES
#define LEAN_PLANES 3
#endif
// Planes each kind of product multiplies (the staged vectors always hold LEAN_PLANES).  A plane costs the matrix
// pipeline a third more time per weight register, so the third plane is spent where 2^-17 matters: the q/k/v
// products, whose outputs are rounded into the cache (one differently rounded cached value is a 2^-8 step that
// every later token attends over), and the LM head, whose outputs are compared.  Measured on the 600M golden
// streams (256 greedy tokens against the CPU oracle, fp32 and bf16 cache, both prefill paths), ms per token:
// two planes everywhere 0.473 and one stream leaves the oracle's at token 91; q/k/v and head with three 0.478,
// all streams identical; three everywhere 0.485, identical (the general kernel: 0.495).
#ifndef LEAN_PL_QKV
#define LEAN_PL_QKV LEAN_PLANES
#endif
#ifndef LEAN_PL_HEAD
#define LEAN_PL_HEAD LEAN_PLANES
#endif
#ifndef LEAN_PL_W13
#define LEAN_PL_W13 2
#endif
#ifndef LEAN_PL_WO
#define LEAN_PL_WO 2
#endif
#ifndef LEAN_PL_W2
#define LEAN_PL_W2 2
#endif
// four values: elements 4 i ... 4 i + 3 of the planes of an n-element vector at `planes`
__device__ __forceinline__ void lean_store_pair4(float *planes, int n, int i, float a, float b, float c, float d) {
    const uint32_t h0 = lean_pack_bf16(a, b), h1 = lean_pack_bf16(c, d);
    const float ra = a - __uint_as_float(h0 << 16), rb = b - __uint_as_float(h0 & 0xffff0000u);
    const float rc = c - __uint_as_float(h1 << 16), rd = d - __uint_as_float(h1 & 0xffff0000u);
    const uint32_t l0 = lean_pack_bf16(ra, rb), l1 = lean_pack_bf16(rc, rd);
    uint32_t *hp = (uint32_t *)planes + 2 * i, *lp = hp + (n >> 1);
    *(uint2 *)hp = make_uint2(h0, h1);
    *(uint2 *)lp = make_uint2(l0, l1);
    if (LEAN_PLANES == 3) {
        const uint32_t m0 = lean_pack_bf16(ra - __uint_as_float(l0 << 16), rb - __uint_as_float(l0 & 0xffff0000u));
        const uint32_t m1 = lean_pack_bf16(rc - __uint_as_float(l1 << 16), rd - __uint_as_float(l1 & 0xffff0000u));
        *(uint2 *)(lp + (n >> 1)) = make_uint2(m0, m1);
    }
}
__device__ __forceinline__ void lean_store_pair1(float *planes, int n, int i, float a) {
    const uint16_t h = f32_to_bf16_rne(a);
    const float r = a - bf16_to_f32(h);
    const uint16_t l = f32_to_bf16_rne(r);
    ((uint16_t *)planes)[i] = h;
    ((uint16_t *)planes)[n + i] = l;
    if (LEAN_PLANES == 3) ((uint16_t *)planes)[2 * n + i] = f32_to_bf16_rne(r - bf16_to_f32(l));
}
// this lane's share of the trace of a result tile (zero off the diagonal); the wave's sum of it is the dot product
__device__ __forceinline__ float lean_tile_diag(const lean_f32x4 &c, int dsel) {
    float r = 0.0f;
    r = dsel == 0 ? c.x : r;
    r = dsel == 1 ? c.y : r;
    r = dsel == 2 ? c.z : r;
    r = dsel == 3 ? c.w : r;
    return r;
}
__device__ __forceinline__ lean_f32x4 lean_mma(const uint4 &w, const uint4 &x, const lean_f32x4 &c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lean_bf16x8, w), __builtin_bit_cast(lean_bf16x8, x), c, 0, 0, 0);
}

// mega_poll_vec for the pair layout: polls n stamped floats into the two planes at dst (see there)
template <bool GAMMA>
__device__ __noinline__ float lean_poll_vec(const float *src, int n, unsigned par, unsigned *abortf, float *dst,
                                            const float *gamma, float *res, int r0, int nres, int pt) {
    constexpr int NB = 2048 / MEGA_PT;
    const int n4 = n >> 2;
    const __amdgpu_buffer_rsrc_t r = make_rsrc(src, n * 4);
    const unsigned pm = par ? 0xffffffffu : 0u;
    float ss = 0.0f;
    bool good = true;
    for (int base = 0; base < n4 && good; base += MEGA_PT * NB) {
        mega_u4 v[NB], g[GAMMA ? NB : 1];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int i = base + b * MEGA_PT + pt;
            g[GAMMA ? b : 0] = mega_u4{0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u};
            if (GAMMA && gamma && i < n4) g[GAMMA ? b : 0] = *(const __attribute__((address_space(1))) mega_u4 *)(gamma + 4 * i);
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int i = base + b * MEGA_PT + pt;
            if (i < n4) v[b] = ld16_coherent(r, i * 16);
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int i = base + b * MEGA_PT + pt;
            if (i < n4 && good) {
                good = repoll16(v[b], r, i * 16, pm, abortf);
                const float x0 = __uint_as_float(v[b].x & ~1u), x1 = __uint_as_float(v[b].y & ~1u), x2 = __uint_as_float(v[b].z & ~1u),
                            x3 = __uint_as_float(v[b].w & ~1u);
                const mega_u4 gb = g[GAMMA ? b : 0];
                lean_store_pair4(dst, n, i, x0 * __uint_as_float(gb.x), x1 * __uint_as_float(gb.y), x2 * __uint_as_float(gb.z),
                                 x3 * __uint_as_float(gb.w));
                ss += x0 * x0 + x1 * x1 + x2 * x2 + x3 * x3;
                const float xe[4] = {x0, x1, x2, x3};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int j = 4 * i + e - r0;
                    if (j >= 0 && j < nres) res[j] = xe[e];
                }
            }
        }
    }
    return good ? ss : -1.0f;
}

#define LEAN_SLOTS_A 16         // 16-byte weight registers per lane of the even phases' set
#define LEAN_ITEMS_B 4          // (row pair, chunk) items per wave of the odd phases' set: 8 registers

struct LeanKind { int K, cpr, pair0, npl, nitems; size_t rb; };

// CE: 512-element chunks of a row of the even phases (dim / 512)
template <int CE, int KVBF16, int HD, int VAR>
__global__ __launch_bounds__(MEGA_THREADS, 1) void k_lean(MegaArgs a) {
    constexpr int PR = LEAN_SLOTS_A / (2 * CE) > 4 ? 4 : LEAN_SLOTS_A / (2 * CE) > 0 ? LEAN_SLOTS_A / (2 * CE) : 1;   // row pairs per round of an even phase
    static_assert(2 * CE * PR <= LEAN_SLOTS_A, "a round of the even phases fits the register set");
    constexpr int KESZ = KVBF16 ? 2 : 4;
    constexpr int KEPL = 16 / KESZ;
    constexpr int LPR = HD / KEPL;               // lanes per cache row
    constexpr int SLOTS = MEGA_THREADS / LPR;    // cache rows per pass
    constexpr int PRE = MEGA_ATT_PRE;            // passes prefetched
    constexpr int REC = HD + MEGA_PREC;          // floats per attention partial record
    extern __shared__ __align__(16) float smem[];
    __shared__ LeanKind kinds[MK_KINDS];
    __shared__ float s_red[2][MEGA_WAVES];
    __shared__ float s_cand_v[MEGA_WAVES];
    __shared__ uint32_t s_cand_i[MEGA_WAVES];
    __shared__ int s_bad;

    int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (tid == 0) s_bad = 0;
    const int G = gridDim.x, b = blockIdx.x;
    const int D = a.D, Q = a.Q, KV = a.KV, H = a.H, V = a.V, L = a.L;
    float *xsb = smem;                                       // LEAN_PLANES bf16 planes of D elements, then as many of max(Q, H)
    constexpr int XF = LEAN_PLANES;                          // half-floats of LDS per staged element
    float *stage = xsb + ((D + max(Q, H)) * XF) / 2;
    const int stage_floats = a.stage_floats;
    const int xres_n = 2 * ((D / 2 + G - 1) / G) + 2;
    float *xresb = stage + stage_floats;
    float *ropes = xresb + 2 * xres_n;
    const void **lptr = (const void **)(ropes + 2 * (((Q + 2 * KV) / 2 + G - 1) / G) + 2);
    for (int i = threadIdx.x; i < MEGA_LPTR * L; i += MEGA_THREADS) {
        const int l = i / MEGA_LPTR, j = i - l * MEGA_LPTR;
        const MegaLayer &ml = a.layers[l];
        lptr[i] = j < 4 ? ml.w[j] : j < 8 ? ml.sc[j - 4] : j == 8 ? (const void *)ml.g1 : j == 9 ? (const void *)ml.g2
                                                         : j == 10 ? (const void *)ml.kc : (const void *)ml.vc;
    }
    if (tid < MK_KINDS) {
        int rows, K;
        switch (tid) {
            case MK_QKV: rows = Q + 2 * KV; K = D; break;
            case MK_WO: rows = D; K = Q; break;
            case MK_W13: rows = 2 * H; K = D; break;
            case MK_W2: rows = D; K = H; break;
            default: rows = V; K = D; break;
        }
        const int npairs = rows >> 1, base = npairs / G, rem = npairs % G;
        LeanKind &k = kinds[tid];
        k.K = K;
        k.cpr = K / 512;
        k.pair0 = b * base + min(b, rem);
        k.npl = base + (b < rem ? 1 : 0);
        k.nitems = k.npl * k.cpr;
        k.rb = (size_t)K * 2;
    }
    const int pos = a.sp->pos, tok = a.sp->tok, use_x_in = a.sp->use_x_in;
    const unsigned ep_layer = a.epochs[0], ep_head = a.epochs[1];
    unsigned *abortf = a.abort;
    __syncthreads();

    if (wave == 0) {
        const LeanKind &k = kinds[MK_QKV];
        for (int p = lane; p < k.npl; p += 64) {
            const int row0 = 2 * (k.pair0 + p);
            const int rr = row0 < Q ? row0 : row0 - Q;
            const int pi2 = (rr % HD) >> 1;
            ropes[2 * p] = a.rope_cos[(size_t)pos * (HD / 2) + pi2];
            ropes[2 * p + 1] = a.rope_sin[(size_t)pos * (HD / 2) + pi2];
        }
    }

    unsigned long long *const prof = (VAR != MEGA_VAR_PLAIN && a.prof && b == a.prof_wg && tid == 0) ? a.prof : nullptr;
    int prof_n = 0;
    auto mark = [&]() { if (prof) prof[prof_n++] = wall_clock64(); };

    const int pt = tid;
    const int last_ph = a.do_head ? 4 * L : 4 * L - 1;
    const int dsel = ((lane & 15) >> 2) == (lane >> 4) ? (lane & 3) : -1;
    const int lane16 = lane * 16;

    // ---- the two weight register sets
    // Set A (even phases: qkv, w13, head): a round is PR row pairs of this wave (local pairs wave + 8 i), slot
    // (q * 2 + row) * CE + c holds chunk c of a row.  Set B (odd phases: wo, w2): the (pair, chunk) items of the
    // workgroup are dealt to the waves one by one (item t to wave t % 8), slot 2 i + row holds the wave's i-th item.
    uint4 wa[LEAN_SLOTS_A], wb[2 * LEAN_ITEMS_B];
#pragma unroll
    for (int i = 0; i < LEAN_SLOTS_A; ++i) wa[i] = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 2 * LEAN_ITEMS_B; ++i) wb[i] = make_uint4(0, 0, 0, 0);
    const char *eW = nullptr;                                // matrix of the even phase being requested
    int e_pair0 = 0, e_npl = 0, e_kind = MK_QKV;
    size_t e_rb = 0;
    // Byte offsets (this lane's 16 bytes included) of the first round's row requests of the two even kinds of a
    // layer and of the first round's items of the two odd kinds: the same in every layer, worked out once, so
    // that a request is a 64-bit add and a load.
    uint32_t qkv_off[2 * PR], w13_off[2 * PR], wo_off[LEAN_ITEMS_B], w2_off[LEAN_ITEMS_B];
    int wo_c[LEAN_ITEMS_B], w2_c[LEAN_ITEMS_B];              // chunk of each first-round item (selects the inputs it multiplies)
#pragma unroll
    for (int h = 0; h < 2 * PR; ++h) {
        const int pl = wave + MEGA_WAVES * (h >> 1);
        qkv_off[h] = (uint32_t)((2 * (kinds[MK_QKV].pair0 + pl) + (h & 1)) * (int)kinds[MK_QKV].rb + lane16);
        w13_off[h] = (uint32_t)((2 * (kinds[MK_W13].pair0 + pl) + (h & 1)) * (int)kinds[MK_W13].rb + lane16);
    }
#pragma unroll
    for (int i = 0; i < LEAN_ITEMS_B; ++i) {
        const int t = wave + MEGA_WAVES * i;
        const int p1 = t / kinds[MK_WO].cpr, p2 = t / kinds[MK_W2].cpr;
        wo_c[i] = t - p1 * kinds[MK_WO].cpr;
        w2_c[i] = t - p2 * kinds[MK_W2].cpr;
        wo_off[i] = (uint32_t)(2 * (kinds[MK_WO].pair0 + p1) * (int)kinds[MK_WO].rb + wo_c[i] * 1024 + lane16);
        w2_off[i] = (uint32_t)(2 * (kinds[MK_W2].pair0 + p2) * (int)kinds[MK_W2].rb + w2_c[i] * 1024 + lane16);
    }
    auto start_even = [&](int ph) {
        const int kind = ph == 4 * L ? MK_HEAD : (ph & 3);
        eW = kind == MK_HEAD ? (const char *)a.embed : (const char *)lptr[(ph >> 2) * MEGA_LPTR + kind];
        e_pair0 = kinds[kind].pair0; e_npl = kinds[kind].npl; e_rb = kinds[kind].rb; e_kind = kind;
    };
    // row `row` of pair q of round r of the even phase start_even named: CE loads
    auto issue_even_row = [&](const int r, const int q, const int row) {
        const int pl = wave + MEGA_WAVES * (r * PR + q);
        if (pl < e_npl) {
            const char *p0;
            if (r == 0 && e_kind != MK_HEAD) p0 = eW + (e_kind == MK_QKV ? qkv_off[q * 2 + row] : w13_off[q * 2 + row]);
            else p0 = eW + (size_t)(2 * (e_pair0 + pl) + row) * e_rb + lane16;
#pragma unroll
            for (int c = 0; c < CE; ++c) wa[(q * 2 + row) * CE + c] = ld_stream_u4(p0 + c * 1024);
        }
    };
    auto issue_even_pair = [&](const int r, const int q) { issue_even_row(r, q, 0); issue_even_row(r, q, 1); };
    // the h-th of the 2 PR row requests of a first round
    auto issue_even_part = [&](const int h) { issue_even_row(0, h >> 1, h & 1); };
    const char *oW = nullptr;
    int o_pair0 = 0, o_nitems = 0, o_cpr = 1;
    bool o_w2 = false;
    size_t o_rb = 0;
    auto start_odd = [&](int ph) {
        const LeanKind &k = kinds[ph & 3];
        oW = (const char *)lptr[(ph >> 2) * MEGA_LPTR + (ph & 3)];
        o_pair0 = k.pair0; o_nitems = k.nitems; o_cpr = k.cpr; o_rb = k.rb; o_w2 = (ph & 3) == MK_W2;
    };
    // the wave's item i of round r of the odd phase start_odd named: item t = wave + 8 (4 r + i) = (pair t / cpr, chunk t % cpr)
    auto issue_odd_item = [&](const int r, const int i) {
        const int t = wave + MEGA_WAVES * (r * LEAN_ITEMS_B + i);
        if (t < o_nitems) {
            const char *p0;
            if (r == 0) p0 = oW + (o_w2 ? w2_off[i] : wo_off[i]);
            else { const int p = t / o_cpr, c = t - p * o_cpr; p0 = oW + (size_t)(2 * (o_pair0 + p)) * o_rb + (size_t)c * 1024 + lane16; }
            wb[2 * i] = ld_stream_u4(p0);
            wb[2 * i + 1] = ld_stream_u4(p0 + o_rb);
        }
    };

    __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0): the set-up loads
    start_even(0);
#pragma unroll
    for (int q = 0; q < PR; ++q) issue_even_pair(0, q);
    if (1 <= last_ph) start_odd(1);

    const int wo_row0 = 2 * kinds[MK_WO].pair0, wo_rows = 2 * kinds[MK_WO].npl;   // same partition for w2

    const int n_att = pos + 1;
    int NS = (n_att + SLOTS * MEGA_ATT_SPLIT_PASSES - 1) / (SLOTS * MEGA_ATT_SPLIT_PASSES);
    NS = max(1, min(NS, a.ns_max));
    const int chunk = (n_att + NS - 1) / NS;
    const float att_scale = 1.0f / sqrtf((float)HD);
    const unsigned par_c = (ep_head + 1u) & 1u;

    for (int ph = 0; ph <= last_ph; ph += 2) {
        asm volatile("" : "+v"(tid), "+v"(lane));
        // ===================================================================== even phase: qkv, w13 or head
        {
        const int l = min(ph >> 2, L - 1);
        const int kind = ph == 4 * L ? MK_HEAD : (ph & 3);
        const unsigned par = (ep_layer + (unsigned)l + 1u) & 1u;
        const float *g1 = (const float *)lptr[l * MEGA_LPTR + 8], *g2 = (const float *)lptr[l * MEGA_LPTR + 9];
        void *kcl = (void *)lptr[l * MEGA_LPTR + 10], *vcl = (void *)lptr[l * MEGA_LPTR + 11];
        float *xs = xsb;
        float *xres_w = xresb + (kind == MK_W13 ? xres_n : 0);
        if (prof && kind != MK_W13) prof_n = (ph >> 2) * MEGA_PROF_SLOTS;
        mark();

        // ---- stage this phase's input vector in xs (two bf16 planes)
        float ss = 0.0f;
        bool ok = true;
        if (kind == MK_QKV && l == 0) {
            for (int i = tid; i < D; i += MEGA_THREADS) {
                float v;
                if (use_x_in) v = a.x_in[i];
                else v = bf16_to_f32(((const uint16_t *)a.embed)[(size_t)tok * D + i]);
                lean_store_pair1(xs, D, i, v * g1[i]);
                ss += v * v;
                if (i >= wo_row0 && i < wo_row0 + wo_rows) xres_w[i - wo_row0] = v;
            }
        } else {
            const float *src = kind == MK_W13 ? a.X2 : a.X;
            const float *gm = kind == MK_QKV ? g1 : kind == MK_W13 ? g2 : a.gfinal;
            const unsigned pr = kind == MK_QKV ? (par ^ 1u) : kind == MK_HEAD ? ((ep_layer + (unsigned)L) & 1u) : par;
            const int nres = kind == MK_HEAD ? 0 : wo_rows;
            ss = lean_poll_vec<true>(src, D, pr, abortf, xs, gm, xres_w, wo_row0, nres, pt);
            if (ss < 0.0f) { ok = false; ss = 0.0f; }
        }
        ss = wave_sum_dpp(ss);
        if (lane == 63) s_red[0][wave] = ss;
        if (!ok) s_bad = 1;
        lds_barrier();
        if (s_bad) return;
        mark();
        __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0): this phase's input and set A are here
        // the odd phase behind this one gets its (first) round now
        if (kind != MK_HEAD) {
#pragma unroll
            for (int i = 0; i < LEAN_ITEMS_B; ++i) issue_odd_item(0, i);
        }
        float inv;
        {
            float t = 0.0f;
#pragma unroll
            for (int w = 0; w < MEGA_WAVES; ++w) t += s_red[0][w];
            inv = 1.0f / sqrtf(t * (1.0f / (float)D) + 1e-5f);
        }

        // ---- this wave's row pairs, PR per round
        float bv = -INFINITY; uint32_t bi = 0x7fffffffu;
        {
            const LeanKind k = kinds[kind];
            const int nmy = k.npl > wave ? (k.npl - wave + MEGA_WAVES - 1) / MEGA_WAVES : 0;
            const char *xh = (const char *)xs + lane16;
            auto even_round = [&](const int r) {
                lean_f32x4 T[PR][2];
#pragma unroll
                for (int q = 0; q < PR; ++q) { T[q][0] = lean_f32x4{0.0f, 0.0f, 0.0f, 0.0f}; T[q][1] = T[q][0]; }
#pragma unroll
                for (int c = 0; c < CE; ++c) {
#pragma unroll
                    for (int pl = 0; pl < LEAN_PLANES; ++pl) {
                        if (pl >= (kind == MK_QKV ? LEAN_PL_QKV : kind == MK_W13 ? LEAN_PL_W13 : LEAN_PL_HEAD)) break;
                        const uint4 bx = *(const uint4 *)(xh + pl * 2 * D + c * 1024);
#pragma unroll
                        for (int q = 0; q < PR; ++q) {
                            // (a pair this wave does not have multiplies stale registers into a tile nobody reads)
                            T[q][0] = lean_mma(wa[(q * 2 + 0) * CE + c], bx, T[q][0]);
                            T[q][1] = lean_mma(wa[(q * 2 + 1) * CE + c], bx, T[q][1]);
                        }
                    }
                }
                if (r == 0) mark();
                if ((r + 1) * PR < nmy) {                     // inside a phase the next round follows into the same set
#pragma unroll
                    for (int q = 0; q < PR; ++q) issue_even_pair(r + 1, q);
                }
                float fin0 = 0.0f, fin1 = 0.0f;
                int n_fin = 0;
#pragma unroll
                for (int q = 0; q < PR; ++q) {
                    if (r * PR + q < nmy) {
                        const float t0 = wave_sum_dpp(lean_tile_diag(T[q][0], dsel)), t1 = wave_sum_dpp(lean_tile_diag(T[q][1], dsel));
                        const float b0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t0), 63));
                        const float b1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t1), 63));
                        if (lane == q) { fin0 = b0; fin1 = b1; }
                        ++n_fin;
                    }
                }
                if (lane < n_fin) {
                    float s0 = fin0, s1 = fin1;
                    const int p = wave + MEGA_WAVES * (r * PR + lane);
                    const int row0 = 2 * (k.pair0 + p);
                    if (kind == MK_QKV) {
                        s0 *= inv; s1 *= inv;
                        if (row0 < Q + KV) {
                            const float c = ropes[2 * p], s = ropes[2 * p + 1];
                            const float e = s0 * c - s1 * s, o = s1 * c + s0 * s;
                            s0 = e; s1 = o;
                        }
                        if (row0 >= Q) {
                            const bool isk = row0 < Q + KV;
                            const int rr = isk ? row0 - Q : row0 - Q - KV;
                            void *cache = isk ? kcl : vcl;
                            if (KVBF16) {
                                const uint16_t eb = f32_to_bf16_rne(s0), ob = f32_to_bf16_rne(s1);
                                uint16_t *cp = (uint16_t *)cache + (size_t)pos * KV + rr;
                                cp[0] = eb; cp[1] = ob;
                                s0 = bf16_to_f32(eb); s1 = bf16_to_f32(ob);
                            } else {
                                s0 = __uint_as_float(__float_as_uint(s0) & ~1u); s1 = __uint_as_float(__float_as_uint(s1) & ~1u);
                                float *cp = (float *)cache + (size_t)pos * KV + rr;
                                cp[0] = s0; cp[1] = s1;
                            }
                        }
                        st_stamped(a.QKV + row0, s0, par);
                        st_stamped(a.QKV + row0 + 1, s1, par);
                    } else if (kind == MK_W13) {
                        const float h1 = s0 * inv, h3 = s1 * inv;
                        float gte;
                        if (a.act == 1) { const float lr = h1 > 0.0f ? h1 : 0.5f * h1; gte = lr * lr * h3; }
                        else { const float sig = 1.0f / (1.0f + expf(-h1)); gte = h1 * sig * h3; }
                        st_stamped(a.GATE + (k.pair0 + p), gte, par);
                    } else {
                        s0 *= inv; s1 *= inv;
                        a.logits[row0] = s0; a.logits[row0 + 1] = s1;
                        if (better(s0, (uint32_t)row0, bv, bi)) { bv = s0; bi = (uint32_t)row0; }
                        if (better(s1, (uint32_t)row0 + 1, bv, bi)) { bv = s1; bi = (uint32_t)row0 + 1; }
                    }
                }
            };
            // The first round is taken outside the loop: there it is known that set A has arrived and that only
            // the odd phase's requests are outstanding (inside the loop a refilled set would have to be assumed,
            // and every use of a weight register would wait for all loads in flight).
            if (nmy > 0) even_round(0);
            for (int r = 1; r * PR < nmy; ++r) even_round(r);
        }
        mark();
        if (kind == MK_HEAD) {
            wave_argbest(bv, bi);
            if (lane == 0) { s_cand_v[wave] = bv; s_cand_i[wave] = bi; }
            lds_barrier();
            if (wave == 0) {
                float cv = lane < MEGA_WAVES ? s_cand_v[lane] : -INFINITY;
                uint32_t ci = lane < MEGA_WAVES ? s_cand_i[lane] : 0x7fffffffu;
                wave_argbest(cv, ci);
                if (lane == 0) {
                    unsigned long long c = (unsigned long long)__float_as_uint(cv) | ((unsigned long long)(ci | (par_c << 31)) << 32);
                    __hip_atomic_store(a.CAND + b, c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            mark();
            break;
        }
        mark();
        }

        // ===================================================================== odd phase: wo or w2
        {
        const int oph = ph + 1;
        const int l = oph >> 2;
        const int kind = oph & 3;
        const unsigned par = (ep_layer + (unsigned)l + 1u) & 1u;
        void *kcl = (void *)lptr[l * MEGA_LPTR + 10], *vcl = (void *)lptr[l * MEGA_LPTR + 11];
        float *xs = xsb + (D * XF) / 2;
        const float *xres_r = xresb + (kind == MK_W2 ? xres_n : 0);
        mark();

        // ---- attention (before the output projection): item (split, head) on workgroup b
        if (kind == MK_WO && b < a.heads * NS) {
            const int sidx = b / a.heads, h = b - sidx * a.heads, g = h / a.gqa;
            const int t0 = sidx * chunk, t1 = min(n_att, t0 + chunk);
            float *qs = stage + MEGA_WAVES * REC, *kcur = qs + HD, *vcur = kcur + HD;
            const int sub = tid % LPR, slot = tid / LPR;
            const char *kb = (const char *)kcl + ((size_t)g * HD + sub * KEPL) * KESZ;
            const char *vb = (const char *)vcl + ((size_t)g * HD + sub * KEPL) * KESZ;
            const size_t rowb = (size_t)KV * KESZ;
            uint4 kr[PRE], vr[PRE];
#pragma unroll
            for (int i = 0; i < PRE; ++i) { kr[i] = make_uint4(0, 0, 0, 0); vr[i] = make_uint4(0, 0, 0, 0); }
            // rows older than the new token are already in the cache: they are fetched before q arrives
#pragma unroll
            for (int i = 0; i < PRE; ++i) {
                const int t = t0 + slot + i * SLOTS;
                if (t < t1 && t != pos) { kr[i] = ldg_u4(kb + (size_t)t * rowb); vr[i] = ldg_u4(vb + (size_t)t * rowb); }
            }
            {
                bool ok = true;
                if (pt < 3 * (HD / 4)) {
                    const int which = pt / (HD / 4), i4 = pt - which * (HD / 4);
                    const float *src = a.QKV + (which == 0 ? h * HD : which == 1 ? Q + g * HD : Q + KV + g * HD);
                    float *dst = which == 0 ? qs : which == 1 ? kcur : vcur;
                    const float mul = which == 0 ? att_scale : 1.0f;
                    const __amdgpu_buffer_rsrc_t r = make_rsrc(src, HD * 4);
                    mega_u4 v = ld16_coherent(r, i4 * 16);
                    ok = repoll16(v, r, i4 * 16, par ? 0xffffffffu : 0u, abortf);
                    dst[4 * i4] = __uint_as_float(v.x & ~1u) * mul; dst[4 * i4 + 1] = __uint_as_float(v.y & ~1u) * mul;
                    dst[4 * i4 + 2] = __uint_as_float(v.z & ~1u) * mul; dst[4 * i4 + 3] = __uint_as_float(v.w & ~1u) * mul;
                }
                if (!ok) s_bad = 1;
                lds_barrier();
                if (s_bad) return;
            }
            mark();
            float qv[KEPL];
#pragma unroll
            for (int e = 0; e < KEPL; ++e) qv[e] = qs[sub * KEPL + e];
            float m = -1e30f, lsum = 0.0f, acc[KEPL];
#pragma unroll
            for (int e = 0; e < KEPL; ++e) acc[e] = 0.0f;
            for (int tb = t0; tb < t1; tb += SLOTS * PRE) {
                if (tb != t0) {
#pragma unroll
                    for (int i = 0; i < PRE; ++i) {
                        const int t = tb + slot + i * SLOTS;
                        if (t < t1 && t != pos) { kr[i] = ldg_u4(kb + (size_t)t * rowb); vr[i] = ldg_u4(vb + (size_t)t * rowb); }
                    }
                }
                float d[PRE];
#pragma unroll
                for (int i = 0; i < PRE; ++i) {
                    const int t = tb + slot + i * SLOTS;
                    float kf[KEPL];
                    if (t == pos) {
#pragma unroll
                        for (int e = 0; e < KEPL; ++e) kf[e] = kcur[sub * KEPL + e];
                    } else {
                        WS<KVBF16 ? WT_BF16 : WT_F32>::decode(kr[i], kf);
                    }
                    float dd = 0.0f;
#pragma unroll
                    for (int e = 0; e < KEPL; ++e) dd = fmaf(qv[e], kf[e], dd);
                    d[i] = dd;
                }
#pragma unroll
                for (int i = 0; i < PRE; ++i) d[i] = group_sum_dpp<LPR>(d[i]);
                float mn = m;
#pragma unroll
                for (int i = 0; i < PRE; ++i)
                    if (tb + slot + i * SLOTS < t1) mn = fmaxf(mn, d[i]);
                const float corr = __expf(m - mn);
                lsum *= corr;
#pragma unroll
                for (int e = 0; e < KEPL; ++e) acc[e] *= corr;
                m = mn;
#pragma unroll
                for (int i = 0; i < PRE; ++i) {
                    const int t = tb + slot + i * SLOTS;
                    if (t < t1) {
                        float vf[KEPL];
                        if (t == pos) {
#pragma unroll
                            for (int e = 0; e < KEPL; ++e) vf[e] = vcur[sub * KEPL + e];
                        } else {
                            WS<KVBF16 ? WT_BF16 : WT_F32>::decode(vr[i], vf);
                        }
                        const float p = __expf(d[i] - mn);
                        lsum += p;
#pragma unroll
                        for (int e = 0; e < KEPL; ++e) acc[e] = fmaf(p, vf[e], acc[e]);
                    }
                }
            }
#pragma unroll
            for (int o = LPR; o < 64; o <<= 1) {
                const float m2 = __shfl_xor(m, o, WAVE), l2 = __shfl_xor(lsum, o, WAVE);
                const float mn = fmaxf(m, m2);
                const float e1 = __expf(m - mn), e2 = __expf(m2 - mn);
                lsum = lsum * e1 + l2 * e2;
#pragma unroll
                for (int e = 0; e < KEPL; ++e) acc[e] = acc[e] * e1 + __shfl_xor(acc[e], o, WAVE) * e2;
                m = mn;
            }
            if (lane < LPR) {
#pragma unroll
                for (int e = 0; e < KEPL; ++e) stage[wave * REC + lane * KEPL + e] = acc[e];
                if (lane == 0) { stage[wave * REC + HD] = m; stage[wave * REC + HD + 1] = lsum; }
            }
            lds_barrier();
            if (tid < HD) {
                float M = -1e30f;
#pragma unroll
                for (int k2 = 0; k2 < MEGA_WAVES; ++k2) M = fmaxf(M, stage[k2 * REC + HD]);
                float Ls = 0.0f, A = 0.0f;
#pragma unroll
                for (int k2 = 0; k2 < MEGA_WAVES; ++k2) {
                    const float w = __expf(stage[k2 * REC + HD] - M);
                    Ls += stage[k2 * REC + HD + 1] * w;
                    A += stage[k2 * REC + tid] * w;
                }
                float *pp = a.PART + ((size_t)sidx * a.heads + h) * REC;
                st_stamped(pp + tid, A, par);
                if (tid < MEGA_PREC) st_stamped(pp + HD + tid, tid == 0 ? M : tid == 1 ? Ls : 0.0f, par);
            }
            lds_barrier();
            mark();
        } else if (kind == MK_WO && b < a.heads * a.ns_max) {
            if (tid < REC) {
                float *pp = a.PART + (size_t)b * REC;
                st_stamped(pp + tid, tid == HD ? -1e30f : 0.0f, par);
            }
        }

        // ---- stage this phase's input: the folded attention partials (wo) or the gate vector (w2)
        // Set A is free since the even phase's last round: the next even phase's first pair goes out here, behind
        // the attention, in front of the wait for the partials -- not in front of the gate poll, whose phase is
        // short (the poll would come back behind these loads).
        if (oph + 1 <= last_ph) start_even(oph + 1);
        const bool more_even = oph + 1 <= last_ph;
        const bool early = kind == MK_WO;
        // A first round is 2 PR row requests.  In front of the wait for the attention partials: the first half of
        // them; behind the staging barrier: all but the last of the rest; behind the publication: the last.
        constexpr int NPART = 2 * PR, NEARLY = NPART / 2;
        if (early && more_even) {
#pragma unroll
            for (int h = 0; h < NEARLY; ++h) issue_even_part(h);
        }
        {
            bool ok = true;
            if (kind == MK_WO) {
                const unsigned pm = par ? 0xffffffffu : 0u;
                const __amdgpu_buffer_rsrc_t r = make_rsrc(a.PART, NS * a.heads * REC * 4);
                for (int c = tid; c < Q / 4 && ok; c += MEGA_THREADS) {
                    const int h = (4 * c) / HD, j = 4 * c - h * HD;
                    float M = -1e30f, Ls = 0.0f, o0 = 0.0f, o1 = 0.0f, o2 = 0.0f, o3 = 0.0f;
                    for (int s0 = 0; s0 < NS && ok; s0 += 4) {
                        mega_u4 va[4], vt[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int off = ((min(s0 + q, NS - 1) * a.heads + h) * REC) * 4;
                            va[q] = ld16_coherent(r, off + j * 4);
                            vt[q] = ld16_coherent(r, off + HD * 4);
                        }
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            if (s0 + q < NS && ok) {
                                const int off = (((s0 + q) * a.heads + h) * REC) * 4;
                                ok = repoll16(va[q], r, off + j * 4, pm, abortf) && repoll16(vt[q], r, off + HD * 4, pm, abortf);
                                const float ms = __uint_as_float(vt[q].x & ~1u), ls = __uint_as_float(vt[q].y & ~1u);
                                const float mn = fmaxf(M, ms);
                                const float e1 = __expf(M - mn), e2 = __expf(ms - mn);
                                Ls = Ls * e1 + ls * e2;
                                o0 = o0 * e1 + __uint_as_float(va[q].x & ~1u) * e2;
                                o1 = o1 * e1 + __uint_as_float(va[q].y & ~1u) * e2;
                                o2 = o2 * e1 + __uint_as_float(va[q].z & ~1u) * e2;
                                o3 = o3 * e1 + __uint_as_float(va[q].w & ~1u) * e2;
                                M = mn;
                            }
                        }
                    }
                    const float rl = Ls > 0.0f ? 1.0f / Ls : 0.0f;
                    lean_store_pair4(xs, Q, c, o0 * rl, o1 * rl, o2 * rl, o3 * rl);
                }
            } else {
                const float ss = lean_poll_vec<false>(a.GATE, H, par, abortf, xs, nullptr, xresb, wo_row0, 0, pt);
                if (ss < 0.0f) ok = false;
            }
            if (!ok) s_bad = 1;
            lds_barrier();
            if (s_bad) return;
        }
        mark();
        __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0): this phase's input and set B are here
        if (more_even) {
#pragma unroll
            for (int h = 0; h < NPART - 1; ++h)
                if (h >= NEARLY || !early) issue_even_part(h);     // (h stays a compile-time constant: the set is a register array)
        }

        // ---- this wave's items, LEAN_ITEMS_B per round; each item's two sums go to LDS
        {
            const LeanKind k = kinds[kind];
            const int nmy = k.nitems > wave ? (k.nitems - wave + MEGA_WAVES - 1) / MEGA_WAVES : 0;
            const char *xh = (const char *)xs + lane16;
            auto odd_round = [&](const int r) {
                float acc[LEAN_ITEMS_B][2];
#pragma unroll
                for (int i = 0; i < LEAN_ITEMS_B; ++i) {
                    acc[i][0] = 0.0f; acc[i][1] = 0.0f;
                    const int t = wave + MEGA_WAVES * (r * LEAN_ITEMS_B + i);
                    if (t < k.nitems) {
                        const int c = r == 0 ? (kind == MK_W2 ? w2_c[i] : wo_c[i]) : t % k.cpr;
                        lean_f32x4 c0 = {0.0f, 0.0f, 0.0f, 0.0f}, c1 = c0;
#pragma unroll
                        for (int pl = 0; pl < LEAN_PLANES; ++pl) {
                            if (pl >= (kind == MK_WO ? LEAN_PL_WO : LEAN_PL_W2)) break;
                            const uint4 bx = *(const uint4 *)(xh + pl * 2 * k.K + c * 1024);
                            c0 = lean_mma(wb[2 * i], bx, c0);
                            c1 = lean_mma(wb[2 * i + 1], bx, c1);
                        }
                        acc[i][0] = lean_tile_diag(c0, dsel); acc[i][1] = lean_tile_diag(c1, dsel);
                    }
                }
                if (r == 0) mark();
                if ((r + 1) * LEAN_ITEMS_B < nmy) {
#pragma unroll
                    for (int i = 0; i < LEAN_ITEMS_B; ++i) issue_odd_item(r + 1, i);
                }
#pragma unroll
                for (int i = 0; i < LEAN_ITEMS_B; ++i) {
                    const int t = wave + MEGA_WAVES * (r * LEAN_ITEMS_B + i);
                    if (t < k.nitems) {
                        const float s0 = wave_sum_dpp(acc[i][0]), s1 = wave_sum_dpp(acc[i][1]);
                        if (lane == 63) { stage[2 * t] = s0; stage[2 * t + 1] = s1; }
                    }
                }
            };
            if (nmy > 0) odd_round(0);                       // (first round outside the loop, as in the even phase)
            for (int r = 1; r * LEAN_ITEMS_B < nmy; ++r) odd_round(r);
            lds_barrier();
            // thread r finishes local row r: the chunks of its pair in order, residual, publish
            if (tid < 2 * k.npl) {
                const int p = tid >> 1, which = tid & 1;
                float sum = 0.0f;
                for (int c = 0; c < k.cpr; ++c) sum += stage[2 * (p * k.cpr + c) + which];
                const int row = 2 * k.pair0 + tid;
                float *dstv = kind == MK_WO ? a.X2 : a.X;
                st_stamped(dstv + row, xres_r[tid] + a.alpha * sum, par);
            }
        }
        // the rest of the next even phase's first round, and the next odd phase's matrix
        if (more_even) issue_even_part(NPART - 1);
        if (oph + 2 <= last_ph) start_odd(oph + 2);
        mark();
        mark();
        }
    }

    if (!a.do_head) {
        if (b == 0 && tid == 0) {
            if (a.advance) a.sp->pos = pos + 1;
            a.epochs[0] = ep_layer + (unsigned)L;
        }
        return;
    }
    // ================= workgroup 0 folds the per-workgroup argmax candidates and advances the step state
    if (b == 0 && wave == 0) {
        float fv = -INFINITY; uint32_t fi = 0x7fffffffu;
        bool ok = true;
        for (int i = lane; i < G && ok; i += 64) {
            unsigned spins = 0;
            unsigned long long c;
            for (;;) {
                c = __hip_atomic_load(a.CAND + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((((unsigned)(c >> 63)) ^ par_c) == 0) break;
                if ((++spins & g_spin_ctl[0]) == 0) {
                    if (ld_abort(abortf)) { ok = false; break; }
                    if (spins > g_spin_ctl[1]) { raise_abort(abortf); ok = false; break; }
                }
            }
            if (ok) {
                const float v = __uint_as_float((unsigned)c);
                const uint32_t ix = (uint32_t)(c >> 32) & 0x7fffffffu;
                if (better(v, ix, fv, fi)) { fv = v; fi = ix; }
            }
        }
        wave_argbest(fv, fi);
        const int bad = __any(!ok);
        if (lane == 0 && !bad) {
            const int stp = a.sp->step;
            if (stp >= 0 && stp < a.ring_cap) a.ring[stp] = fi;
            a.sp->tok = (int)fi;
            a.sp->pos = pos + 1;
            a.sp->step = stp + 1;
            a.epochs[0] = ep_layer + (unsigned)L;
            a.epochs[1] = ep_head + 1u;
        }
        mark();
    }
}
