// The layers of a multi-sample decode step in ONE launch for gfx950: the persistent-kernel scheme of
// hipdec_mega.h (one 512-thread workgroup resident per CU, phases separated by exchanges of stamped
// values through device memory, the next phase's weights requested while the current one runs) for
// R <= 8 rows that advance together (hipdec_batch.h).  What differs from the single-row kernel:
//
//  * the products run on the matrix cores.  A workgroup owns a contiguous band of at most 32 (qkv,
//    w13) or 16 (wo, w2) weight rows; a tile is 16 weight rows, v_mfma_f32_16x16x32_bf16 takes a
//    lane's 16-byte weight load as its A operand as loaded (lane l: row l % 16, reduction elements
//    8 * (l / 16) .. + 8 of a 32-element step), and the R activation rows are the B operand, read
//    from LDS as (hi, lo) bf16 pairs: columns 0..7 of the operand tile are the rows' hi parts,
//    columns 8..15 their lo parts, so ONE instruction per weight load multiplies both (nothing is
//    rounded to 8 bits; the two halves of a result row are added in registers).  The eight waves
//    split the reduction axis; their 16 x 16 partial tiles meet in LDS;
//  * a phase's weights are ONE round of loads per wave (at most 12 or 16 loads of 16 bytes per lane,
//    which is what bounds the model sizes this kernel takes), requested in two halves, one and two
//    phases ahead, into the register set the running phase does not use;
//  * every exchanged vector crosses the fabric once per XCD: the workgroups that share an XCD each
//    copy a share of it into the XCD's own copy, and everybody polls that copy (rows_relay);
//  * a layer is two halves of the same shape that run through one copy of the code;
//  * the staged activation rows are single-buffered (R rows of up to 4096 elements as pairs fill the
//    LDS), so a phase has two workgroup barriers: inputs staged, partial tiles written;
//  * attention items are (split, row, head); a row's keys and values are the shared prompt prefix,
//    then the row's own suffix cache, then the new token from the exchange;
//  * the LM head and the draw stay outside (the streaming GEMM and the per-row head kernels): the
//    kernel ends by writing the last residual rows times the final norm's gains as the (hi, lo)
//    pair, and their chunk sums of squares, where that GEMM reads them.
//
// bf16 weights only.  Every weight load is a buffer load whose descriptor covers exactly the matrix
// (lanes and slots without work aim past it and read zeros), every wait is bounded as in
// hipdec_mega.h, and the arithmetic of a row does not depend on the other rows or on R.
#pragma once
#include "hipdec_batch.h"
#include "hipdec_mega.h"

#define ROWS_THREADS 512
#define ROWS_WAVES 8
#define ROWS_MAX_R 8
#define ROWS_TA 2               // 16-row tiles of an even phase (qkv, w13) per workgroup
#define ROWS_JA 6               // 32-element steps per wave and tile of an even phase: K = dim <= 8 * 32 * 6
#define ROWS_TB 1               // the same for the odd phases (wo, w2)
#define ROWS_JB 16              // K = q_dim or hidden <= 8 * 32 * 16
#define ROWS_XCD_COPIES 8       // per-XCD copies of the exchange vectors (a workgroup on an XCD numbered higher gives up)
#define ROWS_PAD 8              // bf16 elements between staged rows: the 16 lanes of an operand read hit 16 different bank groups
#define ROWS_LPTR 10            // per-layer pointers kept in LDS: w[4], g1, g2, kc, vc, kc_suf, vc_suf
#define ROWS_OOB 0x7ffffff0     // byte offset past every descriptor
#define ROWS_PROF_SLOTS 16      // time stamps per layer in the profiling build
#define ROWS_ATT_PRE 6          // attention: passes of cache rows a thread requests ahead (with R * heads items only a few
                                // splits are to be had, so an item walks more rows than in the single-row kernel)

enum { RK_QKV = 0, RK_WO = 1, RK_W13 = 2, RK_W2 = 3 };

struct RowsArgs {
    const MegaLayer *layers;             // the single-row kernel's table: weights (out-major bf16), gains, prefix caches
    void *const *kc_suf, *const *vc_suf; // [L] per-row suffix caches, [cap_rows][suf_rows][KV]
    const float *x_in;                   // [R][D] embedding rows of this step's tokens
    const float *gfinal, *rope_cos, *rope_sin;
    float *X, *X2, *QKV, *GATE, *PART;   // exchange buffers, R rows each, zeroed when a batch opens
    unsigned *XT;                        // [grid] exchange of the workgroups' XCD numbers
    float *XB;                           // [xb_copies][xb_stride] per-XCD copies of X, X2, GATE and the folded attention output (ordinary memory)
    int xb_copies, xb_stride, xb_x, xb_x2, xb_gate, xb_att;  // stride and offsets in floats
    uint16_t *out_hi, *out_lo;           // [R][D] last residual rows times the final gains, as pairs
    float *out_ssq;                      // [R][D / 256] their chunk sums of squares
    const BatchParams *bp;
    unsigned *epochs;                    // [0] exchange counter (advances by L per launch), [1] launch counter
    unsigned *abort;                     // abort flag (host memory mapped into the device)
    unsigned long long *prof;            // nullable: workgroup 0 writes ROWS_PROF_SLOTS wall-clock stamps per layer here
    int R, D, Q, KV, H, L, heads, gqa, act, ns_max;
    size_t suf_rows;
    float alpha;
};

struct RowsKind { int K, row0, nrows, pair0, npl, ntiles, spw; unsigned bytes; };

struct RowsLds { int xs, xh, xl, red, stage, xres, xres_n, ropes, ssq, lptr, total; };
__host__ __device__ inline RowsLds rows_lds(int R, int D, int Q, int KV, int H, int L, int hd, int G) {
    RowsLds o;
    const int kmax = D > Q ? (D > H ? D : H) : (Q > H ? Q : H);
    o.xs = kmax + ROWS_PAD;
    int off = 0;
    o.xh = off; off += R * o.xs * 2;
    o.xl = off; off += R * o.xs * 2;
    off = (off + 15) & ~15;
    o.red = off; off += ROWS_WAVES * ROWS_TA * 256 * 4;
    o.stage = off; off += (MEGA_WAVES * (hd + MEGA_PREC) + 3 * hd) * 4;
    o.xres_n = 2 * ((D / 2 + G - 1) / G);
    o.xres = off; off += 2 * R * o.xres_n * 4;
    o.ropes = off; off += 2 * (((Q + 2 * KV) / 2 + G - 1) / G) * 4;
    o.ssq = off; off += R * (D / 256) * 4;
    off = (off + 15) & ~15;
    o.lptr = off; off += L * ROWS_LPTR * 8;
    o.total = off;
    return o;
}

typedef __bf16 rows_bf16x8 __attribute__((ext_vector_type(8)));
typedef float rows_f32x4 __attribute__((ext_vector_type(4)));

// one 16-byte weight load: streamed (every byte is used once per step), zeros past the matrix
__device__ __forceinline__ mega_u4 rows_ldw(__amdgpu_buffer_rsrc_t r, int byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 2);
}

__device__ __forceinline__ unsigned rows_xcc_id() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xfu;
}

// Every workgroup reads every exchanged vector: with R rows 50 - 130 KB per workgroup and phase, all of it
// out of the few memory channels the vector lives in.  So a vector crosses the fabric once per XCD: member
// `rank` of the `members` workgroups that share an XCD polls its share of the n4 16-byte slots and stores
// them into the XCD's own copy in ordinary memory (plain stores: they land in that XCD's L2), and every
// workgroup then polls its XCD's copy (device-scope loads, which pass the CU's L1 and are served by that L2).
// plain: the source is ordinary memory an earlier kernel wrote.  The copy carries the stamp par_out whatever
// the source carried: every copy is written once per layer with that layer's stamp, so a copy's stamps
// alternate from write to write, also from one launch to the next, and cleared memory is never taken for a
// value of the first layer.
__device__ __forceinline__ bool rows_relay(const float *src, float *dst, int n4, int members, int rank, unsigned par,
                                           unsigned par_out, unsigned *abortf, bool plain) {
    const int per = (n4 + members - 1) / members, lo = rank * per, hi = min(n4, lo + per);
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(src, n4 * 16), rd = make_rsrc(dst, n4 * 16);
    const unsigned pm = par ? 0xffffffffu : 0u;
    bool ok = true;
    for (int i = lo + (int)threadIdx.x; i < hi && ok; i += ROWS_THREADS) {
        mega_u4 v = ld16_coherent(rs, i * 16);
        if (!plain) ok = repoll16(v, rs, i * 16, pm, abortf);
        v = mega_u4{(v.x & ~1u) | par_out, (v.y & ~1u) | par_out, (v.z & ~1u) | par_out, (v.w & ~1u) | par_out};
        if (ok) __builtin_amdgcn_raw_buffer_store_b128(v, rd, i * 16, 0, 0);
    }
    return ok;
}

// Stages R rows of n floats (n a multiple of 256) as (hi, lo) bf16 pairs: dst[r][i] = src[r][i] * gamma[i].
// The rows come from the XCD's copy of an exchanged vector (rows_relay): polled until every word carries
// the stamp `par`; stamp bit cleared.  A wave's 64 slots of one pass are one 256-element chunk of a row: with SSQ its sum of
// squares goes to ssq[r][chunk].
// Elements [r0, r0 + nres) of every row are also kept raw in res[r][.].  Returns a negative value when
// the wait was aborted.
template <bool GAMMA, bool SSQ>
__device__ __forceinline__ float rows_poll(const float *src, int R, int n, unsigned par, unsigned *abortf, uint16_t *xh,
                                        uint16_t *xl, int XS, const float *gamma, float *ssq, float *res, int r0, int nres,
                                        int res_stride) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int n4 = n >> 2, nch = n >> 8;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(src, R * n * 4);
    const unsigned pm = par ? 0xffffffffu : 0u;
    bool good = true;
    for (int i4 = tid; i4 < n4 && good; i4 += ROWS_THREADS) {
        mega_u4 g = mega_u4{0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u};
        if (GAMMA) g = *(const __attribute__((address_space(1))) mega_u4 *)(gamma + 4 * i4);
        mega_u4 v[ROWS_MAX_R];
#pragma unroll
        for (int r = 0; r < ROWS_MAX_R; ++r) {
            v[r] = mega_u4{0u, 0u, 0u, 0u};
            if (r < R) v[r] = ld16_coherent(rs, (r * n + 4 * i4) * 4);
        }
#pragma unroll
        for (int r = 0; r < ROWS_MAX_R; ++r) {
            if (r < R) {
                if (good) good = repoll16(v[r], rs, (r * n + 4 * i4) * 4, pm, abortf);
                const unsigned keep = ~1u;
                const float x0 = __uint_as_float(v[r].x & keep), x1 = __uint_as_float(v[r].y & keep),
                            x2 = __uint_as_float(v[r].z & keep), x3 = __uint_as_float(v[r].w & keep);
                uint32_t h0, l0, h1, l1;
                pf_split2(x0 * __uint_as_float(g.x), x1 * __uint_as_float(g.y), h0, l0);
                pf_split2(x2 * __uint_as_float(g.z), x3 * __uint_as_float(g.w), h1, l1);
                *(uint2 *)(xh + r * XS + 4 * i4) = make_uint2(h0, h1);
                *(uint2 *)(xl + r * XS + 4 * i4) = make_uint2(l0, l1);
                if (SSQ) {
                    const float ss = wave_sum_dpp((x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3));
                    if (lane == 63) ssq[r * nch + (i4 >> 6)] = ss;
                }
                const int j = 4 * i4 - r0;
                if (j + 3 >= 0 && j < nres) {
                    if (j >= 0 && j < nres) res[r * res_stride + j] = x0;
                    if (j + 1 >= 0 && j + 1 < nres) res[r * res_stride + j + 1] = x1;
                    if (j + 2 >= 0 && j + 2 < nres) res[r * res_stride + j + 2] = x2;
                    if (j + 3 >= 0 && j + 3 < nres) res[r * res_stride + j + 3] = x3;
                }
            }
        }
    }
    return good ? 0.0f : -1.0f;
}

// The input of the output projection, first half: the attention output of (row n, four neighbouring
// channels) is folded from every split's partial record, in split order, as the softmax over the whole
// sequence weighs them.  The R * Q / 4 items are shared out among the workgroups of an XCD like the slots
// of rows_relay (a thread takes one item, four splits in flight), and the folded values go, with the
// layer's stamp, into the XCD's copy `dst`[R][Q], from where every workgroup stages them with rows_poll.
// Records: PART[(split * R + n) * heads + h].
template <int HD>
__device__ __forceinline__ bool rows_fold_relay(const float *PART, float *dst, int NS, int R, int heads, int Q, int members,
                                                int rank, unsigned par, unsigned par_out, unsigned *abortf) {
    constexpr int REC = HD + MEGA_PREC;
    const unsigned pm = par ? 0xffffffffu : 0u;
    const int q4 = Q >> 2, n_items = R * q4;
    const int per = (n_items + members - 1) / members, lo = rank * per, hi = min(n_items, lo + per);
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(PART, NS * R * heads * REC * 4), rd = make_rsrc(dst, n_items * 16);
    bool ok = true;
    for (int it = lo + (int)threadIdx.x; it < hi && ok; it += ROWS_THREADS) {
        const int n = it / q4, cc = it - n * q4;
        const int h = (4 * cc) / HD, j = 4 * cc - h * HD;
        float M = -1e30f, Ls = 0.0f, o0 = 0.0f, o1 = 0.0f, o2 = 0.0f, o3 = 0.0f;
        for (int s0 = 0; s0 < NS && ok; s0 += 4) {
            mega_u4 va[4], vt[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int off = (((min(s0 + q, NS - 1) * R + n) * heads + h) * REC) * 4;
                va[q] = ld16_coherent(rs, off + j * 4);
                vt[q] = ld16_coherent(rs, off + HD * 4);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (s0 + q < NS && ok) {
                    const int off = ((((s0 + q) * R + n) * heads + h) * REC) * 4;
                    ok = repoll16(va[q], rs, off + j * 4, pm, abortf) && repoll16(vt[q], rs, off + HD * 4, pm, abortf);
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
        if (ok) {
            const float rl = Ls > 0.0f ? 1.0f / Ls : 0.0f;
            const mega_u4 v = {(__float_as_uint(o0 * rl) & ~1u) | par_out, (__float_as_uint(o1 * rl) & ~1u) | par_out,
                               (__float_as_uint(o2 * rl) & ~1u) | par_out, (__float_as_uint(o3 * rl) & ~1u) | par_out};
            __builtin_amdgcn_raw_buffer_store_b128(v, rd, it * 16, 0, 0);
        }
    }
    return ok;
}

// VAR: MEGA_VAR_PLAIN, or MEGA_VAR_STAMPS for the build that also takes time stamps (hipdec_debug_batch_step_profile).
template <int KVBF16, int HD, int VAR>
__global__ __launch_bounds__(ROWS_THREADS, 1) void k_rows(RowsArgs a) {
    constexpr int KESZ = KVBF16 ? 2 : 4;
    constexpr int KEPL = 16 / KESZ;
    constexpr int LPR = HD / KEPL;               // lanes per cache row
    constexpr int SLOTS = ROWS_THREADS / LPR;    // cache rows per pass
    constexpr int PRE = ROWS_ATT_PRE;
    constexpr int REC = HD + MEGA_PREC;
    extern __shared__ __align__(16) unsigned char rows_smem[];
    __shared__ RowsKind kinds[4];
    __shared__ int s_bad, s_grp[2];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, c4 = lane >> 4;
    if (tid == 0) s_bad = 0;
    const int G = gridDim.x, b = blockIdx.x;
    const int R = a.R, D = a.D, Q = a.Q, KV = a.KV, H = a.H, L = a.L, heads = a.heads;
    const int N = Q + 2 * KV;
    const RowsLds lo = rows_lds(R, D, Q, KV, H, L, HD, G);
    const int XS = lo.xs;
    uint16_t *const xh = (uint16_t *)(rows_smem + lo.xh), *const xl = (uint16_t *)(rows_smem + lo.xl);
    float *const red = (float *)(rows_smem + lo.red);
    float *const stage = (float *)(rows_smem + lo.stage);
    float *const xresb = (float *)(rows_smem + lo.xres);
    float *const ropes = (float *)(rows_smem + lo.ropes);
    float *const s_ssq = (float *)(rows_smem + lo.ssq);
    const void **const lptr = (const void **)(rows_smem + lo.lptr);
    const int xres_n = lo.xres_n, nchD = D >> 8;

    for (int i = tid; i < ROWS_LPTR * L; i += ROWS_THREADS) {
        const int l = i / ROWS_LPTR, j = i - l * ROWS_LPTR;
        const MegaLayer &ml = a.layers[l];
        lptr[i] = j < 4 ? ml.w[j] : j == 4 ? (const void *)ml.g1 : j == 5 ? (const void *)ml.g2 : j == 6 ? (const void *)ml.kc
                : j == 7 ? (const void *)ml.vc : j == 8 ? (const void *)a.kc_suf[l] : (const void *)a.vc_suf[l];
    }
    if (tid < 4) {
        int rows, K;
        switch (tid) {
            case RK_QKV: rows = N; K = D; break;
            case RK_WO: rows = D; K = Q; break;
            case RK_W13: rows = 2 * H; K = D; break;
            default: rows = D; K = H; break;
        }
        const int npairs = rows >> 1, base = npairs / G, rem = npairs % G;
        RowsKind &k = kinds[tid];
        k.K = K;
        k.pair0 = b * base + min(b, rem);
        k.npl = base + (b < rem ? 1 : 0);
        k.row0 = 2 * k.pair0;
        k.nrows = 2 * k.npl;
        k.ntiles = (k.nrows + 15) >> 4;
        k.spw = K >> 8;                          // 32-element steps per wave: K / 32 / 8
        k.bytes = (unsigned)rows * (unsigned)K * 2u;
    }
    const int pos = a.bp->pos, slot = a.bp->slot, prefix = a.bp->prefix;
    const unsigned ep = a.epochs[0], ep_launch = a.epochs[1];
    unsigned *abortf = a.abort;
    // Which workgroups share this one's XCD (and its L2): every workgroup publishes its XCD number, wave 0
    // reads all of them and counts the members of its own XCD and those among them with a smaller index.
    const unsigned myx = rows_xcc_id();
    const unsigned parT = (ep_launch + 1u) & 1u;             // the launch's parity: stamp of the XCD table
    if (wave == 0) {
        if (lane == 0) __hip_atomic_store(a.XT + b, ((myx + 1u) << 1) | parT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const __amdgpu_buffer_rsrc_t rt = make_rsrc(a.XT, G * 4);
        int cnt = 0, rank = 0;
        bool ok = true;
        for (int base = 0; base < G && ok; base += 256) {
            const int i = (base >> 2) + lane;
            const bool in = 4 * i < G;
            mega_u4 v = mega_u4{0u, 0u, 0u, 0u};
            if (in) { v = ld16_coherent(rt, i * 16); ok = repoll16(v, rt, i * 16, parT ? 0xffffffffu : 0u, abortf); }
            ok = !__any(!ok);
            const unsigned e4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool same = in && (e4[e] >> 1) == myx + 1u;
                cnt += __popcll(__ballot(same));
                rank += __popcll(__ballot(same && 4 * i + e < b));
            }
        }
        if (lane == 0) { s_grp[0] = cnt; s_grp[1] = rank; if (!ok || myx >= (unsigned)a.xb_copies) s_bad = 1; }
    }
    __syncthreads();
    if (s_bad) return;
    const int members = s_grp[0], rank = s_grp[1];
    float *const xb = a.XB + (size_t)myx * a.xb_stride;      // this XCD's copies
    float *const xbX = xb + a.xb_x, *const xbX2 = xb + a.xb_x2, *const xbG = xb + a.xb_gate, *const xbA = xb + a.xb_att;

    if (wave == 0) {
        const RowsKind &k = kinds[RK_QKV];
        for (int p = lane; p < k.npl; p += 64) {
            const int row0 = 2 * (k.pair0 + p);
            const int rr = row0 < Q ? row0 : row0 - Q;
            const int pi2 = (rr % HD) >> 1;
            ropes[2 * p] = a.rope_cos[(size_t)pos * (HD / 2) + pi2];
            ropes[2 * p + 1] = a.rope_sin[(size_t)pos * (HD / 2) + pi2];
        }
    }

    // ---- weight rounds.  Slot (t, j) of a set holds tile t, step wave * spw + j of the wave's share of
    // the reduction axis; lanes past the band's last row and slots past (ntiles, spw) read zeros.
    mega_u4 stA[ROWS_TA * ROWS_JA], stB[ROWS_TB * ROWS_JB];
    constexpr std::integral_constant<int, ROWS_TA> TA_C{};
    constexpr std::integral_constant<int, ROWS_JA> JA_C{};
    constexpr std::integral_constant<int, ROWS_TB> TB_C{};
    constexpr std::integral_constant<int, ROWS_JB> JB_C{};
    // (slots [S0, S1) of the set, in the order (tile, step): a set is requested in parts, each in front of a poll)
    auto issue_part = [&](auto &st, auto tt_c, auto jj_c, auto s0_c, auto s1_c, const int kind, const int l) {
        constexpr int TT = decltype(tt_c)::value, JJ = decltype(jj_c)::value, S0 = decltype(s0_c)::value, S1 = decltype(s1_c)::value;
        const int K = __builtin_amdgcn_readfirstlane(kinds[kind].K), spw = __builtin_amdgcn_readfirstlane(kinds[kind].spw);
        const int nrows = __builtin_amdgcn_readfirstlane(kinds[kind].nrows), row0 = __builtin_amdgcn_readfirstlane(kinds[kind].row0);
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(lptr[l * ROWS_LPTR + kind], (int)kinds[kind].bytes);
        const int lane_off = (row0 + r16) * (K * 2) + (wave * spw * 4 + c4) * 16;
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int j = 0; j < JJ; ++j) {
                if (t * JJ + j >= S0 && t * JJ + j < S1) {
                    const bool valid = (16 * t + r16 < nrows) && (j < spw);
                    st[t * JJ + j] = rows_ldw(rs, valid ? lane_off + t * 16 * (K * 2) + j * 64 : ROWS_OOB);
                }
            }
    };
    auto issue = [&](auto &st, auto tt_c, auto jj_c, const int kind, const int l) {
        issue_part(st, tt_c, jj_c, std::integral_constant<int, 0>{}, std::integral_constant<int, decltype(tt_c)::value * decltype(jj_c)::value>{}, kind, l);
    };
#define ROWS_IC(v) std::integral_constant<int, (v)>{}
    // this wave's partial tiles of a phase into red[(wave * ROWS_TA + t) * 256 + weight row * 16 + activation row]
    auto multiply = [&](const auto &st, auto tt_c, auto jj_c, const int kind) {
        constexpr int TT = decltype(tt_c)::value, JJ = decltype(jj_c)::value;
        const int spw = __builtin_amdgcn_readfirstlane(kinds[kind].spw), ntiles = __builtin_amdgcn_readfirstlane(kinds[kind].ntiles);
        // The 16 columns of the operand tile are the hi parts of the (at most 8) activation rows and, beside them,
        // their lo parts: one instruction per weight load multiplies both, and the two halves of a result row are
        // added before the tile goes to LDS.  (Rows past R repeat row 0; their results are not read.)
        const int nsrc = (r16 & 7) < R ? (r16 & 7) : 0;
        const uint16_t *pp = (r16 < 8 ? xh : xl) + nsrc * XS + wave * spw * 32 + c4 * 8;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
            if (t < ntiles) {
                rows_f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int j = 0; j < JJ; ++j) {
                    if (j < spw) {
                        const rows_bf16x8 w = __builtin_bit_cast(rows_bf16x8, st[t * JJ + j]);
                        const rows_bf16x8 bx = *(const rows_bf16x8 *)(pp + j * 32);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, bx, acc, 0, 0, 0);
                    }
                }
                // columns n and n + 8 of a result row (the hi and lo parts' products) are 8 lanes apart: one rotation
                // within the row of 16 lanes adds them
                acc[0] += dpp_get<0x128, 0xf>(acc[0]); acc[1] += dpp_get<0x128, 0xf>(acc[1]);
                acc[2] += dpp_get<0x128, 0xf>(acc[2]); acc[3] += dpp_get<0x128, 0xf>(acc[3]);
                float *rp = red + (wave * ROWS_TA + t) * 256 + (4 * c4) * 16 + r16;
                rp[0] = acc[0]; rp[16] = acc[1]; rp[32] = acc[2]; rp[48] = acc[3];
            }
        }
    };
    // sums of local rows 2p and 2p + 1 for activation row n, waves in order
    auto tile_pair = [&](const int p, const int n, float &s0, float &s1) {
        const int lr = 2 * p, t = lr >> 4, m = lr & 15;
        s0 = 0.0f; s1 = 0.0f;
#pragma unroll
        for (int w = 0; w < ROWS_WAVES; ++w) {
            const float *rp = red + (w * ROWS_TA + t) * 256 + m * 16 + n;
            s0 += rp[0]; s1 += rp[16];
        }
    };
    auto row_inv = [&](const int n) {
        float t = 0.0f;
        for (int c = 0; c < nchD; ++c) t += s_ssq[n * nchD + c];
        return 1.0f / sqrtf(t * (1.0f / (float)D) + 1e-5f);
    };

    unsigned long long *const prof = (VAR != MEGA_VAR_PLAIN && a.prof && b == 0 && tid == 0) ? a.prof : nullptr;
    int prof_n = 0;
    auto mark = [&]() { if (VAR != MEGA_VAR_PLAIN && prof) prof[prof_n++] = wall_clock64(); };

    __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0): the set-up loads

    const int wo_row0 = kinds[RK_WO].row0, wo_rows = kinds[RK_WO].nrows;     // same band for w2
    const int n_att = pos + 1;
    int NS = (n_att + SLOTS * MEGA_ATT_SPLIT_PASSES - 1) / (SLOTS * MEGA_ATT_SPLIT_PASSES);
    NS = max(1, min(NS, a.ns_max));
    const int chunk = (n_att + NS - 1) / NS;
    const float att_scale = 1.0f / sqrtf((float)HD);
    const int items = R * heads;

    // A layer is two halves of the same shape, and both run through one copy of the code: an "even" phase
    // (q/k/v, or gate / up: input rows polled with the norm's gains, set A) and an "odd" phase (output
    // projection behind the attention, or down projection: set B, residual added).
    // Weight requests: a set is asked for in two parts, each in front of a poll (the wave would wait there
    // anyway; in front of work, the time the memory pipeline takes to accept a part delays that work for
    // every workgroup).  In front of an even phase's poll: the second half of that phase's set A and the
    // first half of the following odd phase's set B; in front of an odd phase's poll: the second half of
    // its set B and the first half of the next even phase's set A.  Loads return in order, so whatever
    // was requested in front of a poll is there when the polled rows are.
    issue_part(stA, TA_C, JA_C, ROWS_IC(0), ROWS_IC(ROWS_JA), RK_QKV, 0);
    for (int hp = 0; hp < 2 * L; ++hp) {
        const int l = hp >> 1, h = hp & 1;
        const unsigned par = (ep + (unsigned)l + 1u) & 1u;   // stamp of layer l's exchanges
        const int ekind = h ? RK_W13 : RK_QKV, okind = h ? RK_W2 : RK_WO;
        float *const xres = xresb + (h ? R * xres_n : 0);    // raw residual inputs of this half's odd phase
        // ================================================================= even phase: q/k/v or gate / up
        if (VAR != MEGA_VAR_PLAIN) prof_n = l * ROWS_PROF_SLOTS + (h ? 9 : 0);
        mark();                                              // 0 / 9 start
        issue_part(stA, TA_C, JA_C, ROWS_IC(ROWS_JA), ROWS_IC(2 * ROWS_JA), ekind, l);
        issue_part(stB, TB_C, JB_C, ROWS_IC(0), ROWS_IC(ROWS_JB / 2), okind, l);
        {
            // the residual rows: the first layer's come from the embedding kernel (ordinary memory; the relay
            // gives them the stamp the poll expects), the others through the exchange
            const float *src = h ? a.X2 : hp == 0 ? a.x_in : a.X;
            float *const cp = h ? xbX2 : xbX;
            const unsigned pr = h ? par : par ^ 1u;
            const bool rok = rows_relay(src, cp, R * D / 4, members, rank, pr, par, abortf, hp == 0);
            const float rc = rows_poll<true, true>(cp, R, D, par, abortf, xh, xl, XS, (const float *)lptr[l * ROWS_LPTR + 4 + h], s_ssq,
                                                   xres, wo_row0, wo_rows, xres_n);
            if (rc < 0.0f || !rok) s_bad = 1;
            lds_barrier();
            if (s_bad) return;
            mark();                                          // 1 / 10 input staged
            __builtin_amdgcn_s_waitcnt(0x0F70);              // set A is here
            multiply(stA, TA_C, JA_C, ekind);
            lds_barrier();
            mark();                                          // 2 / 11 partial tiles written
            const RowsKind k = kinds[ekind];
            if (tid < k.npl * R) {
                const int p = tid / R, n = tid - p * R;
                float s0, s1;
                tile_pair(p, n, s0, s1);
                const float inv = row_inv(n);
                s0 *= inv; s1 *= inv;
                if (h == 0) {
                    const int row0 = 2 * (k.pair0 + p);
                    if (row0 < Q + KV) {                     // q and k rows: RoPE on the pair
                        const float c = ropes[2 * p], s = ropes[2 * p + 1];
                        const float e = s0 * c - s1 * s, o = s1 * c + s0 * s;
                        s0 = e; s1 = o;
                    }
                    if (row0 >= Q) {                         // k and v rows enter the row's suffix cache (and the exchange) in cache precision
                        const bool isk = row0 < Q + KV;
                        const int rr = isk ? row0 - Q : row0 - Q - KV;
                        void *cache = (void *)lptr[l * ROWS_LPTR + (isk ? 8 : 9)];
                        const size_t at = ((size_t)n * a.suf_rows + (size_t)slot) * KV + rr;
                        if (KVBF16) {
                            const uint16_t eb = f32_to_bf16_rne(s0), ob = f32_to_bf16_rne(s1);
                            uint16_t *cp2 = (uint16_t *)cache + at;
                            cp2[0] = eb; cp2[1] = ob;
                            s0 = bf16_to_f32(eb); s1 = bf16_to_f32(ob);
                        } else {
                            s0 = __uint_as_float(__float_as_uint(s0) & ~1u); s1 = __uint_as_float(__float_as_uint(s1) & ~1u);
                            float *cp2 = (float *)cache + at;
                            cp2[0] = s0; cp2[1] = s1;
                        }
                    }
                    st_stamped(a.QKV + (size_t)n * N + row0, s0, par);
                    st_stamped(a.QKV + (size_t)n * N + row0 + 1, s1, par);
                } else {
                    float gte;                               // (s0, s1) = (gate, up) pre-activations
                    if (a.act == 1) { const float lr = s0 > 0.0f ? s0 : 0.5f * s0; gte = lr * lr * s1; }
                    else { const float sig = 1.0f / (1.0f + expf(-s0)); gte = s0 * sig * s1; }
                    st_stamped(a.GATE + (size_t)n * H + (k.pair0 + p), gte, par);
                }
            }
            mark();                                          // 3 / 12 published
        }
        // ================================================================= odd phase: attention + output projection, or down projection
        if (h == 0) {
            const void *kcl = lptr[l * ROWS_LPTR + 6], *vcl = lptr[l * ROWS_LPTR + 7];
            const void *ksl = lptr[l * ROWS_LPTR + 8], *vsl = lptr[l * ROWS_LPTR + 9];
            if (b < items * NS) {
                const int sidx = b / items, rem = b - sidx * items, n = rem / heads, h = rem - n * heads, g = h / a.gqa;
                const int t0 = sidx * chunk, t1 = min(n_att, t0 + chunk);
                float *qs = stage + MEGA_WAVES * REC, *kcur = qs + HD, *vcur = kcur + HD;
                const int sub = tid % LPR, sl = tid / LPR;
                const size_t rowb = (size_t)KV * KESZ, hoff = ((size_t)g * HD + sub * KEPL) * KESZ;
                const char *kb = (const char *)kcl + hoff, *vb = (const char *)vcl + hoff;
                const char *ksb = (const char *)ksl + (size_t)n * a.suf_rows * rowb + hoff;
                const char *vsb = (const char *)vsl + (size_t)n * a.suf_rows * rowb + hoff;
                uint4 kr[PRE], vr[PRE];
                auto fetch = [&](const int tb) {
#pragma unroll
                    for (int i = 0; i < PRE; ++i) {
                        const int t = tb + sl + i * SLOTS;
                        if (t < t1 && t != pos) {
                            const bool shared = t < prefix;
                            const size_t at = (size_t)(shared ? t : t - prefix) * rowb;
                            kr[i] = ldg_u4((shared ? kb : ksb) + at);
                            vr[i] = ldg_u4((shared ? vb : vsb) + at);
                        }
                    }
                };
#pragma unroll
                for (int i = 0; i < PRE; ++i) { kr[i] = make_uint4(0, 0, 0, 0); vr[i] = make_uint4(0, 0, 0, 0); }
                fetch(t0);                                   // rows older than the new token are in the caches already
                {
                    bool ok = true;
                    if (tid < 3 * (HD / 4)) {
                        const int which = tid / (HD / 4), i4 = tid - which * (HD / 4);
                        const float *src = a.QKV + (size_t)n * N + (which == 0 ? h * HD : which == 1 ? Q + g * HD : Q + KV + g * HD);
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
                mark();                                      // 4 q, k, v of the item arrived
                float qv[KEPL];
#pragma unroll
                for (int e = 0; e < KEPL; ++e) qv[e] = qs[sub * KEPL + e];
                float m = -1e30f, lsum = 0.0f, acc[KEPL];
#pragma unroll
                for (int e = 0; e < KEPL; ++e) acc[e] = 0.0f;
                for (int tb = t0; tb < t1; tb += SLOTS * PRE) {
                    if (tb != t0) fetch(tb);
                    float d[PRE];
#pragma unroll
                    for (int i = 0; i < PRE; ++i) {
                        const int t = tb + sl + i * SLOTS;
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
                        if (tb + sl + i * SLOTS < t1) mn = fmaxf(mn, d[i]);
                    const float corr = __expf(m - mn);
                    lsum *= corr;
#pragma unroll
                    for (int e = 0; e < KEPL; ++e) acc[e] *= corr;
                    m = mn;
#pragma unroll
                    for (int i = 0; i < PRE; ++i) {
                        const int t = tb + sl + i * SLOTS;
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
                    float *pp = a.PART + (size_t)b * REC;            // record (split, row, head) = item b
                    st_stamped(pp + tid, A, par);
                    if (tid < MEGA_PREC) st_stamped(pp + HD + tid, tid == 0 ? M : tid == 1 ? Ls : 0.0f, par);
                }
                lds_barrier();
                mark();                                      // 5 partial published
            } else if (b < items * a.ns_max) {
                // a split record nobody fills at this position still takes the layer's stamp (an empty
                // partial), so that it never carries a stamp of unknown age when the split count grows
                if (tid < REC) st_stamped(a.PART + (size_t)b * REC + tid, tid == HD ? -1e30f : 0.0f, par);
            }
        }
        issue_part(stB, TB_C, JB_C, ROWS_IC(ROWS_JB / 2), ROWS_IC(ROWS_JB), okind, l);
        if (hp + 1 < 2 * L) issue_part(stA, TA_C, JA_C, ROWS_IC(0), ROWS_IC(ROWS_JA), h ? RK_QKV : RK_W13, h ? l + 1 : l);
        {
            bool rok;
            if (h == 0) rok = rows_fold_relay<HD>(a.PART, xbA, NS, R, heads, Q, members, rank, par, par, abortf);
            else rok = rows_relay(a.GATE, xbG, R * H / 4, members, rank, par, par, abortf, false);
            const float rc = rows_poll<false, false>(h ? xbG : xbA, R, h ? H : Q, par, abortf, xh, xl, XS, nullptr, nullptr, nullptr, 0, 0, 0);
            if (rc < 0.0f || !rok) s_bad = 1;
            lds_barrier();
            if (s_bad) return;
            mark();                                          // 6 / 13 input staged
            __builtin_amdgcn_s_waitcnt(0x0F70);              // set B is here
            multiply(stB, TB_C, JB_C, okind);
            lds_barrier();
            mark();                                          // 7 / 14 partial tiles written
            const RowsKind k = kinds[okind];
            if (tid < k.npl * R) {
                const int p = tid / R, n = tid - p * R;
                float s0, s1;
                tile_pair(p, n, s0, s1);
                const int row0 = k.row0 + 2 * p;
                float *dstv = h ? a.X : a.X2;
                st_stamped(dstv + (size_t)n * D + row0, xres[n * xres_n + 2 * p] + a.alpha * s0, par);
                st_stamped(dstv + (size_t)n * D + row0 + 1, xres[n * xres_n + 2 * p + 1] + a.alpha * s1, par);
            }
            mark();                                          // 8 / 15 residual published
        }
    }
    if (VAR != MEGA_VAR_PLAIN) prof_n = L * ROWS_PROF_SLOTS;
    mark();

    // ---- the last residual rows for the LM head: workgroup (row, chunk) polls 256 values, wave 0 only
    if (b < R * nchD && wave == 0) {
        const int n = b / nchD, ch = b - n * nchD, i4 = ch * 64 + lane;
        const unsigned parL = (ep + (unsigned)L) & 1u;       // stamp of the last layer
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(a.X, R * D * 4);
        const int off = (n * D + 4 * i4) * 4;
        const mega_u4 g = *(const __attribute__((address_space(1))) mega_u4 *)(a.gfinal + 4 * i4);
        mega_u4 v = ld16_coherent(rs, off);
        const bool ok = repoll16(v, rs, off, parL ? 0xffffffffu : 0u, abortf);
        if (!__any(!ok)) {
            const float x0 = __uint_as_float(v.x & ~1u), x1 = __uint_as_float(v.y & ~1u), x2 = __uint_as_float(v.z & ~1u),
                        x3 = __uint_as_float(v.w & ~1u);
            uint32_t h0, l0, h1, l1;
            pf_split2(x0 * __uint_as_float(g.x), x1 * __uint_as_float(g.y), h0, l0);
            pf_split2(x2 * __uint_as_float(g.z), x3 * __uint_as_float(g.w), h1, l1);
            *(uint2 *)(a.out_hi + (size_t)n * D + 4 * i4) = make_uint2(h0, h1);
            *(uint2 *)(a.out_lo + (size_t)n * D + 4 * i4) = make_uint2(l0, l1);
            const float ss = wave_sum_dpp((x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3));
            if (lane == 63) a.out_ssq[n * nchD + ch] = ss;
        }
    }
    if (b == 0 && tid == 0) { a.epochs[0] = ep + (unsigned)L; a.epochs[1] = ep_launch + 1u; }
}
