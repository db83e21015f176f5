// One-launch-per-token decode step for gfx950: a persistent kernel with one workgroup per CU.
//
// A batch-1 token step is a chain of ~5 dependent matrix-vector products per layer, each only a
// few microseconds of HBM streaming on this machine; launched as separate kernels the chain is
// bound by launch/ramp latency, not by bandwidth.  Here every workgroup stays resident for the
// whole step and the layers' phases are separated by data exchanges through device memory:
//
//  * every activation vector a phase hands to the next one (residual stream, q/k/v of the new
//    token, attention partials, gate vector) is written with device-coherent stores and carries an
//    epoch bit in the least significant mantissa bit of each fp32 value; a consumer polls the
//    values themselves (128-bit device-coherent loads, every 32-bit word self-validating) until
//    every element shows the expected epoch, so one store->load round trip replaces
//    "write, fence, signal, wait, fence, read";
//  * weight addresses do not depend on activations, so each wave requests its next round of
//    16-byte weight loads before it leaves the current phase: while a workgroup waits for its
//    inputs the HBM stream for the next phase is already running;
//  * the phases of all layers run through ONE copy of the polling / streaming / reduction code
//    (a loop over phases with a small switch per phase), which keeps the loop body inside the
//    instruction cache.
//
// All reductions run in a fixed order and the stamp bit is cleared from every value before it is
// used, so a step is bit-reproducible whatever the epoch.  Every wait is bounded:
// a workgroup that spins too long raises an abort flag that makes every other workgroup leave too.
#pragma once
#include "hipdec_kernels.h"
#include <type_traits>

#define MEGA_THREADS 512
#define MEGA_WAVES 8
#define MEGA_DEPTH 4            // tasks per round of the even phases (16 loads of 16 bytes in flight per lane)
#ifndef MEGA_DEPTH_B
#define MEGA_DEPTH_B 2          // tasks per round of the odd phases (wo, w2: few rows per workgroup); divides MEGA_DEPTH
#endif
#define MEGA_SEG_PIECES 128     // 16-byte pieces of one row per task: 2 per lane
#define MEGA_SPIN_LIMIT (1u << 22)
#define MEGA_PREC 4             // attention partial record = HD + 4 floats (acc[HD], max, sum, 0, 0)
#define MEGA_PROF_SLOTS 32      // timestamps per layer when profiling
#ifndef MEGA_ATT_PRE
#define MEGA_ATT_PRE 4          // attention: cache-row passes a thread requests ahead
#endif
#ifndef MEGA_ATT_SPLIT_PASSES
#define MEGA_ATT_SPLIT_PASSES 4 // attention: passes (of 512 / lanes-per-row cache rows) one split covers while splits are to be had
                                // (600M at 256 positions: 1 pass 0.591, 2 passes 0.573, 4 passes 0.556, 8 passes 0.575 ms per token:
                                // every further split is two more polls per thread in the fold)
#endif
#define MEGA_LPTR 12            // pointers per layer in the LDS copy of the layer table
#ifndef MEGA_LDS_TASKS
#define MEGA_LDS_TASKS 2        // odd-phase tasks (4 KB each) per wave that are prefetched into LDS behind the register round
#endif

enum { MK_QKV = 0, MK_WO = 1, MK_W13 = 2, MK_W2 = 3, MK_HEAD = 4, MK_KINDS = 5 };

struct MegaLayer {
    const void *w[4];        // wqkv, wo, w13, w2 (out-major)
    const void *sc[4];       // scales (fp8 / int4)
    const float *g1, *g2;
    void *kc, *vc;
};

struct MegaArgs {
    const MegaLayer *layers;
    const void *embed;
    const float *gfinal, *x_in, *rope_cos, *rope_sin;
    float *X, *QKV, *PART, *X2, *GATE, *logits;      // exchange buffers (device memory, zeroed at creation)
    unsigned long long *CAND;                        // [grid] argmax candidates
    StepParams *sp;
    uint32_t *ring;
    unsigned *epochs;                                // [0] per-layer exchange counter, [1] head counter
    unsigned *abort;                                 // abort flag (host memory mapped into the device)
    unsigned long long *prof;                        // nullable: workgroup 0 writes wall-clock stamps here
    int ring_cap;
    int D, Q, KV, H, V, L, hd, heads, gqa, act, do_head, advance, ns_max, seq, stage_floats;
    int prof_wg;                                     // workgroup whose time stamps the profiling build records
    int lds_tasks;                                   // 0, or MEGA_LDS_TASKS: the LDS has room for that many prefetched tasks per wave
    float alpha;
};

struct MegaKind {            // per-workgroup view of one GEMV kind
    int pieces, segs, pair0, npl, ntasks, K;
    size_t row_bytes;
};

typedef unsigned mega_u4 __attribute__((ext_vector_type(4)));

// Loads through pointers that were themselves loaded from a table have an unknown address space
// and compile to flat loads, which the compiler can only wait for with a full counter drain (and
// which it also drains before issuing more).  These helpers state that the memory is global.
__device__ __forceinline__ uint4 ldg_u4(const void *p) {
    const mega_u4 v = *(const __attribute__((address_space(1))) mega_u4 *)p;
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint16_t ldg_u16(const void *p) {
    return *(const __attribute__((address_space(1))) uint16_t *)p;
}

__device__ __forceinline__ unsigned ld_u32_coherent(const unsigned *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The abort flag of a model lives in pinned host memory that the device maps: the host reads it after
// its wait for the stream without a copy of its own, the kernels touch it only when a wait has lasted
// for many polls.
__device__ __forceinline__ unsigned ld_abort(const unsigned *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void raise_abort(unsigned *p) {
    __hip_atomic_store(p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
// How a waiting thread bounds its wait: it looks at its poll count when (count & mask) == 0 and gives up
// at `limit`.  Constants of the device so that a test can make the waits give up (hipdec_debug_set_spin_limit).
__constant__ unsigned g_spin_ctl[2] = {127u, MEGA_SPIN_LIMIT};
__device__ __forceinline__ void st_stamped(float *p, float v, unsigned par) {
    unsigned u = (__float_as_uint(v) & ~1u) | par;
    __hip_atomic_store((unsigned *)p, u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 128-bit load that bypasses the non-coherent cache levels (sc1: device scope on gfx94x/gfx950)
__device__ __forceinline__ mega_u4 ld16_coherent(__amdgpu_buffer_rsrc_t r, int byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 16);
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ bool stamp_bad(const mega_u4 &v, unsigned pm) {
    return (((v.x ^ pm) | (v.y ^ pm) | (v.z ^ pm) | (v.w ^ pm)) & 1u) != 0;
}
// one 16-byte slot: reload until all four words carry the expected stamp (bounded)
__device__ __forceinline__ bool repoll16(mega_u4 &v, __amdgpu_buffer_rsrc_t r, int byte_off, unsigned pm, unsigned *abortf) {
    unsigned spins = 0;
    while (stamp_bad(v, pm)) {
        if ((++spins & g_spin_ctl[0]) == 0) {
            if (ld_abort(abortf)) return false;
            if (spins > g_spin_ctl[1]) {
                raise_abort(abortf);
                return false;
            }
        }
        v = ld16_coherent(r, byte_off);
    }
    return true;
}

// Layout of a staged input vector in LDS.  The multiply reads it one 16-byte chunk per lane and
// instruction, lane l holding piece l of a segment (a piece = the EPL inputs of one 16-byte weight
// load).  With pieces of 64 or 128 bytes, eight neighbouring lanes of such a read meet in a quarter
// or an eighth of the 32 LDS banks.  The chunks of a piece are therefore stored rotated by the
// piece's index (counted in 128-byte bank rows), which spreads every read over all banks.
// MEGA_SWZ_MIN_EPL: smallest piece (in inputs) stored this way.
#ifndef MEGA_SWZ_MIN_EPL
#define MEGA_SWZ_MIN_EPL 16
#endif
__device__ __forceinline__ int xs_chunk_pos(int chunk, int epl) {     // epl: 0 (plain order), 8, 16 or 32
    if (epl == 0) return chunk;
    const int cpl = epl == 32 ? 3 : epl == 16 ? 2 : 1;                // log2(chunks per piece)
    const int piece = chunk >> cpl, c = chunk & ((1 << cpl) - 1);
    return (piece << cpl) | ((c + (piece >> (3 - cpl))) & ((1 << cpl) - 1));
}
__device__ __forceinline__ int xs_pos(int i, int epl) { return (xs_chunk_pos(i >> 2, epl) << 2) | (i & 3); }

// Polls n stamped floats (n % 4 == 0, src 16-byte aligned) with the polling waves (thread pt of
// MEGA_PT) into dst (LDS): dst[i] = src[i] * (gamma ? gamma[i] : 1); elements with index in
// [r0, r0 + nres) are also copied raw to res[i - r0].  Returns this thread's sum of squares of
// the raw values, or a negative value when the wait was aborted (a flag returned through memory
// would live in scratch memory).  Kept out of line: inlined, the compiler sinks each poll load next
// to its use and the loads of one thread stop overlapping.  The price is that a called function
// starts by waiting for every outstanding load of the wave, the requested weights included; loads
// return in order, so the polled values could not be seen before those anyway.
#define MEGA_PT MEGA_THREADS                        // polling threads
// SWZ_EPL: layout of dst (0 plain order, else xs_chunk_pos(., SWZ_EPL)); NB: slots a thread requests
// before it looks at the first one (every further group of NB costs another round trip).
template <int SWZ_EPL, int NB = 2048 / MEGA_PT, bool GAMMA = true>     // GAMMA false: gamma is null, no registers for it
__device__ __noinline__ float mega_poll_vec(const float *src, int n, unsigned par, unsigned *abortf, float *dst,
                                            const float *gamma, float *res, int r0, int nres, int pt) {
    const int n4 = n >> 2;
    const __amdgpu_buffer_rsrc_t r = make_rsrc(src, n * 4);
    const unsigned pm = par ? 0xffffffffu : 0u;
    float ss = 0.0f;
    bool good = true;
    for (int base = 0; base < n4 && good; base += MEGA_PT * NB) {
        mega_u4 v[NB], g[GAMMA ? NB : 1];
        // the norm weights do not depend on the exchange: request them first so that they are
        // there when the stamped values arrive
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
                // the stamp bit is cleared before use, so a value does not depend on the epoch it travelled in
                float x[4] = {__uint_as_float(v[b].x & ~1u), __uint_as_float(v[b].y & ~1u), __uint_as_float(v[b].z & ~1u),
                              __uint_as_float(v[b].w & ~1u)};
                float4 o;
                const mega_u4 gb = g[GAMMA ? b : 0];
                const float4 gm = make_float4(__uint_as_float(gb.x), __uint_as_float(gb.y), __uint_as_float(gb.z), __uint_as_float(gb.w));
                o.x = x[0] * gm.x; o.y = x[1] * gm.y; o.z = x[2] * gm.z; o.w = x[3] * gm.w;
                *(float4 *)(dst + 4 * xs_chunk_pos(i, SWZ_EPL)) = o;
                ss += x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int j = 4 * i + e - r0;
                    if (j >= 0 && j < nres) res[j] = x[e];
                }
            }
        }
    }
    return good ? ss : -1.0f;
}

// One load-to-LDS instruction of a wave: the 16 bytes at gptr of every active lane l land at LDS byte
// address lds_base + 16 l (lds_base wave-uniform, through M0).  No destination registers, so a round of
// weights requested this way costs no register set; it is counted by vmcnt like any other load and
// completes in order with them.  Issued as assembly: the compiler then places no waits of its own for it
// (the waits that cover it are stated by hand where the data is read).
__device__ __forceinline__ void mega_dma16(const void *gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(gptr), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ uint32_t mega_lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load, which would stall each phase on the weight loads requested for the
// next one; nothing in this kernel passes data between the waves of a workgroup through global
// memory, so the LDS-only form is sufficient.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int WT> struct MegaStage {
    uint4 w[2][2];           // [row of the pair][piece j]
    uint32_t sc[2][2];       // int4 group scales (bf16 bits)
};

// VAR selects one of two builds of the kernel: MEGA_VAR_PLAIN (no time stamps: the stamp code, although
// never executed without a profile buffer, costs the 600M step 1.7 % in registers and branches) and
// MEGA_VAR_STAMPS (the same with time stamps, for the step profile).
enum { MEGA_VAR_PLAIN = 0, MEGA_VAR_STAMPS = 1 };
template <int WT, int KVBF16, int HD, int VAR>
__global__ __launch_bounds__(MEGA_THREADS, 1) void k_mega(MegaArgs a) {
    constexpr int EPL = WS<WT>::EPL;
    constexpr int KESZ = KVBF16 ? 2 : 4;
    constexpr int KEPL = 16 / KESZ;
    constexpr int LPR = HD / KEPL;               // lanes per cache row
    constexpr int SLOTS = MEGA_THREADS / LPR;    // cache rows per pass
    constexpr int PRE = MEGA_ATT_PRE;            // passes prefetched
    constexpr int REC = HD + MEGA_PREC;          // floats per attention partial record
    constexpr int XSWZ = EPL >= MEGA_SWZ_MIN_EPL ? EPL : 0;   // chunk rotation of the staged vectors (0: plain order)
    extern __shared__ __align__(16) float smem[];
    __shared__ MegaKind kinds[MK_KINDS];
    __shared__ float s_red[2][MEGA_WAVES];       // per-wave sums of squares, by phase parity
    __shared__ float s_cand_v[MEGA_WAVES];       // per-wave argmax candidates of the head phase
    __shared__ uint32_t s_cand_i[MEGA_WAVES];
    __shared__ int s_bad;                       // set once by any thread whose wait was aborted

    int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: per-wave bookkeeping stays on the scalar unit
    if (tid == 0) s_bad = 0;
    const int G = gridDim.x, b = blockIdx.x;
    const int D = a.D, Q = a.Q, KV = a.KV, H = a.H, V = a.V, L = a.L;
    // the staged input vector is double-buffered by phase parity: a wave may still read phase p's
    // vector while another already stages phase p+1's.  Even phases (qkv, w13, head) read D floats,
    // odd phases (wo, w2) max(Q, H).
    float *xsb = smem;                                       // [D] then [max(Q, H)]
    float *stage = xsb + D + max(Q, H);                      // attention: per-wave partials, q / k / v of the new token; odd phases: per-task sums
    const int stage_floats = a.stage_floats;                 // host: max(MEGA_WAVES * REC + 3 * HD, 2 * tasks of an odd phase)
    const int xres_n = 2 * ((D / 2 + G - 1) / G) + 2;
    float *xresb = stage + stage_floats;                     // [2][xres_n] residual inputs of this workgroup's wo / w2 rows
    float *ropes = xresb + 2 * xres_n;                       // (cos, sin) of this workgroup's q/k row pairs
    // weight / scale pointers of every layer, copied once so that computing a load address never
    // waits on device memory: [L][MEGA_LPTR] = w[4], sc[4], g1, g2, kc, vc
    const void **lptr = (const void **)(ropes + 2 * (((Q + 2 * KV) / 2 + G - 1) / G) + 2);
    // prefetch area of the odd phases: [wave][task][load] kilobytes, 1 KB aligned (present when a.lds_tasks != 0)
    char *const wl = (char *)(((uintptr_t)(lptr + MEGA_LPTR * L) + 1023) & ~(uintptr_t)1023);
    for (int i = threadIdx.x; i < MEGA_LPTR * L; i += MEGA_THREADS) {
        const int l = i / MEGA_LPTR, j = i - l * MEGA_LPTR;
        const MegaLayer &ml = a.layers[l];
        lptr[i] = j < 4 ? ml.w[j] : j < 8 ? ml.sc[j - 4] : j == 8 ? (const void *)ml.g1 : j == 9 ? (const void *)ml.g2
                                                         : j == 10 ? (const void *)ml.kc : (const void *)ml.vc;
    }

    // ---- per-workgroup partition of each GEMV kind
    if (tid < MK_KINDS) {
        int rows, K;
        switch (tid) {
            case MK_QKV: rows = Q + 2 * KV; K = D; break;
            case MK_WO: rows = D; K = Q; break;
            case MK_W13: rows = 2 * H; K = D; break;
            case MK_W2: rows = D; K = H; break;
            default: rows = V; K = D; break;
        }
        int npairs = rows >> 1, base = npairs / G, rem = npairs % G;
        MegaKind &k = kinds[tid];
        k.K = K;
        k.pieces = K / EPL;
        k.segs = (k.pieces + MEGA_SEG_PIECES - 1) / MEGA_SEG_PIECES;
        k.pair0 = b * base + min(b, rem);
        k.npl = base + (b < rem ? 1 : 0);
        k.ntasks = k.npl * k.segs;
        k.row_bytes = WS<WT>::row_bytes(K);
    }
    const int pos = a.sp->pos, tok = a.sp->tok, use_x_in = a.sp->use_x_in;
    const unsigned ep_layer = a.epochs[0], ep_head = a.epochs[1];
    unsigned *abortf = a.abort;
    __syncthreads();

    if (wave == 0) {
        const MegaKind &k = kinds[MK_QKV];
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

    // The GEMV phases run in the order l*4 + kind (qkv, wo, w13, w2 of layer l), then the head.  Even
    // phases (qkv, w13, head: many rows, reduction over D) and odd phases (wo, w2: D rows shared by all
    // workgroups, long reductions) alternate, and each kind of phase has a register set of its own for
    // the weights it streams:
    //  * set A, MEGA_DEPTH tasks per round.  A task is (row pair, segment of MEGA_SEG_PIECES pieces);
    //    wave w owns the local pairs w, w + 8, ... and walks each pair's segments in order, keeps per-lane
    //    sums across the segments, reduces them across lanes once, and its last lane finishes and
    //    publishes the two outputs, so the waves never wait for each other after staging;
    //  * set B, MEGA_DEPTH_B tasks per round.  An odd phase has only a few row pairs per workgroup, so
    //    its (pair, segment) tasks are dealt to the waves one by one (task t to wave t % 8); the per-task
    //    sums meet in LDS and the first threads of the workgroup finish the rows.
    // The first round of a phase is requested when the input of the phase BEFORE it has been seen, into
    // the set that phase does not use: it streams while that phase multiplies and publishes and while
    // the exchange travels.  Inside a phase the next round follows the current one into the same set.
    // Each set is written at fixed places of the loop body, always after its last use, so the loads
    // land in the registers the multiply reads (a set refilled on only one of two merging paths is
    // copied register by register at the merge, which waits for the loads).
    const int pt = tid;                                      // every thread polls
    const int last_ph = a.do_head ? 4 * L : 4 * L - 1;
    MegaStage<WT> stA[MEGA_DEPTH], stB[MEGA_DEPTH_B];
    int e_left = 0, e_pl = 0, e_sg = 0;                      // cursor of set A: tasks left in its phase, next (local pair, segment)
    int o_left = 0, o_pl = 0, o_sg = 0;                      // cursor of set B
    // Lanes past the end of a row and padding tasks issue nothing (a skipped load is not free if it
    // is issued anyway: it still occupies the address unit) and are ignored when the round is consumed.
    struct IssueCtx {                                        // what the loads of one phase's rounds need
        int pieces, segs, pair0, kg;
        size_t rb;
        const char *W;
        const uint16_t *SC;
    };
    auto prep_issue = [&](int ph) {
        const int kind = ph == 4 * L ? MK_HEAD : (ph & 3);
        const MegaKind &k = kinds[kind];
        IssueCtx c;
        c.pieces = k.pieces; c.segs = k.segs; c.pair0 = k.pair0; c.kg = k.K / 128; c.rb = k.row_bytes;
        c.W = kind == MK_HEAD ? (const char *)a.embed : (const char *)lptr[(ph >> 2) * MEGA_LPTR + kind];
        c.SC = kind == MK_HEAD ? nullptr : (const uint16_t *)lptr[(ph >> 2) * MEGA_LPTR + 4 + kind];
        return c;
    };
    IssueCtx ctxA = prep_issue(0), ctxB = prep_issue(0);     // of the phase each cursor walks
    auto start_even = [&](int ph) {
        const int kind = ph == 4 * L ? MK_HEAD : (ph & 3);
        const int npl = kinds[kind].npl;
        e_left = npl > wave ? ((npl - wave + MEGA_WAVES - 1) / MEGA_WAVES) * kinds[kind].segs : 0;
        e_pl = wave; e_sg = 0;
        ctxA = prep_issue(ph);
    };
    // the next task of set A's cursor into t
    auto issue_even_one = [&](const IssueCtx &c, MegaStage<WT> &t) {
        if (e_left > 0) {
            const size_t row = (size_t)2 * (c.pair0 + e_pl);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int piece = e_sg * MEGA_SEG_PIECES + j * 64 + lane;
                if (piece < c.pieces) {
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        t.w[r][j] = ld_stream_u4(c.W + (row + r) * c.rb + (size_t)piece * 16);
                        if (WT == WT_INT4) t.sc[r][j] = ldg_u16(c.SC + (row + r) * c.kg + (piece >> 2));   // 4-bit models keep the head outside
                    }
                }
            }
            --e_left;
            if (++e_sg == c.segs) { e_sg = 0; e_pl += MEGA_WAVES; }
        }
    };
    auto issue_even = [&]() {
#pragma unroll
        for (int s = 0; s < MEGA_DEPTH; ++s) issue_even_one(ctxA, stA[s]);
    };
    auto start_odd = [&](int ph) {
        const MegaKind &k = kinds[ph & 3];
        o_left = k.ntasks > wave ? (k.ntasks - wave + MEGA_WAVES - 1) / MEGA_WAVES : 0;
        o_pl = 0; o_sg = wave;
        while (o_sg >= k.segs) { o_sg -= k.segs; ++o_pl; }
        ctxB = prep_issue(ph);
    };
    auto issue_odd_one = [&](const IssueCtx &c, MegaStage<WT> &t) {
        if (o_left > 0) {
            const size_t row = (size_t)2 * (c.pair0 + o_pl);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int piece = o_sg * MEGA_SEG_PIECES + j * 64 + lane;
                if (piece < c.pieces) {
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        t.w[r][j] = ld_stream_u4(c.W + (row + r) * c.rb + (size_t)piece * 16);
                        if (WT == WT_INT4) t.sc[r][j] = ldg_u16(c.SC + (row + r) * c.kg + (piece >> 2));
                    }
                }
            }
            --o_left;
            o_sg += MEGA_WAVES;
            while (o_sg >= c.segs) { o_sg -= c.segs; ++o_pl; }
        }
    };
    auto issue_odd = [&]() {
#pragma unroll
        for (int s = 0; s < MEGA_DEPTH_B; ++s) issue_odd_one(ctxB, stB[s]);
    };
    // The tasks behind the register round of an odd phase, requested into LDS: up to MEGA_LDS_TASKS per wave,
    // each wave into its own slots, which only it reads back (so its own vmcnt wait is all the
    // synchronisation there is).  Requested in front of the phase's poll -- the wait for the attention
    // partials or for the gate vector, during which the memory pipeline would otherwise idle.
    int l_n = 0;                                             // tasks of the coming odd phase this wave has in LDS
    uint32_t l_sc[MEGA_LDS_TASKS][2][2];                     // their 4-bit group scales
    const uint32_t wl_wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)mega_lds_addr(wl)) + (uint32_t)wave * (MEGA_LDS_TASKS * 4096u);
    auto issue_odd_lds = [&]() {
        l_n = 0;
        if (!a.lds_tasks) return;
#pragma unroll
        for (int q = 0; q < MEGA_LDS_TASKS; ++q) {
            if (o_left > 0) {
                const IssueCtx &c = ctxB;
                const size_t row = (size_t)2 * (c.pair0 + o_pl);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int piece = o_sg * MEGA_SEG_PIECES + j * 64 + lane;
                    if (piece < c.pieces) {
#pragma unroll
                        for (int r = 0; r < 2; ++r) {
                            mega_dma16(c.W + (row + r) * c.rb + (size_t)piece * 16, wl_wave + (uint32_t)((q * 4 + j * 2 + r) * 1024));
                            if (WT == WT_INT4) l_sc[q][r][j] = ldg_u16(c.SC + (row + r) * c.kg + (piece >> 2));
                        }
                    }
                }
                --o_left;
                o_sg += MEGA_WAVES;
                while (o_sg >= c.segs) { o_sg -= c.segs; ++o_pl; }
                ++l_n;
            }
        }
    };
    auto read_lds_task = [&](const int q, MegaStage<WT> &t) {
        const char *base = wl + ((size_t)wave * MEGA_LDS_TASKS + q) * 4096 + lane * 16;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                t.w[r][j] = *(const uint4 *)(base + (j * 2 + r) * 1024);
                if (WT == WT_INT4) t.sc[r][j] = l_sc[q][r][j];
            }
    };
    // one task: both rows of a pair times the staged vector over one segment
    auto mul_task = [&](const MegaStage<WT> &t, const float *xs, const int sg, const int pieces, float &o0, float &o1) {
        o0 = 0.0f; o1 = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int piece = sg * MEGA_SEG_PIECES + j * 64 + lane;
            if (piece < pieces) {
                float xv[EPL];
                constexpr int CPP = EPL / 4;                              // chunks per piece
                const int rot = XSWZ ? piece >> (EPL == 32 ? 0 : EPL == 16 ? 1 : 2) : 0;
#pragma unroll
                for (int e = 0; e < EPL; e += 4) {
                    float4 tq = *(const float4 *)(xs + piece * EPL + 4 * ((e / 4 + rot) & (CPP - 1)));
                    xv[e] = tq.x; xv[e + 1] = tq.y; xv[e + 2] = tq.z; xv[e + 3] = tq.w;
                }
                float w0[EPL], w1[EPL];
                WS<WT>::decode(t.w[0][j], w0);
                WS<WT>::decode(t.w[1][j], w1);
                float p0 = 0.0f, p1 = 0.0f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) { p0 = fmaf(w0[e], xv[e], p0); p1 = fmaf(w1[e], xv[e], p1); }
                if (WT == WT_INT4) {
                    p0 *= bf16_to_f32(t.sc[0][j]) * WS<WT_INT4>::SCALE_MUL;
                    p1 *= bf16_to_f32(t.sc[1][j]) * WS<WT_INT4>::SCALE_MUL;
                }
                o0 += p0; o1 += p1;
            }
        }
    };
    // Drain the set-up loads here, once: a load still pending on entry to the phase loop would make
    // the compiler wait for "everything outstanding" at the top of every iteration, which later
    // includes the weights requested for the phase.
    __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0)
    // A model whose phases are a single round for every wave (the widest share of a kind: ceil(pairs / G)
    // pairs) is bound by the exchanges, not by the stream: there, a request is only put in front of a
    // poll when the multiply behind that poll needs it (loads return in order, so the polled vector
    // is seen after everything requested before it).  A model with several rounds per phase keeps the
    // earliest possible requests.
    auto own_rounds = [&](int rows, int kind) { return (((rows / 2 + G - 1) / G + MEGA_WAVES - 1) / MEGA_WAVES) * kinds[kind].segs; };
    auto dealt_rounds = [&](int rows, int kind) { return (((rows / 2 + G - 1) / G) * kinds[kind].segs + MEGA_WAVES - 1) / MEGA_WAVES; };
    const bool qkv_one_round = own_rounds(Q + 2 * KV, MK_QKV) <= MEGA_DEPTH;
    const bool b0_late = qkv_one_round && own_rounds(2 * H, MK_W13) <= MEGA_DEPTH && dealt_rounds(D, MK_WO) <= MEGA_DEPTH_B &&
                         dealt_rounds(D, MK_W2) <= MEGA_DEPTH_B;
    start_even(0);
    issue_even();
    o_left = 0;
    if (1 <= last_ph) { start_odd(1); if (!b0_late) issue_odd_one(ctxB, stB[0]); }

    const int wo_row0 = 2 * kinds[MK_WO].pair0, wo_rows = 2 * kinds[MK_WO].npl;   // same partition for w2

    const int n_att = pos + 1;
    int NS = (n_att + SLOTS * MEGA_ATT_SPLIT_PASSES - 1) / (SLOTS * MEGA_ATT_SPLIT_PASSES);
    NS = max(1, min(NS, a.ns_max));
    const int chunk = (n_att + NS - 1) / NS;
    const float att_scale = 1.0f / sqrtf((float)HD);
    const unsigned par_c = (ep_head + 1u) & 1u;

    for (int ph = 0; ph <= last_ph; ph += 2) {
        // The thread's index is made opaque here, so that nothing derived from it (addresses, lane
        // masks) is kept in registers across the phases; recomputing is a few instructions per use.
        asm volatile("" : "+v"(tid), "+v"(lane));
        // ===================================================================== even phase: qkv, w13 or head
        {
        const int l = min(ph >> 2, L - 1);
        const int kind = ph == 4 * L ? MK_HEAD : (ph & 3);
        const unsigned par = (ep_layer + (unsigned)l + 1u) & 1u;      // stamp of layer l's exchanges
        const float *g1 = (const float *)lptr[l * MEGA_LPTR + 8], *g2 = (const float *)lptr[l * MEGA_LPTR + 9];
        void *kcl = (void *)lptr[l * MEGA_LPTR + 10], *vcl = (void *)lptr[l * MEGA_LPTR + 11];
        float *xs = xsb;
        // residual inputs: the qkv stage keeps x for the wo epilogue in buffer 0, the w13 stage keeps
        // x2 for the w2 epilogue in buffer 1
        float *xres_w = xresb + (kind == MK_W13 ? xres_n : 0);
        if (prof && kind != MK_W13) prof_n = (ph >> 2) * MEGA_PROF_SLOTS;
        mark();

        // ---- stage this phase's input vector in xs
        float ss = 0.0f;
        bool ok = true;
        if (kind == MK_QKV && l == 0) {
            for (int i = tid; i < D; i += MEGA_THREADS) {
                float v;
                if (use_x_in) v = a.x_in[i];
                else if (WT == WT_F32) v = ((const float *)a.embed)[(size_t)tok * D + i];
                else v = bf16_to_f32(((const uint16_t *)a.embed)[(size_t)tok * D + i]);
                xs[xs_pos(i, XSWZ)] = v * g1[i];
                ss += v * v;
                if (i >= wo_row0 && i < wo_row0 + wo_rows) xres_w[i - wo_row0] = v;
            }
        } else {
            // qkv / head: X of the previous layer; w13: X2
            const float *src = kind == MK_W13 ? a.X2 : a.X;
            const float *gm = kind == MK_QKV ? g1 : kind == MK_W13 ? g2 : a.gfinal;
            const unsigned pr = kind == MK_QKV ? (par ^ 1u) : kind == MK_HEAD ? ((ep_layer + (unsigned)L) & 1u) : par;
            const int nres = kind == MK_HEAD ? 0 : wo_rows;
            ss = mega_poll_vec<XSWZ>(src, D, pr, abortf, xs, gm, xres_w, wo_row0, nres, pt);
            if (ss < 0.0f) { ok = false; ss = 0.0f; }
        }
        ss = wave_sum_dpp(ss);                    // (no LDS round trips; total in lane 63)
        if (lane == 63) s_red[0][wave] = ss;
        if (!ok) s_bad = 1;
        lds_barrier();
        if (s_bad) return;
        mark();
        // This phase's input is here, and so is set A (requested a phase ago; the multiply needs it now
        // anyway).  The explicit wait tells the compiler so: from here on only the loads requested below
        // are outstanding, and the multiply of set A runs without waiting for them.
        __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0)
        // Requests are spread over the phases, one task (four loads per lane) at a time, so that each one
        // finds room in the memory pipeline: requested in one block, a round holds the wave at the
        // address unit for a good part of the time the block takes to stream.  Here: the second task of
        // the odd phase behind this one (its first went out at the end of the odd phase before, or goes
        // out here: b0_late).
        if (b0_late) issue_odd_one(ctxB, stB[0]);
#pragma unroll
        for (int s = 1; s < MEGA_DEPTH_B; ++s) issue_odd_one(ctxB, stB[s]);
        float inv;
        {
            float t = 0.0f;
#pragma unroll
            for (int w = 0; w < MEGA_WAVES; ++w) t += s_red[0][w];
            inv = 1.0f / sqrtf(t * (1.0f / (float)D) + 1e-5f);
        }

        // ---- stream this workgroup's rows in rounds of MEGA_DEPTH tasks
        float bv = -INFINITY; uint32_t bi = 0x7fffffffu;      // head phase: best logit this lane has finished
        {
            const MegaKind k = kinds[kind];
            const int nm = k.npl > wave ? ((k.npl - wave + MEGA_WAVES - 1) / MEGA_WAVES) * k.segs : 0;
            const float *fsc = (WT == WT_FP8 && kind != MK_HEAD) ? (const float *)lptr[l * MEGA_LPTR + 4 + kind] : nullptr;
            int c_pl = wave, c_sg = 0;                        // (local pair, segment) of the next task to fold
            int f_sg = 0;                                     // segment of the next task to multiply
            float run0 = 0.0f, run1 = 0.0f;                   // per-lane sums of the pair being walked
            auto even_round = [&](const int i) {
                // (all sums are given their zero before the first task: an element left undefined at that point
                // is filled from whatever register is at hand -- one of the other set's, whose loads are in
                // flight -- and reading it waits for those loads)
                float acc[MEGA_DEPTH][2];
#pragma unroll
                for (int s = 0; s < MEGA_DEPTH; ++s) { acc[s][0] = 0.0f; acc[s][1] = 0.0f; }
#pragma unroll
                for (int s = 0; s < MEGA_DEPTH; ++s) {
                    if (i + s < nm) {
                        const int sg = f_sg;
                        if (++f_sg == k.segs) f_sg = 0;
                        mul_task(stA[s], xs, sg, k.pieces, acc[s][0], acc[s][1]);
                        // Tasks are not interleaved: the operands of four tasks side by side take more
                        // registers than the two weight sets leave, and the scheduler would take them.
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if (i == 0) mark();
                // inside a phase the next round is requested before the sums are finished (its latency
                // overlaps them); the next phase's rounds belong to the odd phase in between
                if (i + MEGA_DEPTH < nm) issue_even();
                float fin0 = 0.0f, fin1 = 0.0f;
                int fin_p = 0, n_fin = 0;
#pragma unroll
                for (int s = 0; s < MEGA_DEPTH; ++s) {
                  if (i + s < nm) {
                    run0 += acc[s][0]; run1 += acc[s][1];
                    if (++c_sg == k.segs) {
                      // a finished pair: its two sums go to lane n_fin; the pairs of a round are finished
                      // side by side in different lanes, after the round's last task
                      const float t0 = wave_sum_dpp(run0), t1 = wave_sum_dpp(run1);
                      const float b0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t0), 63));
                      const float b1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t1), 63));
                      if (lane == n_fin) { fin0 = b0; fin1 = b1; fin_p = c_pl; }
                      ++n_fin;
                      run0 = 0.0f; run1 = 0.0f; c_sg = 0; c_pl += MEGA_WAVES;
                    }
                  }
                }
                if (lane < n_fin) {
                      float s0 = fin0, s1 = fin1;
                      const int p = fin_p;
                      {
                const int row0 = 2 * (k.pair0 + p);
                if (fsc) { s0 *= fsc[row0]; s1 *= fsc[row0 + 1]; }
                if (kind == MK_QKV) {
                    s0 *= inv; s1 *= inv;
                    if (row0 < Q + KV) {            // q and k rows: RoPE on the pair
                        const float c = ropes[2 * p], s = ropes[2 * p + 1];
                        const float e = s0 * c - s1 * s, o = s1 * c + s0 * s;
                        s0 = e; s1 = o;
                    }
                    if (row0 >= Q) {                // k and v rows enter the cache (and the exchange) in cache precision
                        const bool isk = row0 < Q + KV;
                        const int rr = isk ? row0 - Q : row0 - Q - KV;
                        void *cache = isk ? kcl : vcl;
                        if (KVBF16) {
                            const uint16_t eb = f32_to_bf16_rne(s0), ob = f32_to_bf16_rne(s1);
                            uint16_t *cp = (uint16_t *)cache + (size_t)pos * KV + rr;
                            cp[0] = eb; cp[1] = ob;
                            s0 = bf16_to_f32(eb); s1 = bf16_to_f32(ob);
                        } else {
                            // the cache keeps what the exchange delivers (stamp bit cleared), so this step and
                            // every later one attend over the same key / value bits
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
                }
            };
            // The first round is taken outside the loop: it runs straight behind the request of the odd
            // phase's weights, where it is known that set A has arrived and that only the new loads are
            // outstanding (inside the loop a refilled set A would have to be assumed, and every use of a
            // weight register would wait for all loads in flight, the other set's included).
            if (nm > 0) even_round(0);
            for (int i = MEGA_DEPTH; i < nm; i += MEGA_DEPTH) even_round(i);
        }
        mark();
        if (kind == MK_HEAD) {
            // the eight per-wave candidates meet in LDS; wave 0 publishes the workgroup's best
            wave_argbest(bv, bi);                             // (each finishing lane kept its own best)
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
        float *xs = xsb + D;
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
                // q of head h, k and v of kv-head g: three HD-float pieces of the QKV exchange vector
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
                // the PRE scores of this pass first (independent chains), then one softmax update
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
            // the slots of a wave first (lanes o apart hold the same channels of two slots), then the
            // eight per-wave partials through LDS
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
            // A split record that no workgroup fills at this position still takes this layer's stamp
            // (an empty partial: maximum -1e30, sum 0).  Consumers only read the first NS splits, but the
            // split count grows with the position: a record that had skipped launches would carry a
            // stamp of unknown age, which a consumer could take for the current one.
            if (tid < REC) {
                float *pp = a.PART + (size_t)b * REC;              // record (split b / heads, head b % heads)
                st_stamped(pp + tid, tid == HD ? -1e30f : 0.0f, par);
            }
        }

        // ---- stage this phase's input: the folded attention partials (wo) or the gate vector (w2)
        // Set A is free since the even phase's last round: the first two tasks of the next even phase go
        // out here, behind the attention (the workgroups that attend are the ones every other workgroup
        // waits for; nothing that can wait is put in front of their work).
        e_left = 0;
        if (oph + 1 <= last_ph) start_even(oph + 1);
        // (Not in front of the gate poll when the qkv phase is a single round per wave: the poll would
        // come back behind these loads, and a phase that short does not need the head start -- 600M
        // 0.522 -> 0.504 ms per token; the 5B model, whose qkv phase is several rounds, loses 3 % without
        // the early request and keeps it.)
        const bool early = !(kind == MK_W2 && qkv_one_round);
        issue_odd_lds();                                     // (needed sooner than the next even phase's tasks)
        if (early) {
            issue_even_one(ctxA, stA[0]);
            if (MEGA_DEPTH > 1) issue_even_one(ctxA, stA[1]);
        }
        {
            bool ok = true;
            if (kind == MK_WO) {
                // Thread c folds four neighbouring channels of the attention output: from every split's
                // record it polls those four sums and the record's (maximum, sum of weights), four splits
                // in flight at a time, and merges them in split order as the softmax of the whole sequence
                // would weigh them.  No staging of the records, no pass over them by a few threads, no
                // barrier before the fold.
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
                    *(float4 *)(xs + 4 * xs_chunk_pos(c, XSWZ)) = make_float4(o0 * rl, o1 * rl, o2 * rl, o3 * rl);
                }
            } else {
                const float ss = mega_poll_vec<XSWZ>(a.GATE, H, par, abortf, xs, nullptr, xresb, wo_row0, 0, pt);
                if (ss < 0.0f) ok = false;
            }
            if (!ok) s_bad = 1;
            lds_barrier();
            if (s_bad) return;
        }
        mark();
        // this phase's input and set B are here (see the even phase): the even phase behind it gets its
        // first round now
        __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0)
        if (!early) {
            issue_even_one(ctxA, stA[0]);
            if (MEGA_DEPTH > 1) issue_even_one(ctxA, stA[1]);
        }
        if (MEGA_DEPTH > 2) issue_even_one(ctxA, stA[2]);

        // ---- stream this workgroup's rows: wave w multiplies tasks w, w + 8, ... in rounds of MEGA_DEPTH_B
        // and leaves each task's two sums in LDS (the staging area of the partials is free by now)
        {
            const MegaKind k = kinds[kind];
            const int nm = k.ntasks > wave ? (k.ntasks - wave + MEGA_WAVES - 1) / MEGA_WAVES : 0;
            int f_t = wave, f_sg = wave;                     // next task and its segment
            while (f_sg >= k.segs) f_sg -= k.segs;
            // src_lds: the round's tasks come from this wave's LDS slots (q = s) instead of set B; next: request the
            // round that follows in set B
            auto odd_round = [&](const int i, const int cnt, const bool src_lds, const bool next) {
                float acc[MEGA_DEPTH_B][2];
                int slot_t[MEGA_DEPTH_B];
#pragma unroll
                for (int s = 0; s < MEGA_DEPTH_B; ++s) { acc[s][0] = 0.0f; acc[s][1] = 0.0f; slot_t[s] = 0; }
#pragma unroll
                for (int s = 0; s < MEGA_DEPTH_B; ++s) {
                    slot_t[s] = f_t;
                    if (s < cnt) {
                        if (src_lds) {
                            MegaStage<WT> tl;
                            read_lds_task(s, tl);
                            mul_task(tl, xs, f_sg, k.pieces, acc[s][0], acc[s][1]);
                        } else {
                            mul_task(stB[s], xs, f_sg, k.pieces, acc[s][0], acc[s][1]);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                        f_t += MEGA_WAVES; f_sg += MEGA_WAVES;
                        while (f_sg >= k.segs) f_sg -= k.segs;
                    }
                }
                if (i == 0) mark();
                if (next) issue_odd();
#pragma unroll
                for (int s = 0; s < MEGA_DEPTH_B; ++s) {
                    if (s < cnt) {
                        const float s0 = wave_sum_dpp(acc[s][0]), s1 = wave_sum_dpp(acc[s][1]);
                        if (lane == 63) { stage[2 * slot_t[s]] = s0; stage[2 * slot_t[s] + 1] = s1; }
                    }
                }
            };
            static_assert(MEGA_LDS_TASKS <= MEGA_DEPTH_B, "an LDS round is at most one round of set B");
            // round 0 from set B (first round outside the loop, as in the even phase); the tasks in LDS were
            // requested behind it and are multiplied behind it; set B is refilled with what follows them
            if (nm > 0) odd_round(0, min(nm, MEGA_DEPTH_B), false, MEGA_DEPTH_B + l_n < nm);
            if (l_n > 0) odd_round(MEGA_DEPTH_B, l_n, true, false);
            for (int i = MEGA_DEPTH_B + l_n; i < nm; i += MEGA_DEPTH_B) odd_round(i, min(nm - i, MEGA_DEPTH_B), false, i + MEGA_DEPTH_B < nm);
            lds_barrier();
            // thread r finishes local row r: the segments of its pair in order, scale, residual, publish
            if (tid < 2 * k.npl) {
                const int p = tid >> 1, which = tid & 1;
                float sum = 0.0f;
                for (int sg = 0; sg < k.segs; ++sg) sum += stage[2 * (p * k.segs + sg) + which];
                const int row = 2 * k.pair0 + tid;
                if (WT == WT_FP8) sum *= ((const float *)lptr[l * MEGA_LPTR + 4 + kind])[row];
                float *dstv = kind == MK_WO ? a.X2 : a.X;
                st_stamped(dstv + row, xres_r[tid] + a.alpha * sum, par);
            }
            // (the next writer of the staging area is the next attention phase or this loop's next round
            // of sums, both behind a barrier of the phases in between)
        }
        // the rest of the next even phase's first round, and (set B is free) the first task of the next odd phase
#pragma unroll
        for (int s = 3; s < MEGA_DEPTH; ++s) issue_even_one(ctxA, stA[s]);
        o_left = 0;
        if (oph + 2 <= last_ph) { start_odd(oph + 2); if (!b0_late) issue_odd_one(ctxB, stB[0]); }
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
