// A small host-side stand-in for the parts of the GPU programming model the few-row GEMM kernels use, so that
// the kernels' own source text runs on the CPU (test infrastructure: one OS thread per GPU thread, a workgroup
// at a time).  Cross-lane operations (wave shuffles, matrix instructions) meet at a per-wave barrier, which is
// sound where the kernel calls them under wave-uniform control flow, as these kernels do.
#pragma once
#include <cmath>
#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

struct uint4 { uint32_t x, y, z, w; };
struct uint2 { uint32_t x, y; };
struct dim3 { unsigned x, y, z; };
static inline uint4 make_uint4(uint32_t x, uint32_t y, uint32_t z, uint32_t w) { return uint4{x, y, z, w}; }
static inline uint2 make_uint2(uint32_t x, uint32_t y) { return uint2{x, y}; }
struct float4 { float x, y, z, w; };
struct float2 { float x, y; };
static inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
static inline float2 make_float2(float x, float y) { return float2{x, y}; }
struct pf_bf16x8 { uint16_t v[8]; };
template <class T> static inline T min(T a, T b) { return b < a ? b : a; }
template <class T> static inline T max(T a, T b) { return a < b ? b : a; }

// (the two conversions of hipdec_common.h that the kernels' helpers call)
static inline float bf16_to_f32(uint16_t h) { const uint32_t u = (uint32_t)h << 16; float f; std::memcpy(&f, &u, 4); return f; }
static inline uint16_t f32_to_bf16_rne(float f) {
    uint32_t u; std::memcpy(&u, &f, 4);
    if ((u & 0x7f800000u) == 0x7f800000u) return (uint16_t)(u >> 16);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
enum { WT_F32 = 0, WT_BF16 = 1, WT_FP8 = 2, WT_INT4 = 3 };

namespace emu {
class Barrier {
public:
    explicit Barrier(int n) : n_(n) {}
    void wait() {
        std::unique_lock<std::mutex> lk(m_);
        const unsigned gen = gen_;
        if (++count_ == n_) { count_ = 0; ++gen_; cv_.notify_all(); }
        else cv_.wait(lk, [&] { return gen_ != gen; });
    }
private:
    std::mutex m_;
    std::condition_variable cv_;
    int n_, count_ = 0;
    unsigned gen_ = 0;
};
// one lane's side of the shuffles: value n of the lane (two slots, by the parity of n), how many it has published
// and how many of them its partners have read
struct ShuffleBox {
    float val[2] = {0.0f, 0.0f};
    std::atomic<uint64_t> published{0}, consumed[2] = {{0}, {0}};   // consumed: reads of the values a slot has held
    uint64_t count = 0;                                  // (touched by the owning lane only)
};
struct Wave {
    Barrier bar{64};
    uint32_t a[64][4], b[64][4];
    ShuffleBox box[64];
};
struct Block {
    // the dynamic LDS is a heap block of exactly the size the launch asked for: under AddressSanitizer an access past
    // it is reported like one past any other buffer
    explicit Block(int threads, size_t lds_bytes) : bar(threads), waves((threads + 63) / 64), lds((unsigned char *)std::malloc(lds_bytes ? lds_bytes : 1)) {}
    ~Block() { std::free(lds); }
    Barrier bar;
    std::vector<Wave> waves;
    unsigned char *lds;
};
inline thread_local dim3 tl_thread, tl_block, tl_grid, tl_blockdim;
inline thread_local Block *tl_blk = nullptr;
inline Wave &wave() { return tl_blk->waves[tl_thread.x >> 6]; }
inline int lane() { return (int)(tl_thread.x & 63); }
inline uint16_t *lds() { return (uint16_t *)tl_blk->lds; }
inline void sync_block() { tl_blk->bar.wait(); }
inline float bf16_to_float(uint16_t h) { const uint32_t u = (uint32_t)h << 16; float f; std::memcpy(&f, &u, 4); return f; }
inline float uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
// A shuffle is a rendezvous of the two lanes that exchange, not of the wave: the kernels also shuffle inside
// branches that only some lane groups of a wave take (every lane's partner takes the same branch, so the two run
// the same sequence of shuffles).  Lane l publishes its n-th value, waits for its partner's n-th, reads it and
// says so; it reuses a slot only after every value the slot has held has been read (reads of different values can
// finish out of order: their readers are different lanes).
inline float shfl_xor(float v, int mask, int) {
    Wave &w = wave();
    ShuffleBox &mine = w.box[lane()], &theirs = w.box[lane() ^ mask];
    const uint64_t n = ++mine.count;
    while (mine.consumed[n & 1].load(std::memory_order_acquire) < (n - 1) / 2) std::this_thread::yield();   // the slot's earlier values
    mine.val[n & 1] = v;
    mine.published.store(n, std::memory_order_release);
    while (theirs.published.load(std::memory_order_acquire) < n) std::this_thread::yield();
    const float r = theirs.val[n & 1];
    theirs.consumed[n & 1].fetch_add(1, std::memory_order_release);
    return r;
}
inline int shfl_xor(int v, int mask, int width) {
    float f; std::memcpy(&f, &v, 4);
    f = shfl_xor(f, mask, width);                        // (bits only: nothing is computed on the way)
    std::memcpy(&v, &f, 4);
    return v;
}
// v_perm_b32: result byte i is byte sel[i] of the eight bytes {s0 (4..7), s1 (0..3)}
inline uint32_t perm(uint32_t s0, uint32_t s1, uint32_t sel) {
    const uint64_t both = ((uint64_t)s0 << 32) | s1;
    uint32_t r = 0;
    for (int i = 0; i < 4; ++i) {
        const unsigned pick = (sel >> (8 * i)) & 0xff;
        r |= (uint32_t)((both >> (8 * (pick & 7))) & 0xff) << (8 * i);     // (selectors above 7 are not used by these kernels)
    }
    return r;
}
// v_mfma_f32_16x16x32_bf16: D = A (16 x 32) . B (32 x 16) + C.  Lane l supplies row l % 16 of A and column
// l % 16 of B, reduction elements 8 * (l / 16) .. + 7 of each; register r of lane l holds D[4 * (l / 16) + r][l % 16].
template <class V4>
inline V4 mfma_16x16x32_bf16(pf_bf16x8 a, pf_bf16x8 b, V4 c, int, int, int) {
    Wave &w = wave();
    const int l = lane();
    std::memcpy(w.a[l], a.v, 16);
    std::memcpy(w.b[l], b.v, 16);
    w.bar.wait();
    V4 d = c;
    for (int r = 0; r < 4; ++r) {
        const int i = 4 * (l / 16) + r, j = l % 16;
        double s = 0.0;
        for (int k = 0; k < 32; ++k) {
            const uint16_t *ar = (const uint16_t *)w.a[(k / 8) * 16 + i], *br = (const uint16_t *)w.b[(k / 8) * 16 + j];
            s += (double)bf16_to_float(ar[k % 8]) * (double)bf16_to_float(br[k % 8]);
        }
        d[r] = (float)((double)c[r] + s);
    }
    w.bar.wait();
    return d;
}
// OCP e4m3fn -> float (exact): 1 sign, 4 exponent bits (bias 7), 3 mantissa bits; exponent 0 is subnormal
inline float e4m3_to_float(uint8_t b) {
    const int e = (b >> 3) & 15, m = b & 7;
    float v;
    if (e == 15 && m == 7) v = std::nanf("");
    else if (e == 0) v = std::ldexp((float)m, -9);
    else v = std::ldexp(1.0f + (float)m / 8.0f, e - 7);
    return (b & 0x80) ? -v : v;
}
struct bf16x2 { uint16_t v[2]; };
// v_cvt_scalef32_pk_bf16_fp8: bytes 0, 1 (hi = false) or 2, 3 (hi = true) of src as two bf16 numbers times scale
inline bf16x2 cvt_scalef32_pk_bf16_fp8(uint32_t src, float scale, bool hi) {
    bf16x2 r;
    for (int i = 0; i < 2; ++i) {
        const float f = e4m3_to_float((uint8_t)(src >> (8 * ((hi ? 2 : 0) + i)))) * scale;
        uint32_t u;
        std::memcpy(&u, &f, 4);
        r.v[i] = (uint16_t)(u >> 16);                      // every e4m3 number is a bf16 number: nothing is rounded away
    }
    return r;
}
// v_mfma_f32_32x32x16_bf16: D = A (32 x 16) . B (16 x 32) + C.  Lane l supplies row l % 32 of A and column l % 32
// of B, reduction elements 8 * (l / 32) .. + 7 of each; register i of lane l holds
// D[8 * (i / 4) + 4 * (l / 32) + i % 4][l % 32].
template <class V16>
inline V16 mfma_32x32x16_bf16(pf_bf16x8 a, pf_bf16x8 b, V16 c, int, int, int) {
    Wave &w = wave();
    const int l = lane();
    std::memcpy(w.a[l], a.v, 16);
    std::memcpy(w.b[l], b.v, 16);
    w.bar.wait();
    V16 d = c;
    for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r / 4) + 4 * (l / 32) + r % 4, j = l % 32;
        double s = 0.0;
        for (int k = 0; k < 16; ++k) {
            const uint16_t *ar = (const uint16_t *)w.a[(k / 8) * 32 + i], *br = (const uint16_t *)w.b[(k / 8) * 32 + j];
            s += (double)bf16_to_float(ar[k % 8]) * (double)bf16_to_float(br[k % 8]);
        }
        d[r] = (float)((double)c[r] + s);
    }
    w.bar.wait();
    return d;
}
// v_mfma_f32_32x32x16_f16: the same tile shape and lane layout with fp16 operands
template <class H8, class V16>
inline V16 mfma_32x32x16_f16(H8 a, H8 b, V16 c, int, int, int) {
    Wave &w = wave();
    const int l = lane();
    std::memcpy(w.a[l], &a, 16);
    std::memcpy(w.b[l], &b, 16);
    w.bar.wait();
    V16 d = c;
    for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r / 4) + 4 * (l / 32) + r % 4, j = l % 32;
        double s = 0.0;
        for (int k = 0; k < 16; ++k) {
            _Float16 x, y;
            std::memcpy(&x, (const uint16_t *)w.a[(k / 8) * 32 + i] + k % 8, 2);
            std::memcpy(&y, (const uint16_t *)w.b[(k / 8) * 32 + j] + k % 8, 2);
            s += (double)(float)x * (double)(float)y;
        }
        d[r] = (float)((double)c[r] + s);
    }
    w.bar.wait();
    return d;
}
typedef __fp16 f16x2 __attribute__((ext_vector_type(2)));
// v_cvt_pkrtz_f16_f32: two floats as packed fp16, rounded toward zero (the kernels only pass values fp16 holds exactly)
inline f16x2 cvt_pkrtz(float a, float b) {
    auto rtz = [](float f) { _Float16 h = (_Float16)f; if (std::fabs((float)h) > std::fabs(f)) { uint16_t u; std::memcpy(&u, &h, 2); --u; std::memcpy(&h, &u, 2); } return h; };
    const _Float16 x = rtz(a), y = rtz(b);
    f16x2 r;
    std::memcpy(&r, &x, 2);
    std::memcpy((char *)&r + 2, &y, 2);
    return r;
}
typedef float f32x2 __attribute__((ext_vector_type(2)));
// v_cvt_pk_f32_fp8: bytes 0, 1 (hi = false) or 2, 3 (hi = true) of src as two floats
inline f32x2 cvt_pk_f32_fp8(uint32_t src, bool hi) {
    f32x2 r;
    for (int i = 0; i < 2; ++i) r[i] = e4m3_to_float((uint8_t)(src >> (8 * ((hi ? 2 : 0) + i))));
    return r;
}
// v_cvt_off_f32_i4: the low four bits as a two's complement number, over 16
inline float cvt_off_f32_i4(int x) { int n = x & 15; if (n >= 8) n -= 16; return (float)n / 16.0f; }
inline uint32_t float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
// runs body() as every thread of every workgroup of the grid, one workgroup after the other
template <class F>
inline void launch_fn(F body, dim3 grid, unsigned threads, size_t lds_bytes) {
    for (unsigned bz = 0; bz < grid.z; ++bz)
        for (unsigned by = 0; by < grid.y; ++by)
            for (unsigned bx = 0; bx < grid.x; ++bx) {
                Block blk((int)threads, lds_bytes);
                std::vector<std::thread> ts;
                ts.reserve(threads);
                for (unsigned t = 0; t < threads; ++t)
                    ts.emplace_back([&, t] {
                        tl_thread = dim3{t, 0, 0}; tl_block = dim3{bx, by, bz}; tl_grid = grid; tl_blockdim = dim3{threads, 1, 1}; tl_blk = &blk;
                        body();
                    });
                for (auto &th : ts) th.join();
            }
}
template <class K, class A>
inline void launch(K kernel, dim3 grid, unsigned threads, size_t lds_bytes, const A &args) {
    launch_fn([&] { kernel(args); }, grid, threads, lds_bytes);
}
}  // namespace emu

#define __global__
#define __device__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define threadIdx emu::tl_thread
#define blockIdx emu::tl_block
#define gridDim emu::tl_grid
#define blockDim emu::tl_blockdim
#define WAVE 64
#define __syncthreads() emu::sync_block()
#define __shfl_xor(v, m, w) emu::shfl_xor((v), (m), (w))
#define __uint_as_float(u) emu::uint_as_float(u)
#define __expf(x) expf(x)
#define __threadfence() std::atomic_thread_fence(std::memory_order_seq_cst)
#define __host__
// single-rounding float operations (the programs that use them are built with floating-point contraction off)
#define __fadd_rn(a, b) ((float)(a) + (float)(b))
#define __fsub_rn(a, b) ((float)(a) - (float)(b))
#define __fmul_rn(a, b) ((float)(a) * (float)(b))
#define __fdiv_rn(a, b) ((float)(a) / (float)(b))
#define __float_as_int(f) ((int)emu::float_as_uint(f))
// (workgroups run one after the other here, so "the last workgroup to arrive" is the last of the grid)
static inline unsigned atomicAdd(unsigned *p, unsigned v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
#define __builtin_amdgcn_perm(a, b, s) emu::perm((a), (b), (s))
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) emu::mfma_16x16x32_bf16((a), (b), (c), (x), (y), (z))
#define __shared__ static
#define __float_as_uint(f) emu::float_as_uint(f)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) emu::mfma_32x32x16_bf16((a), (b), (c), (x), (y), (z))
#define __builtin_amdgcn_cvt_pk_f32_fp8(s, h) emu::cvt_pk_f32_fp8((s), (h))
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) emu::mfma_32x32x16_f16((a), (b), (c), (x), (y), (z))
#define __builtin_amdgcn_cvt_pkrtz(a, b) emu::cvt_pkrtz((a), (b))
#define __builtin_amdgcn_cvt_off_f32_i4(x) emu::cvt_off_f32_i4(x)
#define __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(s, f, h) emu::cvt_scalef32_pk_bf16_fp8((s), (f), (h))
#define PF_REG_CONST_S(var, lit) var = lit
#define PF_REG_CONST_V(var, lit) var = lit
// (the wave reduction of hipdec_common.h: xor shuffles over 32 .. 1)
static inline float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
