// Prefill contraction Y[M,N] = X[M,K] . dequant(W)^T on the matrix cores (gfx950 MFMA, fp16 in / f32 out).
//
// Roofline: for M >= 64 this is a dense contraction bounded by MFMA throughput, not by HBM.  The weights
// stay in their raw GGUF blocks; a wave reads the bytes of its 32 weight rows straight from global memory
// one 256-element super-block ahead, expands them to fp16 in registers (four vector operations per pair of
// elements, issued behind the matrix instructions) and feeds v_mfma_f32_32x32x16_f16.  Dequantized weights
// never touch LDS or HBM.
//
// Operands
//   A = 32 weight rows x 16 k   (expanded in registers)
//   B = 16 k x 32 tokens        (X, fp16, brought to LDS in 64-k tiles by LDS-DMA loads, ring of 4 stages)
//   D = 32 rows x 32 tokens f32 (16 registers per lane)
// The k order inside a tile is whatever falls out of the cheapest nibble expansion; X is laid out in the
// same order by the pre-pass, so nothing is shuffled in the inner loop:
//   tile element E(s, h, e) = 32*(s>>1) + 16*h + 8*(s&1) + {0,2,1,3,4,6,5,7}[e]
//   for MFMA step s = 0..3, lane half h = lane/32, register element e = 0..7.
//
// fp16 range: activations of a transformer can exceed 65504, so the pre-pass scales every row of X by a
// power of two that brings its largest magnitude into [2^14, 2^15) (exact) and the epilogue multiplies it
// back.  Nibbles enter fp16 as 1 + q/16 (bit pattern 0x3C00 | q << 6, exact); the weight is then
//   w = ((1 + q/16) - 1) * (16*d*sc) - dmin*m   (packed subtract, exact, then one packed fma).
//
// Work split: a wave owns 32 weight rows x (32*MF) tokens -- the expansion of a weight element is shared by
// MF matrix instructions, which is what keeps the vector ALU under the matrix pipe; a workgroup is NW such
// waves side by side along n, two waves per SIMD so that one wave's loads, barriers and scale preparation
// hide behind the other's matrix instructions.  When the tiles would leave CUs idle the k range is split
// across workgroups on super-block boundaries; the splits write partial tiles to a workspace and a second
// kernel adds them (no floating-point atomics: across XCDs they are served by memory, not by L2).
#include "rt_device.h"

#include <algorithm>
#include <atomic>
#include <type_traits>
#include <cstring>

namespace rt {

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));


constexpr int kBK = 64;          // k per tile
constexpr int kMaxSplit = 8;     // most k splits of one launch

// ---- pre-pass: X f32 [M,K] -> fp16, row-scaled, k-permuted; inv_scale[m] undoes the row scale.
// One workgroup per row; output chunk g (8 halves) is the aligned group of 8 floats at
// 64*(g>>3) + 32*(s>>1) + 16*h + 8*(s&1) with s = (g&7)>>1, h = g&1, its elements in the order 0,2,1,3,4,6,5,7.
// A thread keeps its (up to kXprepChunks) groups in registers between the maximum and the conversion, so the
// row is read once; longer rows take the groups beyond that from memory again.
constexpr int kXprepChunks = 6;
__global__ __launch_bounds__(256) void xprep_kernel(const float *X, size_t K, _Float16 *Xp, float *inv_scale) {
    __shared__ float red[4];
    const size_t m = blockIdx.x;
    const float *x = X + m * K;
    const size_t n_chunks = K / 8;
    auto src_of = [](size_t g) {
        const int sh = (int)(g & 7), s = sh >> 1, h = sh & 1;
        return 64 * (g >> 3) + 32 * (size_t)(s >> 1) + 16 * (size_t)h + 8 * (size_t)(s & 1);
    };
    float4 lo[kXprepChunks], hi[kXprepChunks];
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < kXprepChunks; j++) {
        const size_t g = threadIdx.x + 256 * (size_t)j;
        if (g < n_chunks) {
            const float4 *p = reinterpret_cast<const float4 *>(x + src_of(g));
            lo[j] = p[0];
            hi[j] = p[1];
            amax = fmaxf(amax, fmaxf(fmaxf(fmaxf(fabsf(lo[j].x), fabsf(lo[j].y)), fmaxf(fabsf(lo[j].z), fabsf(lo[j].w))),
                                     fmaxf(fmaxf(fabsf(hi[j].x), fabsf(hi[j].y)), fmaxf(fabsf(hi[j].z), fabsf(hi[j].w)))));
        }
    }
    for (size_t g = threadIdx.x + 256 * (size_t)kXprepChunks; g < n_chunks; g += 256) {
        const float4 *p = reinterpret_cast<const float4 *>(x + src_of(g));
        const float4 a = p[0], b = p[1];
        amax = fmaxf(amax, fmaxf(fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))),
                                 fmaxf(fmaxf(fabsf(b.x), fabsf(b.y)), fmaxf(fabsf(b.z), fabsf(b.w)))));
    }
    amax = block_max(amax, red);
    int e = 0;
    float scale = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        (void)frexpf(amax, &e);                 // amax = f * 2^e, f in [0.5, 1)
        int se = 15 - e;
        se = se > 100 ? 100 : (se < -100 ? -100 : se);
        scale = ldexpf(1.f, se);
        inv = ldexpf(1.f, -se);
    }
    if (threadIdx.x == 0) inv_scale[m] = inv;
    auto emit = [&](size_t g, const float4 &a, const float4 &b) {
        half8v o = { (_Float16)(a.x * scale), (_Float16)(a.z * scale), (_Float16)(a.y * scale), (_Float16)(a.w * scale),
                     (_Float16)(b.x * scale), (_Float16)(b.z * scale), (_Float16)(b.y * scale), (_Float16)(b.w * scale) };
        *reinterpret_cast<half8v *>(Xp + m * K + 8 * g) = o;
    };
#pragma unroll
    for (int j = 0; j < kXprepChunks; j++) {
        const size_t g = threadIdx.x + 256 * (size_t)j;
        if (g < n_chunks) emit(g, lo[j], hi[j]);
    }
    for (size_t g = threadIdx.x + 256 * (size_t)kXprepChunks; g < n_chunks; g += 256) {
        const float4 *p = reinterpret_cast<const float4 *>(x + src_of(g));
        emit(g, p[0], p[1]);
    }
}

// ---- the pre-pass fused with the operation that produces the activation matrix.  A thread keeps its groups of the
// row in registers from the first read to the conversion: rows of up to THREADS * kXprepChunks * 8 elements
// (12 288 with 256 threads, 49 152 with 1024).
__device__ __forceinline__ void plane_load8(const PlaneSum &p, size_t off, float *v) {
    const float4 a = *reinterpret_cast<const float4 *>(p.base + off), b = *reinterpret_cast<const float4 *>(p.base + off + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    for (int z = 1; z < p.n; z++) {
        const float4 c = *reinterpret_cast<const float4 *>(p.base + (size_t)z * p.stride + off),
                     d = *reinterpret_cast<const float4 *>(p.base + (size_t)z * p.stride + off + 4);
        v[0] += c.x; v[1] += c.y; v[2] += c.z; v[3] += c.w; v[4] += d.x; v[5] += d.y; v[6] += d.z; v[7] += d.w;
    }
}

struct RowSrc {
    PlaneSum a, b;          // rmsnorm: a = the matrix; swiglu: a = gate, b = up
    const float *res;       // rmsnorm: added to a (optional)
    float *x_out;           // rmsnorm: a + res is stored here (optional)
    const float *gamma;
    float eps;
};

constexpr int kPrepRms = 1, kPrepSwiglu = 2;

template <int MODE, int THREADS>
__global__ __launch_bounds__(THREADS) void xprep_fused_kernel(RowSrc S, size_t K, _Float16 *Xp, float *inv_scale) {
    __shared__ float red[THREADS / 64];
    const size_t m = blockIdx.x, n_chunks = K / 8;
    auto src_of = [](size_t g) {
        const int sh = (int)(g & 7), s = sh >> 1, h = sh & 1;
        return 64 * (g >> 3) + 32 * (size_t)(s >> 1) + 16 * (size_t)h + 8 * (size_t)(s & 1);
    };
    float v[kXprepChunks][8];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kXprepChunks; j++) {
        const size_t g = threadIdx.x + THREADS * (size_t)j;
        if (g < n_chunks) {
            const size_t off = m * K + src_of(g);
            if (MODE == kPrepRms) {
                plane_load8(S.a, off, v[j]);
                if (S.res) {
                    const float4 a = *reinterpret_cast<const float4 *>(S.res + off), b = *reinterpret_cast<const float4 *>(S.res + off + 4);
                    v[j][0] += a.x; v[j][1] += a.y; v[j][2] += a.z; v[j][3] += a.w; v[j][4] += b.x; v[j][5] += b.y; v[j][6] += b.z; v[j][7] += b.w;
                }
                if (S.x_out) {
                    *reinterpret_cast<float4 *>(S.x_out + off) = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
                    *reinterpret_cast<float4 *>(S.x_out + off + 4) = make_float4(v[j][4], v[j][5], v[j][6], v[j][7]);
                }
#pragma unroll
                for (int e = 0; e < 8; e++) ss += v[j][e] * v[j][e];
            } else {
                float gt[8], up[8];
                plane_load8(S.a, off, gt);
                plane_load8(S.b, off, up);
#pragma unroll
                for (int e = 0; e < 8; e++) v[j][e] = up[e] * (gt[e] * (1.0f / (1.0f + expf(-gt[e]))));
            }
        }
    }
    if (MODE == kPrepRms) {
        ss = block_sum(ss, red);
        const float rms = sqrtf(ss / (float)K + S.eps);
#pragma unroll
        for (int j = 0; j < kXprepChunks; j++) {
            const size_t g = threadIdx.x + THREADS * (size_t)j;
            if (g < n_chunks) {
                const float *gp = S.gamma + src_of(g);
                const float4 a = *reinterpret_cast<const float4 *>(gp), b = *reinterpret_cast<const float4 *>(gp + 4);
                const float gm[8] = { a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w };
#pragma unroll
                for (int e = 0; e < 8; e++) v[j][e] = gm[e] * (v[j][e] / rms);
            }
        }
    }
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < kXprepChunks; j++) {
        const size_t g = threadIdx.x + THREADS * (size_t)j;
        if (g < n_chunks)
#pragma unroll
            for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[j][e]));
    }
    amax = block_max(amax, red);
    int ex = 0;
    float scale = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        (void)frexpf(amax, &ex);                // amax = f * 2^ex, f in [0.5, 1)
        int se = 15 - ex;
        se = se > 100 ? 100 : (se < -100 ? -100 : se);
        scale = ldexpf(1.f, se);
        inv = ldexpf(1.f, -se);
    }
    if (threadIdx.x == 0) inv_scale[m] = inv;
#pragma unroll
    for (int j = 0; j < kXprepChunks; j++) {
        const size_t g = threadIdx.x + THREADS * (size_t)j;
        if (g < n_chunks) {
            half8v o = { (_Float16)(v[j][0] * scale), (_Float16)(v[j][2] * scale), (_Float16)(v[j][1] * scale), (_Float16)(v[j][3] * scale),
                         (_Float16)(v[j][4] * scale), (_Float16)(v[j][6] * scale), (_Float16)(v[j][5] * scale), (_Float16)(v[j][7] * scale) };
            *reinterpret_cast<half8v *>(Xp + m * K + 8 * g) = o;
        }
    }
}

// ---- weights of one super-block (256 k) on their way to the lanes that expand them
//
// MFMA lane (nl, h) needs bytes of weight row nl only, and rows lie row_bytes apart: loading them lane by
// lane touches 32 cache lines per instruction and the address path becomes the bottleneck.  So a wave fetches
// its 32 row-blocks as consecutive 16-byte chunks (chunk c = 64 i + lane of instruction i; the chunks of one
// row-block are adjacent in memory), parks them in a wave-private LDS area at 16 c, and every lane reads its
// row's pieces back.  LDS operations of one wave execute in order, so no barrier is involved.
template <int TYPE> struct WGeo;
template <> struct WGeo<RT_GGML_Q4_K> {
    static constexpr int blk = 144, chunks = 9, loads = 5, tail = 0, reads = 5, stage_bytes = 32 * 144;
};
template <> struct WGeo<RT_GGML_Q6_K> {   // 13 whole chunks (208 bytes) + the 2-byte d, parked behind the rows
    static constexpr int blk = 210, chunks = 13, loads = 7, tail = 1, reads = 8, stage_bytes = 32 * 208 + 32 * 4;
};

template <int TYPE> struct WTmp { u32x4 c[WGeo<TYPE>::loads]; uint32_t tail; };

// per-lane byte offsets (from the weight row of the wave's first row) of the chunk each load instruction fetches
template <int TYPE> struct WOff { uint32_t c[WGeo<TYPE>::loads]; uint32_t tail; };

template <int TYPE>
__device__ __forceinline__ void make_woff(WOff<TYPE> &o, int lane, int rows_left, size_t row_bytes) {
    using G = WGeo<TYPE>;
#pragma unroll
    for (int i = 0; i < G::loads; i++) {
        const int c = 64 * i + lane, row = c / G::chunks, part = c - row * G::chunks;
        o.c[i] = (uint32_t)(min(row, rows_left - 1) * row_bytes) + 16u * part;     // rows past the matrix repeat its last row
    }
    o.tail = (uint32_t)(min(lane & 31, rows_left - 1) * row_bytes) + 208u;
}

// global load OP of WGeo::loads + WGeo::tail of the chunks of super-block sb
template <int TYPE, int OP>
__device__ __forceinline__ void load_op(WTmp<TYPE> &r, const WOff<TYPE> &o, const uint8_t *base, int lane) {
    using G = WGeo<TYPE>;
    // Written as assembly so that the compiler keeps no book on them: with LDS-DMA loads in flight its own
    // wait before the first use would be "all vector memory operations", i.e. the X tile requested last.
    // The waits that cover these loads are the vmcnt waits of superblock().
    if constexpr (OP < G::loads) {
        if (64 * OP + lane < 32 * G::chunks)
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r.c[OP]) : "v"(base + o.c[OP]) : "memory");
    } else {
        if (lane < 32) asm volatile("global_load_ushort %0, %1, off" : "=v"(r.tail) : "v"(base + o.tail) : "memory");
    }
}

// LDS accesses and their waits are written by hand: with LDS-DMA loads in the same loop the compiler's own
// wait insertion falls back to "wait for everything" before each use, which exposes the full LDS latency
// every other step.  LDS operations return in order, so "at most n outstanding" pins which have completed.
template <int OFF> __device__ __forceinline__ half8v lds_read16(uint32_t addr) {
    half8v r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
template <int OFF> __device__ __forceinline__ u32x4 lds_read16u(uint32_t addr) {
    u32x4 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
template <int OFF> __device__ __forceinline__ uint32_t lds_read4(uint32_t addr) {
    uint32_t r;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
template <int OFF> __device__ __forceinline__ void lds_write16(uint32_t addr, u32x4 v) {
    asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <int OFF> __device__ __forceinline__ void lds_write4(uint32_t addr, uint32_t v) {
    asm volatile("ds_write_b32 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <int N> __device__ __forceinline__ void wait_lgkmcnt_c() {
    static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit counter");
    __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));
}
// s_waitcnt that only constrains the vector-memory counter (gfx9 encoding: vmcnt in bits 3:0 and 15:14;
// lgkmcnt = 15 and expcnt = 7 mean no constraint).
template <int N> __device__ __forceinline__ void wait_vmcnt_c() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// compile-time loop: f(std::integral_constant<int, I>) for I = B .. E-1 (indices stay constants, so the
// register-resident structs below are never addressed dynamically)
template <int B, int E, class F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// park the fetched chunks: lane's chunk of instruction i goes to 16 * (64 i + lane); operation OP of
// WGeo::loads + WGeo::tail (every lane of the wave issues each of them, partly masked)
template <int TYPE, int OP>
__device__ __forceinline__ void park_op(const WTmp<TYPE> &r, uint32_t wpark, int lane) {
    using G = WGeo<TYPE>;
    if constexpr (OP < G::loads) {
        if (64 * OP + lane < 32 * G::chunks) lds_write16<1024 * OP>(wpark, r.c[OP]);
    } else {
        if (lane < 32) lds_write4<32 * 208>(wpark - 12u * (uint32_t)lane, r.tail);     // 16 lane - 12 lane = 4 lane
    }
}
template <int TYPE> struct WParkOps { static constexpr int n = WGeo<TYPE>::loads + WGeo<TYPE>::tail; };

// ---- raw weight bytes of one lane (weight row nl, k half h) for one super-block
template <int TYPE> struct WSb;
template <> struct WSb<RT_GGML_Q4_K> { u32x4 hdr; u32x4 qs[4]; };                 // d|dmin, 12 scale bytes; 16 bytes per 64-k tile
template <> struct WSb<RT_GGML_Q6_K> { u32x4 A[2], B[2], H[2], sc; uint32_t d; };  // per 128-k half: ql[l], ql[l+32], qh[l]

// Read-back operation OP of WGeo::reads; la.wrow is the LDS address of this lane's row-block in the wave's
// area, wrow_h the same + 16 h for the half-dependent pieces.  The order is the order of first use: what the
// constants need (OP 0 / 0..1), then tile 0, then the rest.
template <int OP> __device__ __forceinline__ void fetch_op(WSb<RT_GGML_Q4_K> &w, uint32_t wrow, uint32_t wrow_h, uint32_t) {
    if constexpr (OP == 0) w.hdr = lds_read16u<0>(wrow);
    else w.qs[OP - 1] = lds_read16u<16 + 32 * (OP - 1)>(wrow_h);
}
template <int OP> __device__ __forceinline__ void fetch_op(WSb<RT_GGML_Q6_K> &w, uint32_t wrow, uint32_t wrow_h, uint32_t wtail) {
    if constexpr (OP == 0) w.d = lds_read4<0>(wtail);
    else if constexpr (OP == 1) w.sc = lds_read16u<192>(wrow);
    else if constexpr (OP == 2) w.A[0] = lds_read16u<0>(wrow_h);
    else if constexpr (OP == 3) w.H[0] = lds_read16u<128>(wrow_h);
    else if constexpr (OP == 4) w.B[0] = lds_read16u<32>(wrow_h);
    else if constexpr (OP == 5) w.A[1] = lds_read16u<64>(wrow_h);
    else if constexpr (OP == 6) w.B[1] = lds_read16u<96>(wrow_h);
    else w.H[1] = lds_read16u<160>(wrow_h);
}

__device__ __forceinline__ half2v splat(float f) {
    _Float16 v = (_Float16)f;
    return half2v{ v, v };
}
__device__ __forceinline__ half2v splat_h(_Float16 v) { return half2v{ v, v }; }
__device__ __forceinline__ half2v as_h2(uint32_t u) { return __builtin_bit_cast(half2v, u); }
__device__ __forceinline__ _Float16 h_bits(uint32_t u) { return __builtin_bit_cast(_Float16, (uint16_t)u); }
// (v & m) | g in one instruction; g lives in a vector register, m in a scalar one
__device__ __forceinline__ uint32_t and_or(uint32_t v, uint32_t m, uint32_t g) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(m), "v"(g));
    return r;
}
// Keeps the computation of v where it is written: without it the optimizer sinks work whose result is only
// needed after the loop branch into the next iteration, i.e. out from behind the matrix instructions.
template <class T> __device__ __forceinline__ void pin(T &v) { asm volatile("" : "+v"(v)); }

// Exponent patterns of the in-place integer -> fp16 conversion, kept in vector registers (operands of
// v_and_or_b32).  A field of an fp16 mantissa under the exponent 2^E reads as 2^E + field * 2^(E-10):
//   Q4_K: nibble n at bits 3:0 under 2^6 is 64 + n/16, at bits 7:4 under 2^2 it is 4 + n/16;
//   Q6_K: 6-bit v at bits 5:0 under 2^4 is 16 + v/64.
struct ExpPat { uint32_t lo, hi; };

// Per-super-block constants of one lane's weight row: everything of the expansion that does not depend on the
// MFMA step.  One register holds the pair the two halves of a tile need; the fma picks the half.  They are
// computed in kPrepPieces small pieces so that the work can be placed behind matrix instructions of the
// previous super-block; the trailing fields are intermediates shared by the pieces.
template <int TYPE> struct SbK;
template <> struct SbK<RT_GGML_Q4_K> {
    half2v a[4], c[4];   // tile t: (16*d*sc, -dmin*m) of sub-blocks 2t (low nibbles) and 2t+1 (high nibbles)
    uint32_t sc_lo, sc_hi, m_lo, m_hi;
    half2v d16, nmin;
};
template <> struct SbK<RT_GGML_Q6_K> {
    half2v a[4];         // tile t: 64*d*sc of the tile's two 16-element runs of this lane
    half2v d64;
};
constexpr int kPrepPieces = 9;

// bytes i and i+1 (i = 0 or 2) of v as two exact fp16 numbers: one byte permute builds 0x6400 | b = 1024 + b
__device__ __forceinline__ half2v byte_pair(uint32_t v, int i) {
    return as_h2(__builtin_amdgcn_perm(0x64646464u, v, i ? 0x04030402u : 0x04010400u)) - splat(1024.f);
}

__device__ __forceinline__ void prep_piece(SbK<RT_GGML_Q4_K> &k, const WSb<RT_GGML_Q4_K> &w, int, int piece) {
    if (piece == 0) {
        const uint32_t y = w.hdr.y, z = w.hdr.z, x = w.hdr.w;
        k.sc_lo = y & 0x3f3f3f3fu;
        k.m_lo = z & 0x3f3f3f3fu;
        k.sc_hi = (x & 0x0f0f0f0fu) | ((y >> 2) & 0x30303030u);
        k.m_hi = ((x >> 4) & 0x0f0f0f0fu) | ((z >> 2) & 0x30303030u);
        // fp16 products of an 11-bit and a 6-bit number round once: the same value as the f32 product rounded to fp16
        k.d16 = splat_h(h_bits(w.hdr.x & 0xFFFF)) * splat(16.f);
        k.nmin = -splat_h(h_bits(w.hdr.x >> 16));
        pin(k.sc_lo); pin(k.m_lo); pin(k.sc_hi); pin(k.m_hi); pin(k.d16); pin(k.nmin);
    } else {
        const int i = piece - 1, t = i >> 1;
        if (i & 1) {
            k.c[t] = byte_pair(t < 2 ? k.m_lo : k.m_hi, 2 * (t & 1)) * k.nmin;
            pin(k.c[t]);
        } else {
            k.a[t] = byte_pair(t < 2 ? k.sc_lo : k.sc_hi, 2 * (t & 1)) * k.d16;
            pin(k.a[t]);
        }
    }
}

// Packed pair u (k slots 2u, 2u+1 of this lane's row) of the fp16 A operand for MFMA step s of tile t.
// A step's operand is four such pairs; they are produced one at a time so that each can be issued behind
// one matrix instruction.  w = (n/16) * (16*d*sc) - dmin*m: the subtraction of the exponent's 2^E is exact, so
// the only roundings are those of the scale, of the offset and of the final fma.
// The three dependent operations of a pair are separate stages (bits -> fp16 with the exponent, exact subtraction
// of the exponent's value, scale and offset), so that the caller can interleave the stages of different pairs:
// two dependent vector operations issued back to back cost a wait state each.
__device__ __forceinline__ uint32_t expand_s1(const WSb<RT_GGML_Q4_K> &w, const SbK<RT_GGML_Q4_K> &, int t, int s, int u, ExpPat G) {
    const int hi = s >> 1;
    const u32x4 qs = w.qs[t];
    const uint32_t q = (s & 1) ? ((u & 2) ? qs.w : qs.z) : ((u & 2) ? qs.y : qs.x);
    // pair u & 1 = 0 takes bytes 0 and 2 of the word, pair 1 bytes 1 and 3 (one shift brings them down)
    const uint32_t src = (u & 1) ? (q >> 8) : q;
    return hi ? and_or(src, 0x00F000F0u, G.hi) : and_or(src, 0x000F000Fu, G.lo);
}
__device__ __forceinline__ half2v expand_s2(const SbK<RT_GGML_Q4_K> &, uint32_t x, int, int s) {
    return as_h2(x) - ((s >> 1) ? splat(4.f) : splat(64.f));
}
__device__ __forceinline__ half2v expand_s3(const SbK<RT_GGML_Q4_K> &k, half2v y, int t, int s) {
    const int hi = s >> 1;
    return y * splat_h(k.a[t][hi]) + splat_h(k.c[t][hi]);
}

__device__ __forceinline__ void prep_piece(SbK<RT_GGML_Q6_K> &k, const WSb<RT_GGML_Q6_K> &w, int h, int piece) {
    // tile t = 2*hf + p: half hf of the super-block, runs 2p and 2p+1 of that half; of a run's 32 elements this
    // lane holds 16 with scale index 2*run + h among the half's 8 scales, i.e. bytes h and h+2 of word 2*hf + p
    if (piece == 0) {
        k.d64 = splat_h(h_bits(w.d)) * splat(64.f);
        pin(k.d64);
    } else if (piece <= 4) {
        const int t = piece - 1;
        // int8 b -> fp16: 0x6400 | (b ^ 0x80) is 1024 + b + 128
        const uint32_t v = __builtin_amdgcn_perm(0x64646464u, w.sc[t] >> (8 * h), 0x04020400u) ^ 0x00800080u;
        k.a[t] = (as_h2(v) - splat(1152.f)) * k.d64;
        pin(k.a[t]);
    }
}

__device__ __forceinline__ uint32_t expand_s1(const WSb<RT_GGML_Q6_K> &w, const SbK<RT_GGML_Q6_K> &, int t, int s, int u, ExpPat G) {
    const int hf = t >> 1, p = t & 1, j = s >> 1, tt = s & 1;
    const u32x4 L = j ? w.B[hf] : w.A[hf];    // run parity = j: even runs read ql[l], odd runs ql[l + 32]
    const u32x4 H = w.H[hf];
    const uint32_t l = tt ? ((u & 2) ? L.w : L.z) : ((u & 2) ? L.y : L.x);
    const uint32_t hq = tt ? ((u & 2) ? H.w : H.z) : ((u & 2) ? H.y : H.x);
    // 6-bit values, one per byte: nibble of ql (low for p = 0, high for p = 1), two bits of qh at 2*(2p + j)
    const uint32_t lo = (p ? (l >> 4) : l) & 0x0f0f0f0fu;
    const int shh = 2 * (2 * p + j);
    const uint32_t hb = shh <= 4 ? (hq << (4 - shh)) : (hq >> (shh - 4));
    const uint32_t v = (hb & 0x30303030u) | lo;
    const uint32_t src = (u & 1) ? (v >> 8) : v;
    return and_or(src, 0x003F003Fu, G.lo);
}
// 16 + v/64 minus 16.5 is (v - 32)/64 exactly, so w = 64*d*sc * (v - 32)/64 carries only the rounding of the
// scale and of the product
__device__ __forceinline__ half2v expand_s2(const SbK<RT_GGML_Q6_K> &, uint32_t x, int, int) { return as_h2(x) - splat(16.5f); }
__device__ __forceinline__ half2v expand_s3(const SbK<RT_GGML_Q6_K> &k, half2v y, int t, int s) { return y * splat_h(k.a[t][s >> 1]); }

template <int TYPE>
__device__ __forceinline__ half2v expand_unit(const WSb<TYPE> &w, const SbK<TYPE> &k, int t, int s, int u, ExpPat G) {
    return expand_s3(k, expand_s2(k, expand_s1(w, k, t, s, u, G), t, s), t, s);
}

template <int TYPE>
__device__ __forceinline__ half8v expand_step(const WSb<TYPE> &w, const SbK<TYPE> &k, int t, int s, ExpPat G) {
    half2v r0 = expand_unit(w, k, t, s, 0, G), r1 = expand_unit(w, k, t, s, 1, G), r2 = expand_unit(w, k, t, s, 2, G),
           r3 = expand_unit(w, k, t, s, 3, G);
    return half8v{ r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1] };
}

// LDS addresses a lane works with
struct LaneLds {
    uint32_t b[4];       // B fragment of step s (stage and fragment go into the instruction's offset field)
    uint32_t wpark;      // where this lane parks chunk 0 (wave area + 16 lane)
    uint32_t wrow, wrow_h, wtail;   // its row-block in the wave area, the same + 16 h, its Q6_K d
};

// One super-block (256 k = 4 tiles x 4 MFMA steps) of a wave's 32 rows x 32*MF tokens, as one software
// pipeline: every step issues, in this pinned order, the LDS reads of the next step's B fragments, then MF
// times { matrix instruction; one slice of the next step's A expansion; one slice of other work }.
// "Next step" crosses tile and super-block borders, so the matrix pipe never waits for an operand:
//   - the last step of the super-block expands from the next super-block's bytes (wn) with its constants (kn);
//   - those bytes were requested from global memory at the top of this super-block (tmp), are parked in LDS
//     and read back by their lanes in the last step of tile 2, and the constants are prepared, a piece per
//     slot, during tile 3;
//   - the barrier that publishes X tile t+1 sits in the middle of tile t (before step 2), so the LDS reads
//     of its first fragments are covered by steps 2 and 3.
//
// X tiles (BM rows x 64 k, fp16) go from global memory straight into a ring of 4 LDS stages with 16-byte
// LDS-DMA loads; since a split starts on a super-block boundary, tile t of every super-block lives in stage
// t.  The load of tile kt+3 is issued right after the barrier in tile kt: by then every wave has left tile
// kt-1, whose stage it overwrites.  LDS stage: row m holds 8 chunks of 16 bytes, chunk c at position
// c ^ ((m >> 1) & 7), so that the 16 lanes that read the same chunk index of 16 consecutive rows fall on
// distinct banks.
//
// Vector-memory operations complete in order, so "at most n outstanding" pins which have landed.  Issue order
// per super-block: weights of the next super-block (WL loads) at the top, one X tile (XI loads) after each
// barrier.  At the barrier of tile t the operations younger than X tile kt+1 are X tile kt+2 and, for
// t < 2, the weight prefetch.  Past the end of the k range the same loads are issued for the last tile /
// super-block again (the data is not used), which keeps the counts -- and the code -- uniform.
// Slices of work that ride along with the steps of a super-block (t = tile, s = step), all compile-time:
//   global loads of the next super-block's chunks: tile 0, steps 0 and 1 (before that tile's barrier)
//   parking them in LDS:                            tile 2, steps 2 and 3 (after the wait that proves they landed)
//   reading them back per lane:                     from tile 2 step 3 on, two per step, in order of first use
template <int TYPE> struct Ride {
    using G = WGeo<TYPE>;
    static constexpr int n_load = G::loads + G::tail, n_park = n_load, n_fetch = G::reads;
    static constexpr int half_load = (n_load + 1) / 2, half_park = (n_park + 1) / 2;
    static constexpr int load_lo(int t, int s) { return t == 0 && s == 0 ? 0 : (t == 0 && s == 1 ? half_load : n_load); }
    static constexpr int load_hi(int t, int s) { return t == 0 && s == 0 ? half_load : n_load; }
    static constexpr int park_lo(int t, int s) { return t == 2 && s == 2 ? 0 : (t == 2 && s == 3 ? half_park : n_park); }
    static constexpr int park_hi(int t, int s) { return t == 2 && s == 2 ? half_park : n_park; }
    // first read-back slot is (2,3); slot index = 4*(t-2) + s - 3
    static constexpr int fetch_lo(int t, int s) { int k = 4 * (t - 2) + s - 3; return k < 0 ? n_fetch : (2 * k < n_fetch ? 2 * k : n_fetch); }
    static constexpr int fetch_hi(int t, int s) { int k = 4 * (t - 2) + s - 3; return k < 0 ? n_fetch : (2 * k + 2 < n_fetch ? 2 * k + 2 : n_fetch); }
};

// (stage, pair) in issue order, three per matrix instruction at MF = 4, six at MF = 2
constexpr int kExpandOrder[12][2] = { {1, 0}, {1, 1}, {1, 2}, {1, 3}, {2, 0}, {2, 1}, {2, 2}, {2, 3}, {3, 0}, {3, 1}, {3, 2}, {3, 3} };

template <int TYPE, int MF, int XI, class IssueX>
__device__ __forceinline__ void superblock(float16v (&acc)[MF], const WSb<TYPE> &w, const SbK<TYPE> &k, WTmp<TYPE> &tmp,
                                           const WOff<TYPE> &woff, const uint8_t *wnext, WSb<TYPE> &wn, SbK<TYPE> &kn, half8v &a,
                                           half8v (&bb)[2][MF], const LaneLds &la, int lane, int h, ExpPat G, int kt, int kt_last,
                                           IssueX issue_x) {
    using Geo = WGeo<TYPE>;
    using R = Ride<TYPE>;
    constexpr int WL = Geo::loads + Geo::tail;
    static_assert(12 % MF == 0, "the stage operations are dealt evenly over the matrix instructions");
    constexpr int PPS = (kPrepPieces + 2 * MF - 1) / (2 * MF);   // preparation pieces per slot of tile 3, steps 1 and 2
    constexpr int kStageBytes = 32 * MF * kBK * 2;
    static_for<0, 4>([&](auto T) {
        constexpr int t = decltype(T)::value;
        static_for<0, 4>([&](auto S) {
            constexpr int s = decltype(S)::value;
            constexpr int cur = s & 1, nxt = cur ^ 1;             // 16 steps per super-block: the parity carries over
            if constexpr (s == 2) {
                wait_vmcnt_c<(t < 2 ? XI + WL : XI)>();
                __builtin_amdgcn_s_barrier();
            }
            // the X tile three ahead, one load instruction per step from the barrier on (spreads the burst of
            // the eight waves over the address path)
            if constexpr (s >= 2 && s - 2 < XI) issue_x(min(kt + t + 3, kt_last), (t + 3) & 3, s - 2);
            static_for<R::load_lo(t, s), R::load_hi(t, s)>([&](auto O) { load_op<TYPE, decltype(O)::value>(tmp, woff, wnext, lane); });
            constexpr int tn = s < 3 ? t : t + 1, sn = (s + 1) & 3;   // tn == 4: tile 0 of the next super-block
            half2v an[4];
            static_for<R::park_lo(t, s), R::park_hi(t, s)>([&](auto O) { park_op<TYPE, decltype(O)::value>(tmp, la.wpark, lane); });
            static_for<0, MF>([&](auto I) {
                constexpr int i = decltype(I)::value;
                bb[nxt][i] = lds_read16<(tn & 3) * kStageBytes + i * 32 * kBK * 2>(la.b[sn]);
            });
            static_for<R::fetch_lo(t, s), R::fetch_hi(t, s)>([&](auto O) { fetch_op<decltype(O)::value>(wn, la.wrow, la.wrow_h, la.wtail); });
            wait_lgkmcnt_c<MF + R::fetch_hi(t, s) - R::fetch_lo(t, s)>();
            __builtin_amdgcn_sched_barrier(0);
            uint32_t ex[4];
            half2v ey[4];
            // stage g (1 bits, 2 subtraction, 3 scale) of pair q of the next step's operand
            auto stage = [&](auto Gc, auto Qc) {
                constexpr int g = decltype(Gc)::value, q = decltype(Qc)::value;
                if constexpr (tn < 4) {
                    if constexpr (g == 1) { ex[q] = expand_s1(w, k, tn, sn, q, G); pin(ex[q]); }
                    else if constexpr (g == 2) { ey[q] = expand_s2(k, ex[q], tn, sn); pin(ey[q]); }
                    else { an[q] = expand_s3(k, ey[q], tn, sn); pin(an[q]); }
                } else {
                    if constexpr (g == 1) { ex[q] = expand_s1(wn, kn, 0, 0, q, G); pin(ex[q]); }
                    else if constexpr (g == 2) { ey[q] = expand_s2(kn, ex[q], 0, 0); pin(ey[q]); }
                    else { an[q] = expand_s3(kn, ey[q], 0, 0); pin(an[q]); }
                }
            };
            static_for<0, MF>([&](auto J) {
                constexpr int j = decltype(J)::value;
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bb[cur][j], a, acc[j], 0, 0, 0);
                // The 12 stage operations of the four pairs are dealt over the MF slots in the order of
                // kExpandOrder: three other operations lie between an operation and the one that depends on it.
                static_for<j * (12 / MF), (j + 1) * (12 / MF)>([&](auto I) {
                    constexpr int i = decltype(I)::value;
                    stage(std::integral_constant<int, kExpandOrder[i][0]>{}, std::integral_constant<int, kExpandOrder[i][1]>{});
                });
                if constexpr (t == 3 && (s == 1 || s == 2)) {
                    constexpr int p0 = ((s - 1) * MF + j) * PPS, p1 = p0 + PPS < kPrepPieces ? p0 + PPS : kPrepPieces;
                    static_for<p0, p1>([&](auto P) { prep_piece(kn, wn, h, decltype(P)::value); });
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            a = half8v{ an[0][0], an[0][1], an[1][0], an[1][1], an[2][0], an[2][1], an[3][0], an[3][1] };
        });
    });
}

// Grid: 1-D and XCD-aware.  Tiles are ordered by (m-tile, k-split) "slab" first, n-tile second; workgroup b
// runs on XCD b % 8 (round-robin dispatch), and XCD x is given a contiguous run of that order, so the
// workgroups that share an L2 share an X slab and the slab is read from HBM once.
// Y_out: Y itself (ksplit == 1; res, when given, is added) or the first of ksplit partial planes of
// plane_stride floats each.
// LDS: [4 stages][BM][64] fp16 of X, then NW wave-private areas of WGeo::stage_bytes.
template <int TYPE, int NW, int MF>
__global__ __launch_bounds__(64 * NW) void qgemm_kernel(const uint8_t *W, size_t row_bytes, int N, int K, const _Float16 *Xp,
                                                        const float *inv_scale, int M, float *Y_out, size_t plane_stride,
                                                        const float *res, int sb_per_split, int ksplit, int tiles_n,
                                                        int n_tiles_total, int per_xcd, const uint8_t *W2, float *Y2, int tiles_one) {
    using Geo = WGeo<TYPE>;
    constexpr int BM = 32 * MF, BN = 32 * NW, XI = BM / 8 / NW;
    static_assert(XI >= 1 && XI * 8 * NW == BM, "every wave issues whole 8-row LDS-DMA loads");
    constexpr int kStageHalves = BM * kBK;   // halves per stage (no padding: swizzled)
    RT_DYN_LDS(_Float16, xs);
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, nl = lane & 31, h = lane >> 5;
    // tile of this workgroup
    int t = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || t >= n_tiles_total) return;
    // a second weight matrix of the same shape against the same X (q and k, gate and up): its tiles follow the first one's
    if (t >= tiles_one) {
        t -= tiles_one;
        W = W2;
        Y_out = Y2;
    }
    const int slab = t / tiles_n, nt = t - slab * tiles_n;
    const int mt = slab / ksplit, kz = slab - mt * ksplit;
    const int n0 = nt * BN, m0 = mt * BM;
    const int sb0 = kz * sb_per_split, sb1 = min(K / 256, sb0 + sb_per_split);
    if (sb0 >= sb1) return;      // the launcher sizes the splits so that none is empty

    // weights: the wave's first row (clamped into the matrix) and the per-lane chunk offsets from it
    const int wrow0 = min(n0 + wave * 32, N - 1);
    const uint8_t *wbase = W + (size_t)wrow0 * row_bytes;
    WOff<TYPE> woff;
    make_woff(woff, lane, N - wrow0, row_bytes);

    // LDS-DMA: instruction i of this wave fills LDS rows (wave*XI + i)*8 .. +8 of a stage; lane L lands at
    // row + L/8, position L%8, which must hold chunk (L%8) ^ ((row >> 1) & 7) of that X row.
    const _Float16 *xsrc[XI];
#pragma unroll
    for (int i = 0; i < XI; i++) {
        int row = (wave * XI + i) * 8 + (lane >> 3);
        int c = (lane & 7) ^ ((row >> 1) & 7);
        xsrc[i] = Xp + (size_t)min(m0 + row, M - 1) * K + 8 * c;
    }
    auto issue_x = [&](int kt, int st, int i) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xsrc[i] + (size_t)kt * kBK),
                                         (__attribute__((address_space(3))) void *)(xs + (size_t)st * kStageHalves + (size_t)(wave * XI + i) * 8 * kBK),
                                         16, 0, 0);
    };

    float16v acc[MF];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.f;

    // B fragments: lane (token nl of fragment i, half h) reads chunk 2s+h of stage row i*32 + nl
    LaneLds la;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) _Float16 *)xs;
#pragma unroll
    for (int sn = 0; sn < 4; sn++) la.b[sn] = lds0 + (uint32_t)nl * (kBK * 2) + 16u * (uint32_t)((2 * sn + h) ^ ((nl >> 1) & 7));
    const uint32_t warea = lds0 + 4u * kStageHalves * 2u + (uint32_t)wave * Geo::stage_bytes;
    la.wpark = warea + 16u * (uint32_t)lane;
    la.wrow = warea + (uint32_t)nl * (16u * Geo::chunks);
    la.wrow_h = la.wrow + 16u * (uint32_t)h;
    la.wtail = warea + 32u * 208u + 4u * (uint32_t)nl;
    ExpPat G;
    if (TYPE == RT_GGML_Q4_K) {
        asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(G.lo));
        asm volatile("v_mov_b32 %0, 0x44004400" : "=v"(G.hi));
    } else {
        asm volatile("v_mov_b32 %0, 0x4c004c00" : "=v"(G.lo));
        G.hi = 0;
    }

    // prologue: three X tiles and the first super-block's weights in flight, constants and operands of step 0
    const int kt0 = 4 * sb0, kt_last = 4 * sb1 - 1;
    WTmp<TYPE> tmp;
    WSb<TYPE> wA, wB;
    SbK<TYPE> kA, kB;
    static_for<0, Ride<TYPE>::n_load>([&](auto O) { load_op<TYPE, decltype(O)::value>(tmp, woff, wbase + (size_t)sb0 * Geo::blk, lane); });
#pragma unroll
    for (int d = 0; d < 3; d++)
#pragma unroll
        for (int i = 0; i < XI; i++) issue_x(min(kt0 + d, kt_last), d, i);
    wait_vmcnt_c<3 * XI>();                // the weights have landed, the X tiles may still be in flight
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, Ride<TYPE>::n_park>([&](auto O) { park_op<TYPE, decltype(O)::value>(tmp, la.wpark, lane); });
    static_for<0, Ride<TYPE>::n_fetch>([&](auto O) { fetch_op<decltype(O)::value>(wA, la.wrow, la.wrow_h, la.wtail); });
    wait_lgkmcnt_c<0>();
    __builtin_amdgcn_sched_barrier(0);     // the scheduler does not know that the wait guards wA
    static_for<0, kPrepPieces>([&](auto P) { prep_piece(kA, wA, h, decltype(P)::value); });
    half8v a = expand_step(wA, kA, 0, 0, G), bb[2][MF];
    wait_vmcnt_c<2 * XI>();                // this wave's part of X tile 0
    __builtin_amdgcn_s_barrier();
    static_for<0, MF>([&](auto I) { bb[0][decltype(I)::value] = lds_read16<decltype(I)::value * 32 * kBK * 2>(la.b[0]); });

    for (int sb = sb0;;) {
        superblock<TYPE, MF, XI>(acc, wA, kA, tmp, woff, wbase + (size_t)min(sb + 1, sb1 - 1) * Geo::blk, wB, kB, a, bb, la, lane, h, G,
                                 4 * sb, kt_last, issue_x);
        if (++sb >= sb1) break;
        superblock<TYPE, MF, XI>(acc, wB, kB, tmp, woff, wbase + (size_t)min(sb + 1, sb1 - 1) * Geo::blk, wA, kA, a, bb, la, lane, h, G,
                                 4 * sb, kt_last, issue_x);
        if (++sb >= sb1) break;
    }
    // The last step leaves loads in flight (X tiles past the end of the range into this workgroup's LDS, and
    // the LDS reads of the operands of a step that does not follow).  Their destination registers are dead
    // to the compiler, which would hand them to the code below while the data is still on its way.
    wait_vmcnt_c<0>();
    wait_lgkmcnt_c<0>();
    __builtin_amdgcn_sched_barrier(0);

    // X fragments are the first operand, so D = X . W^T: register r of lane L holds token 8*(r/4) + 4*(L/32) + r%4
    // of the fragment and weight row L % 32.  A store instruction then writes two runs of 32 consecutive floats.
    float *Yp = Y_out + (size_t)kz * plane_stride;
    const int n = n0 + wave * 32 + nl;
    const bool add_res = res && ksplit == 1;
    // the scales of the lane's tokens, four consecutive ones per load (the array is padded past M)
    float4 inv[MF][4];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int mb = m0 + i * 32 + 8 * g + 4 * h;
            inv[i][g] = mb < M ? *reinterpret_cast<const float4 *>(inv_scale + mb) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    auto scaled = [&](int i, int r) {
        const float4 q = inv[i][r >> 2];
        return acc[i][r] * ((r & 3) == 0 ? q.x : (r & 3) == 1 ? q.y : (r & 3) == 2 ? q.z : q.w);
    };
    if (m0 + BM <= M && n0 + BN <= N) {
        // whole tile inside the matrix: no per-element guards, so the stores go out back to back (a guard is a
        // branch, and behind a branch the compiler waits for every earlier store before the next one)
        float *yp = Yp + (size_t)(m0 + 4 * h) * N + n;
        if (add_res) {
            const float *rp = res + (size_t)(m0 + 4 * h) * N + n;
#pragma unroll
            for (int i = 0; i < MF; i++) {
                float rv[16];
#pragma unroll
                for (int r = 0; r < 16; r++) rv[r] = rp[(size_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * N];
#pragma unroll
                for (int r = 0; r < 16; r++) yp[(size_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * N] = scaled(i, r) + rv[r];
            }
        } else {
#pragma unroll
            for (int i = 0; i < MF; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) yp[(size_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * N] = scaled(i, r);
        }
    } else if (n < N) {
        __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0): the scales, before the guarded stores
#pragma unroll
        for (int i = 0; i < MF; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m >= M) continue;
                float v = scaled(i, r);
                if (add_res) v += res[(size_t)m * N + n];
                Yp[(size_t)m * N + n] = v;
            }
        }
    }
}

// Y = sum of the partial planes (+ res)
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *P, size_t plane_stride, int ksplit, const float *res, float *Y, size_t n4) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
        float4 a = reinterpret_cast<const float4 *>(P)[i];
        for (int z = 1; z < ksplit; z++) {
            float4 b = reinterpret_cast<const float4 *>(P + (size_t)z * plane_stride)[i];
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        if (res) {
            float4 b = reinterpret_cast<const float4 *>(res)[i];
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        reinterpret_cast<float4 *>(Y)[i] = a;
    }
}

struct GemmPlan { int mf, ksplit, sb_per_split; };

constexpr int kGemmWaves = 8;     // waves per workgroup: two per SIMD, one workgroup per CU

// Shape of the launch: token fragments per wave (tile 32*mf tokens x 256 rows) and k splits.
GemmPlan gemm_plan(size_t M, size_t N, size_t K, int matrices = 1) {
    GemmPlan p;
    p.mf = M > 64 ? 4 : 2;
    const size_t bm = 32 * (size_t)p.mf, nsb = K / 256;
    const size_t tiles = (size_t)matrices * ((M + bm - 1) / bm) * ((N + 32 * kGemmWaves - 1) / (32 * kGemmWaves));
    // split k while that fills more of the 256 CUs in whole rounds and leaves every split at least two super-blocks
    p.ksplit = 1;
    while (tiles * p.ksplit * 2 <= 256 && nsb / (p.ksplit * 2) >= 2 && p.ksplit < kMaxSplit) p.ksplit *= 2;
    p.sb_per_split = (int)((nsb + p.ksplit - 1) / p.ksplit);
    p.ksplit = (int)((nsb + p.sb_per_split - 1) / p.sb_per_split);     // no empty split
    return p;
}

template <int TYPE, int NW, int MF>
hipError_t launch_cfg(hipStream_t s, const GemmPlan &p, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const _Float16 *Xp,
                      const float *inv_scale, size_t M, float *Y, const float *res, float *partial, bool reduce, const uint8_t *w2 = nullptr,
                      float *planes2 = nullptr) {
    constexpr int BM = 32 * MF, BN = 32 * NW;
    const size_t lds = (size_t)4 * BM * kBK * sizeof(_Float16) + (size_t)NW * WGeo<TYPE>::stage_bytes;
    auto kern = qgemm_kernel<TYPE, NW, MF>;
    // Per instantiation and device (the attribute belongs to the function as loaded on a device).  Only a cache of "already
    // asked": setting the attribute twice is harmless, so two threads that both find the flag clear just both set it.
    static std::atomic<bool> attr_set[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    if (lds > 64 * 1024 && !attr_set[dev].load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set[dev].store(true, std::memory_order_release);
    }
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    const int one = tiles_m * p.ksplit * tiles_n, total = w2 ? 2 * one : one;
    const int per_xcd = (total + 7) / 8;
    const size_t plane = M * N;
    kern<<<dim3((unsigned)(8 * per_xcd)), 64 * NW, lds, s>>>(w, row_bytes, (int)N, (int)K, Xp, inv_scale, (int)M, p.ksplit > 1 ? partial : Y,
                                                             plane, res, p.sb_per_split, p.ksplit, tiles_n, total, per_xcd, w2, planes2, one);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || p.ksplit == 1 || !reduce) return e;
    const size_t n4 = plane / 4;
    const unsigned grid = (unsigned)std::min<size_t>((n4 + 255) / 256, 2048);
    splitk_reduce_kernel<<<grid, 256, 0, s>>>(partial, plane, p.ksplit, res, Y, n4);
    return hipGetLastError();
}

template <int TYPE>
hipError_t launch_type(hipStream_t s, const GemmPlan &p, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const _Float16 *Xp,
                       const float *inv_scale, size_t M, float *Y, const float *res, float *partial, bool reduce = true,
                       const uint8_t *w2 = nullptr, float *planes2 = nullptr) {
    if (p.mf == 4) return launch_cfg<TYPE, kGemmWaves, 4>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial, reduce, w2, planes2);
    return launch_cfg<TYPE, kGemmWaves, 2>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial, reduce, w2, planes2);
}

// 3..15 rows of X against Q4_K / Q6_K: too few for the 16-row tiles of the fused contraction, enough for the integer
// matrix-core GEMV, eight rows per launch.
bool few_rows_on_matrix_cores(int type, size_t M, size_t N, size_t K) {
    return M >= (size_t)kGemvMbMinBatch && M < 16 && qgemv_mb_serves(type, N, K, (int)std::min<size_t>(M, 8));
}

bool mfma_path(int type, size_t N, size_t K, size_t M) {
    return (type == RT_GGML_Q4_K || type == RT_GGML_Q6_K) && M >= 16 && K % 256 == 0 && N % 4 == 0;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace


// workspace: fp16 X, one f32 per row of X, and the partial planes of a k-split launch
bool qgemm_on_matrix_cores(int type, size_t M, size_t N, size_t K) { return mfma_path(type, N, K, M); }

size_t qgemm_scratch_bytes(int type, size_t M, size_t N, size_t K) {
    if (!mfma_path(type, N, K, M)) {
        if (hgemm_serves(type, M, N, K)) return hgemm_scratch_bytes(type, M, N, K);
        return few_rows_on_matrix_cores(type, M, N, K) ? qgemv_mb_scratch_bytes(K) : 0;
    }
    GemmPlan p = gemm_plan(M, N, K);
    return align256(M * K * sizeof(_Float16)) + align256(M * sizeof(float)) + (p.ksplit > 1 ? (size_t)p.ksplit * M * N * sizeof(float) : 0);
}

size_t qgemm_planes_bytes(int type, size_t M, size_t N, size_t K) {
    if (!mfma_path(type, N, K, M)) return 0;
    return (size_t)gemm_plan(M, N, K).ksplit * M * N * sizeof(float);
}

hipError_t launch_xprep(hipStream_t s, const float *X, size_t M, size_t K, _Float16 *Xp, float *inv_scale) {
    if (M == 0 || K == 0 || K % 256 != 0) return hipErrorInvalidValue;
    xprep_kernel<<<dim3((unsigned)M), 256, 0, s>>>(X, K, Xp, inv_scale);
    return hipGetLastError();
}

hipError_t launch_xprep_rmsnorm(hipStream_t s, PlaneSum in, const float *res, float *x_out, const float *gamma, float eps, size_t M, size_t K,
                                _Float16 *Xp, float *inv_scale) {
    if (M == 0 || K == 0 || K % 256 != 0 || K > kXprepFusedMaxK || in.n < 1 || !in.base || !gamma) return hipErrorInvalidValue;
    RowSrc S{ in, PlaneSum{ nullptr, 0, 0 }, res, x_out, gamma, eps };
    if (K <= 256 * kXprepChunks * 8) xprep_fused_kernel<kPrepRms, 256><<<dim3((unsigned)M), 256, 0, s>>>(S, K, Xp, inv_scale);
    else xprep_fused_kernel<kPrepRms, 1024><<<dim3((unsigned)M), 1024, 0, s>>>(S, K, Xp, inv_scale);
    return hipGetLastError();
}

hipError_t launch_xprep_swiglu(hipStream_t s, PlaneSum gate, PlaneSum up, size_t M, size_t K, _Float16 *Xp, float *inv_scale) {
    if (M == 0 || K == 0 || K % 256 != 0 || K > kXprepFusedMaxK || gate.n < 1 || up.n < 1 || !gate.base || !up.base) return hipErrorInvalidValue;
    RowSrc S{ gate, up, nullptr, nullptr, nullptr, 0.f };
    if (K <= 256 * kXprepChunks * 8) xprep_fused_kernel<kPrepSwiglu, 256><<<dim3((unsigned)M), 256, 0, s>>>(S, K, Xp, inv_scale);
    else xprep_fused_kernel<kPrepSwiglu, 1024><<<dim3((unsigned)M), 1024, 0, s>>>(S, K, Xp, inv_scale);
    return hipGetLastError();
}

// The contraction alone: Xp / inv_scale come from one of the pre-pass launches above, the k splits stay as planes.
hipError_t launch_qgemm_planes(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const _Float16 *Xp,
                               const float *inv_scale, size_t M, float *planes, size_t planes_bytes, PlaneSum *out) {
    if (!mfma_path(type, N, K, M) || !out) return hipErrorInvalidValue;
    const GemmPlan p = gemm_plan(M, N, K);
    if ((size_t)p.ksplit * M * N * sizeof(float) > planes_bytes) return hipErrorInvalidValue;
    *out = PlaneSum{ planes, M * N, p.ksplit };
    if (type == RT_GGML_Q4_K) return launch_type<RT_GGML_Q4_K>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, planes, nullptr, planes, false);
    return launch_type<RT_GGML_Q6_K>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, planes, nullptr, planes, false);
}

// Two weight matrices of one shape and format against the same prepared X in one launch (q and k, gate and up): the tiles of
// both fill the CUs together, so k is split less than for either alone.
hipError_t launch_qgemm_planes2(hipStream_t s, int type, const uint8_t *wa, const uint8_t *wb, size_t N, size_t K, size_t row_bytes,
                                const _Float16 *Xp, const float *inv_scale, size_t M, float *planes_a, float *planes_b, size_t planes_bytes,
                                PlaneSum *out_a, PlaneSum *out_b) {
    if (!mfma_path(type, N, K, M) || !out_a || !out_b || !wa || !wb) return hipErrorInvalidValue;
    const GemmPlan p = gemm_plan(M, N, K, 2);
    if ((size_t)p.ksplit * M * N * sizeof(float) > planes_bytes) return hipErrorInvalidValue;
    *out_a = PlaneSum{ planes_a, M * N, p.ksplit };
    *out_b = PlaneSum{ planes_b, M * N, p.ksplit };
    if (type == RT_GGML_Q4_K)
        return launch_type<RT_GGML_Q4_K>(s, p, wa, N, K, row_bytes, Xp, inv_scale, M, planes_a, nullptr, planes_a, false, wb, planes_b);
    return launch_type<RT_GGML_Q6_K>(s, p, wa, N, K, row_bytes, Xp, inv_scale, M, planes_a, nullptr, planes_a, false, wb, planes_b);
}

hipError_t launch_plane_sum(hipStream_t s, PlaneSum in, const float *res, float *Y, size_t n) {
    if (n == 0 || n % 4 != 0 || in.n < 1) return hipErrorInvalidValue;
    const size_t n4 = n / 4;
    const unsigned grid = (unsigned)std::min<size_t>((n4 + 255) / 256, 2048);
    splitk_reduce_kernel<<<grid, 256, 0, s>>>(in.base, in.stride, in.n, res, Y, n4);
    return hipGetLastError();
}

// res (optional) is added to the result; it may be Y itself only on the row-by-row path.
// x_prepared: the workspace still holds the pre-pass of this very X (same M and K) from the previous call, as
// when several weights meet one activation matrix; the pre-pass is then skipped.
hipError_t launch_qgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes,
                        const float *X, size_t M, float *Y, const float *res, void *scratch, size_t scratch_bytes, bool x_prepared) {
    if (mfma_path(type, N, K, M) && res != Y) {
        if (scratch_bytes < qgemm_scratch_bytes(type, M, N, K)) return hipErrorInvalidValue;
        const GemmPlan p = gemm_plan(M, N, K);
        char *base = reinterpret_cast<char *>(scratch);
        _Float16 *Xp = reinterpret_cast<_Float16 *>(base);
        float *inv_scale = reinterpret_cast<float *>(base + align256(M * K * sizeof(_Float16)));
        float *partial = reinterpret_cast<float *>(base + align256(M * K * sizeof(_Float16)) + align256(M * sizeof(float)));
        if (!x_prepared) {
            xprep_kernel<<<dim3((unsigned)M), 256, 0, s>>>(X, K, Xp, inv_scale);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
        }
        if (type == RT_GGML_Q4_K) return launch_type<RT_GGML_Q4_K>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial);
        return launch_type<RT_GGML_Q6_K>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial);
    }
    // formats without a fused contraction: the fp16 matrix-core kernel over an fp16 copy of the weights
    if (hgemm_serves(type, M, N, K) && scratch_bytes >= hgemm_scratch_bytes(type, M, N, K))
        return launch_hgemm(s, type, w, N, K, row_bytes, X, M, Y, res, scratch, scratch_bytes);
    if (few_rows_on_matrix_cores(type, M, N, K) && scratch_bytes >= qgemv_mb_scratch_bytes(K) && ((uintptr_t)scratch & 255) == 0) {
        for (size_t m0 = 0; m0 < M; m0 += 8) {
            const int b = (int)std::min<size_t>(8, M - m0);
            const float *r = res ? res + m0 * N : nullptr;
            hipError_t e;
            if (b >= kGemvMbMinBatch) {
                e = launch_qgemv_mb(s, type, w, row_bytes, N, K, X + m0 * K, b, Y + m0 * N, r, scratch);
            } else {
                GemvArgs a;
                memset(&a, 0, sizeof a);
                a.n = 1;
                a.p[0].w = w; a.p[0].x = X + m0 * K; a.p[0].stage = kStageF32; a.p[0].y = Y + m0 * N; a.p[0].res = r;
                a.p[0].row_bytes = row_bytes; a.p[0].type = type; a.p[0].N = (int)N; a.p[0].K = (int)K;
                e = launch_qgemv(s, a, b);
            }
            if (e != hipSuccess) return e;
        }
        return hipSuccess;
    }
    // Row-by-row form (few rows, in-place residual of the fused contraction): the GEMV kernel, one grid slice per row of X.
    GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = 1;
    a.p[0].w = w; a.p[0].x = X; a.p[0].stage = kStageF32; a.p[0].y = Y; a.p[0].res = res; a.p[0].row_bytes = row_bytes;
    a.p[0].type = type; a.p[0].N = (int)N; a.p[0].K = (int)K;
    return launch_qgemv(s, a, (int)M);
}

}  // namespace rt
