// Device-side helpers shared by the kernel translation units (gfx950, wave64).
#pragma once

#include "rt_internal.h"

#include <hip/hip_fp16.h>

// The launch-sized LDS region of a kernel.  A CPU build of the device code (bounds / race checking) predefines
// this macro to hand out its own per-workgroup buffer.
#ifndef RT_DYN_LDS
#define RT_DYN_LDS(T, name) extern __shared__ T name[]
#endif

namespace rt {


__device__ __forceinline__ float h2f(uint32_t bits16) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)bits16);
}
__device__ __forceinline__ uint16_t f2h_rne(float f) {
    return __builtin_bit_cast(unsigned short, (_Float16)f);
}

// Loads through a byte pointer with no alignment promise (Q6_K / Q8_0 / Q4_0 blocks are only 2-byte aligned).
__device__ __forceinline__ uint4 ld16u(const uint8_t *p) { uint4 v; __builtin_memcpy(&v, p, 16); return v; }
__device__ __forceinline__ uint2 ld8u(const uint8_t *p) { uint2 v; __builtin_memcpy(&v, p, 8); return v; }
__device__ __forceinline__ uint32_t ld4u(const uint8_t *p) { uint32_t v; __builtin_memcpy(&v, p, 4); return v; }
__device__ __forceinline__ uint32_t ld2u(const uint8_t *p) { unsigned short v; __builtin_memcpy(&v, p, 2); return v; }
__device__ __forceinline__ uint4 ld16a(const uint8_t *p) { return *reinterpret_cast<const uint4 *>(p); }

__device__ __forceinline__ int sdot4(uint32_t a, int b, int c) { return __builtin_amdgcn_sdot4((int)a, b, c, false); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Block-wide sum / max through LDS (red must hold blockDim/64 floats). All threads get the result.
__device__ __forceinline__ float block_sum(float v, float *red) {
    v = wave_sum(v);
    int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; i++) t += red[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float *red) {
    v = wave_max(v);
    int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nw; i++) t = fmaxf(t, red[i]);
    return t;
}


// --------------------------------------------------------- exact block decode
// One element of a tensor row, evaluated exactly as the block definition is written
// (f32, no contraction), so a dump of these values can be memcmp'd against the CPU decode.
#pragma clang fp contract(off)
__device__ inline float deq_elem(int type, const uint8_t *row, size_t col) {
    switch (type) {
    case RT_GGML_F32: { float f; __builtin_memcpy(&f, row + 4 * col, 4); return f; }
    case RT_GGML_F16: return h2f(ld2u(row + 2 * col));
    case RT_GGML_Q8_0: {
        const uint8_t *b = row + 34 * (col >> 5);
        float d = h2f(ld2u(b));
        return d * (float)(int)(int8_t)b[2 + (col & 31)];
    }
    case RT_GGML_Q8_1: {       // { f16 d; f16 s; i8 qs[32] }: s = d * sum(qs) serves integer dot products and is not part of a value
        const uint8_t *b = row + 36 * (col >> 5);
        float d = h2f(ld2u(b));
        return d * (float)(int)(int8_t)b[4 + (col & 31)];
    }
    case RT_GGML_Q4_0: {
        const uint8_t *b = row + 18 * (col >> 5);
        float d = h2f(ld2u(b));
        int j = (int)(col & 31);
        int q = j < 16 ? (b[2 + j] & 0x0F) : (b[2 + j - 16] >> 4);
        return (float)(q - 8) * d;
    }
    case RT_GGML_Q4_1: {       // { f16 d; f16 m; u8 qs[16] }
        const uint8_t *b = row + 20 * (col >> 5);
        float d = h2f(ld2u(b)), m = h2f(ld2u(b + 2));
        int j = (int)(col & 31);
        int q = j < 16 ? (b[4 + j] & 0x0F) : (b[4 + j - 16] >> 4);
        return (float)q * d + m;
    }
    case RT_GGML_Q5_0: {       // { f16 d; u8 qh[4]; u8 qs[16] }: bit j of qh (little-endian u32) is the fifth bit of element j
        const uint8_t *b = row + 22 * (col >> 5);
        float d = h2f(ld2u(b));
        int j = (int)(col & 31);
        int q = (j < 16 ? (b[6 + j] & 0x0F) : (b[6 + j - 16] >> 4)) | (((b[2 + (j >> 3)] >> (j & 7)) & 1) << 4);
        return (float)(q - 16) * d;
    }
    case RT_GGML_Q5_1: {       // { f16 d; f16 m; u8 qh[4]; u8 qs[16] }
        const uint8_t *b = row + 24 * (col >> 5);
        float d = h2f(ld2u(b)), m = h2f(ld2u(b + 2));
        int j = (int)(col & 31);
        int q = (j < 16 ? (b[8 + j] & 0x0F) : (b[8 + j - 16] >> 4)) | (((b[4 + (j >> 3)] >> (j & 7)) & 1) << 4);
        return (float)q * d + m;
    }
    case RT_GGML_Q2_K: {       // { u8 scales[16]; u8 qs[64]; f16 d; f16 dmin }: 2-bit values, per 16 elements a 4-bit scale and a 4-bit minimum
        const uint8_t *b = row + 84 * (col >> 8);
        int e = (int)(col & 255);
        int n = e >> 7, j = (e >> 5) & 3, l = e & 31;
        uint8_t sc = b[8 * n + 2 * j + (l >> 4)];
        float dl = h2f(ld2u(b + 80)) * (float)(sc & 0xF), ml = h2f(ld2u(b + 82)) * (float)(sc >> 4);
        int q = (b[16 + 32 * n + l] >> (2 * j)) & 3;
        return dl * (float)q - ml;
    }
    case RT_GGML_Q3_K: {       // { u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d }: 2 low bits in qs, the third in hmask, 16 six-bit scales
        const uint8_t *b = row + 110 * (col >> 8);
        int e = (int)(col & 255);
        int n = e >> 7, j = (e >> 5) & 3, l = e & 31;      // half, 32-run within the half, position
        int k = 8 * n + 2 * j + (l >> 4);                  // scale of the 16 elements around e
        const uint8_t *s = b + 96;
        int lo4 = k < 8 ? (s[k] & 15) : (s[k - 8] >> 4);
        int hi2 = (s[8 + (k & 3)] >> (2 * (k >> 2))) & 3;
        float dl = h2f(ld2u(b + 108)) * (float)((lo4 | (hi2 << 4)) - 32);
        int q = ((b[32 + 32 * n + l] >> (2 * j)) & 3) - (((b[l] >> (4 * n + j)) & 1) ? 0 : 4);
        return dl * (float)q;
    }
    case RT_GGML_Q4_K: {
        const uint8_t *b = row + 144 * (col >> 8);
        int e = (int)(col & 255);
        int j = e >> 5;             // sub-block 0..7
        int l = e & 31;
        const uint8_t *s = b + 4;
        int sc, m;
        if (j < 4) { sc = s[j] & 63; m = s[j + 4] & 63; }
        else { sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4); m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4); }
        float d = h2f(ld2u(b)) * (float)sc;
        float mn = h2f(ld2u(b + 2)) * (float)m;
        uint8_t qb = b[16 + 32 * (j >> 1) + l];
        int q = (j & 1) ? (qb >> 4) : (qb & 0x0F);
        return d * (float)q - mn;
    }
    case RT_GGML_Q5_K: {       // { f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128] }: Q4_K with a fifth bit per element in qh
        const uint8_t *b = row + 176 * (col >> 8);
        int e = (int)(col & 255);
        int j = e >> 5;             // sub-block 0..7: its fifth bits are bit j of qh[l]
        int l = e & 31;
        const uint8_t *s = b + 4;
        int sc, m;
        if (j < 4) { sc = s[j] & 63; m = s[j + 4] & 63; }
        else { sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4); m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4); }
        float d = h2f(ld2u(b)) * (float)sc;
        float mn = h2f(ld2u(b + 2)) * (float)m;
        uint8_t qb = b[48 + 32 * (j >> 1) + l];
        int q = ((j & 1) ? (qb >> 4) : (qb & 0x0F)) + (((b[16 + l] >> j) & 1) ? 16 : 0);
        return d * (float)q - mn;
    }
    case RT_GGML_Q6_K: {
        const uint8_t *b = row + 210 * (col >> 8);
        int e = (int)(col & 255);
        int h = e >> 7;             // half 0..1
        int r = (e >> 5) & 3;       // 32-run within the half
        int l = e & 31;
        const uint8_t *ql = b + 64 * h, *qh = b + 128 + 32 * h;
        const int8_t *sc = (const int8_t *)(b + 192 + 8 * h);
        uint8_t lo = ql[l + 32 * (r & 1)];
        int nib = (r & 2) ? (lo >> 4) : (lo & 0x0F);
        int q = (nib | (((qh[l] >> (2 * r)) & 3) << 4)) - 32;
        float d = h2f(ld2u(b + 208));
        return d * (float)(int)sc[(l >> 4) + 2 * r] * (float)q;
    }
    }
    return 0.f;
}

#pragma clang fp contract(fast)

// Activation accesses that must be coherent across XCDs inside one launch (COH) go out as device-scope
// relaxed atomics, which bypass the per-XCD L2; otherwise they are plain cached accesses.
template <bool COH> __device__ __forceinline__ float ld_f(const float *p) {
    if (COH) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}
template <bool COH> __device__ __forceinline__ void st_f(float *p, float v) {
    if (COH) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}
template <bool COH> __device__ __forceinline__ float4 ld_f4(const float *p) {  // p is 16-byte aligned
    if (COH) {
        const unsigned long long *q = reinterpret_cast<const unsigned long long *>(p);
        unsigned long long a = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned long long b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return make_float4(__uint_as_float((unsigned)a), __uint_as_float((unsigned)(a >> 32)), __uint_as_float((unsigned)b),
                           __uint_as_float((unsigned)(b >> 32)));
    }
    return *reinterpret_cast<const float4 *>(p);
}

// Sum over the 64 lanes of a wave with DPP row operations (no LDS traffic); every lane must be active.
// The total is returned to all lanes.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, true);
    return v + __int_as_float(r);
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v = dpp_add<0xB1, 0xF>(v);    // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xF>(v);    // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xF>(v);   // row_half_mirror
    v = dpp_add<0x140, 0xF>(v);   // row_mirror: every lane of a 16-lane row holds the row sum
    v = dpp_add<0x142, 0xA>(v);   // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xC>(v);   // row_bcast:31 into rows 2 and 3: lane 63 holds the total
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// The 4-element quantization step shared by every producer of the xq form: returns the packed high / low
// int8 planes, the block scale and the sum of the 16-element run the lane belongs to.
struct Q4Pack {
    uint32_t hi, lo;
    float s;
    int sum16, sum32;
};
__device__ __forceinline__ Q4Pack quantize4(float4 v) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
    // (a block whose largest magnitude is below 16383 / FLT_MAX makes inv infinite: its zeros then give NaN, which the
    // conversion below turns into 0, its other elements saturate and are clamped; the scale is as tiny as the values)
    float inv = amax > 0.f ? 16383.0f / amax : 0.f;
    Q4Pack r;
    r.s = amax / 16383.0f;
    int q0 = max(-16383, min(16383, __float2int_rn(v.x * inv)));
    int q1 = max(-16383, min(16383, __float2int_rn(v.y * inv)));
    int q2 = max(-16383, min(16383, __float2int_rn(v.z * inv)));
    int q3 = max(-16383, min(16383, __float2int_rn(v.w * inv)));
    r.hi = ((uint32_t)(q0 >> 7) & 0xFF) | (((uint32_t)(q1 >> 7) & 0xFF) << 8) | (((uint32_t)(q2 >> 7) & 0xFF) << 16) |
           (((uint32_t)(q3 >> 7) & 0xFF) << 24);
    r.lo = (uint32_t)(q0 & 127) | ((uint32_t)(q1 & 127) << 8) | ((uint32_t)(q2 & 127) << 16) | ((uint32_t)(q3 & 127) << 24);
    int sum = q0 + q1 + q2 + q3;
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    r.sum16 = sum;
    r.sum32 = sum + __shfl_xor(sum, 4, 64);
    return r;
}

// The operand form of the small-batch matrix-core GEMV (rt_gemv_mb.hip): up to 8 activation rows ("tokens") of K elements
// in one workspace -- 16 K bytes of int8 planes, then xs[K / 32][8] (block scales) and xb[K / 32][8] (scale x block sum).
// Per 32-element block 512 bytes in the order the GEMV's lanes load them: [k chunk c = 0..3][matrix row i = 8 * plane +
// token][8 bytes].  Stores the four elements i4 * 4 .. + 3 of row `token`; the 8 lanes that hold a block must be
// consecutive lanes of one wave, all active.  Rows that carry no token must be stored as zeros (the GEMV multiplies all 8).
struct Xq8Work {
    uint8_t *xq;
    float *xs, *xb;
};
__device__ __host__ __forceinline__ Xq8Work xq8_work(void *work, size_t K) {
    uint8_t *xq = static_cast<uint8_t *>(work);
    float *xs = reinterpret_cast<float *>(xq + 16 * K);
    return Xq8Work{ xq, xs, xs + K / 4 };
}
__device__ __forceinline__ void xq8_store4(float4 v, int i4, int token, const Xq8Work &w) {
    const Q4Pack p = quantize4(v);
    const int blk = i4 >> 3, l8 = i4 & 7;
    uint8_t *base = w.xq + (size_t)blk * 512 + (l8 >> 1) * 128 + token * 8 + (l8 & 1) * 4;
    *reinterpret_cast<uint32_t *>(base) = p.hi;
    *reinterpret_cast<uint32_t *>(base + 64) = p.lo;
    if (l8 == 0) {
        w.xs[blk * 8 + token] = p.s;
        w.xb[blk * 8 + token] = p.s * (float)p.sum32;
    }
}

}  // namespace rt
