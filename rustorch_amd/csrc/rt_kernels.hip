// Decode-path kernels for gfx950 (wave64): block decode, activation
// quantization, dequant-fused GEMV, RMSNorm, RoPE, KV append, single-query
// attention, SwiGLU, residual add, argmax, embedding row, dense f32 matmul.
//
// Block layouts are the public ggml ones (byte sizes as in
// example-cli/src/model/formats/gguf.rs:125-144):
//   Q8_0 34 B / 32 el : f16 d; i8 qs[32]
//   Q4_0 18 B / 32 el : f16 d; u8 qs[16]        (low nibbles = el 0..15, high = 16..31)
//   Q4_K 144 B / 256  : f16 d; f16 dmin; u8 scales[12]; u8 qs[128]
//   Q6_K 210 B / 256  : u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d
#include "rt_internal.h"

#include <hip/hip_fp16.h>

namespace rt {

// ------------------------------------------------------------------ helpers

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
__device__ float deq_elem(int type, const uint8_t *row, size_t col) {
    switch (type) {
    case RT_GGML_F32: { float f; __builtin_memcpy(&f, row + 4 * col, 4); return f; }
    case RT_GGML_F16: return h2f(ld2u(row + 2 * col));
    case RT_GGML_Q8_0: {
        const uint8_t *b = row + 34 * (col >> 5);
        float d = h2f(ld2u(b));
        return d * (float)(int)(int8_t)b[2 + (col & 31)];
    }
    case RT_GGML_Q4_0: {
        const uint8_t *b = row + 18 * (col >> 5);
        float d = h2f(ld2u(b));
        int j = (int)(col & 31);
        int q = j < 16 ? (b[2 + j] & 0x0F) : (b[2 + j - 16] >> 4);
        return (float)(q - 8) * d;
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

__global__ void dequant_kernel(int type, const uint8_t *w, size_t row_bytes, size_t n_rows, size_t n_cols, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = n_rows * n_cols;
    for (; i < total; i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i / n_cols, c = i - r * n_cols;
        out[i] = deq_elem(type, w + r * row_bytes, c);
    }
}

__global__ void embed_row_kernel(int type, const uint8_t *w, size_t row_bytes, size_t n_cols, const int *token_dev,
                                 int vocab, float *out) {
    int tok = *token_dev;
    if (tok < 0) tok = 0;
    if (tok >= vocab) tok = vocab - 1;
    size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c < n_cols) out[c] = deq_elem(type, w + (size_t)tok * row_bytes, c);
}
#pragma clang fp contract(fast)

// ----------------------------------------------------- activation quantization
// Quantize 4 consecutive elements (e % 4 == 0) of a K-vector into xq.  The 8 lanes that
// hold one 32-element block must be consecutive lanes of one wave and all active.
__device__ __forceinline__ void quantize_store4(float4 v, size_t e, uint8_t *xq, size_t K) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
    float inv = amax > 0.f ? 16383.0f / amax : 0.f;
    float s = amax / 16383.0f;
    int q0 = max(-16383, min(16383, __float2int_rn(v.x * inv)));
    int q1 = max(-16383, min(16383, __float2int_rn(v.y * inv)));
    int q2 = max(-16383, min(16383, __float2int_rn(v.z * inv)));
    int q3 = max(-16383, min(16383, __float2int_rn(v.w * inv)));
    uint32_t hi = ((uint32_t)(q0 >> 7) & 0xFF) | (((uint32_t)(q1 >> 7) & 0xFF) << 8) |
                  (((uint32_t)(q2 >> 7) & 0xFF) << 16) | (((uint32_t)(q3 >> 7) & 0xFF) << 24);
    uint32_t lo = (uint32_t)(q0 & 127) | ((uint32_t)(q1 & 127) << 8) | ((uint32_t)(q2 & 127) << 16) |
                  ((uint32_t)(q3 & 127) << 24);
    int sum = q0 + q1 + q2 + q3;
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    *reinterpret_cast<uint32_t *>(xq + e) = hi;
    *reinterpret_cast<uint32_t *>(xq + K + e) = lo;
    float *sp = reinterpret_cast<float *>(xq + 2 * K);
    float *bp = sp + K / 32;
    if ((e & 15) == 0) bp[e >> 4] = s * (float)sum;
    if ((e & 31) == 0) sp[e >> 5] = s;
}

__global__ __launch_bounds__(256) void quantize_x_kernel(const float *x, uint8_t *xq, size_t K) {
    size_t m = blockIdx.y;
    size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 * 4 >= K) return;  // whole 8-lane groups leave together because K % 32 == 0
    float4 v = reinterpret_cast<const float4 *>(x + m * K)[i4];
    quantize_store4(v, i4 * 4, xq + m * xq_stride(K), K);
}

// Several independent vectors in one launch (grid.y = vector index).
__global__ __launch_bounds__(256) void quantize_group_kernel(QuantGroupArgs a) {
    int p = blockIdx.y;
    size_t K = (size_t)a.K[p];
    size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 * 4 >= K) return;
    float4 v = reinterpret_cast<const float4 *>(a.x[p])[i4];
    quantize_store4(v, i4 * 4, a.xq[p], K);
}

// ------------------------------------------------------------ GEMV unit dots
// A "unit" is the slice of one weight row a lane consumes in one go.  x lives in LDS in
// xq form: xh / xl as dwords of 4 int8, xs per 32-block, xb per 16-run.

struct XLds {
    const int *xh, *xl;
    const float *xs, *xb;
};

// Q4_K unit u: super-block u/4, 64-element group g = u%4 (32 qs bytes; low nibbles = sub-block 2g, high = 2g+1).
__device__ __forceinline__ float unit_q4k(const uint8_t *row, int u, const XLds &X) {
    int sb = u >> 2, g = u & 3;
    const uint8_t *blk = row + (size_t)sb * 144;
    uint4 hdr = ld16a(blk);
    uint4 qa = ld16a(blk + 16 + 32 * g);
    uint4 qb = ld16a(blk + 32 + 32 * g);
    uint32_t scw, mw;
    if (g < 2) {
        scw = hdr.y & 0x3f3f3f3fu;
        mw = hdr.z & 0x3f3f3f3fu;
    } else {
        scw = (hdr.w & 0x0f0f0f0fu) | ((hdr.y >> 2) & 0x30303030u);
        mw = ((hdr.w >> 4) & 0x0f0f0f0fu) | ((hdr.z >> 2) & 0x30303030u);
    }
    int sh = (g & 1) * 16;
    float sc0 = (float)((scw >> sh) & 0xFF), sc1 = (float)((scw >> (sh + 8)) & 0xFF);
    float m0 = (float)((mw >> sh) & 0xFF), m1 = (float)((mw >> (sh + 8)) & 0xFF);
    float d = h2f(hdr.x & 0xFFFF), dmin = h2f(hdr.x >> 16);
    uint32_t q[8] = { qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w };
    int e4 = u * 16;
    int dh0 = 0, dl0 = 0, dh1 = 0, dl1 = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint32_t lo = q[i] & 0x0f0f0f0fu, hi = (q[i] >> 4) & 0x0f0f0f0fu;
        dh0 = sdot4(lo, X.xh[e4 + i], dh0);
        dl0 = sdot4(lo, X.xl[e4 + i], dl0);
        dh1 = sdot4(hi, X.xh[e4 + 8 + i], dh1);
        dl1 = sdot4(hi, X.xl[e4 + 8 + i], dl1);
    }
    float t0 = (float)((dh0 << 7) + dl0), t1 = (float)((dh1 << 7) + dl1);
    int b = u * 2;
    float s0 = X.xs[b], s1 = X.xs[b + 1];
    float bs0 = X.xb[2 * b] + X.xb[2 * b + 1], bs1 = X.xb[2 * b + 2] + X.xb[2 * b + 3];
    return d * (sc0 * (s0 * t0) + sc1 * (s1 * t1)) - dmin * (m0 * bs0 + m1 * bs1);
}

// Q6_K unit u: super-block u/4, half h = (u/2)%2, l-range c = u%2 (l in [16c, 16c+16)); four 16-element runs.
__device__ __forceinline__ float unit_q6k(const uint8_t *row, int u, const XLds &X) {
    int sb = u >> 2, h = (u >> 1) & 1, c = u & 1;
    const uint8_t *blk = row + (size_t)sb * 210;
    uint4 A4 = ld16u(blk + 64 * h + 16 * c);
    uint4 B4 = ld16u(blk + 64 * h + 32 + 16 * c);
    uint4 H4 = ld16u(blk + 128 + 32 * h + 16 * c);
    uint2 scw = ld8u(blk + 192 + 8 * h);
    float d = h2f(ld2u(blk + 208));
    uint32_t A[4] = { A4.x, A4.y, A4.z, A4.w }, B[4] = { B4.x, B4.y, B4.z, B4.w }, H[4] = { H4.x, H4.y, H4.z, H4.w };
    int dh[4] = { 0, 0, 0, 0 }, dl[4] = { 0, 0, 0, 0 };
    int xd = 64 * sb + 32 * h + 4 * c;  // dword index of run 0
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t q1 = (A[i] & 0x0f0f0f0fu) | ((H[i] << 4) & 0x30303030u);
        uint32_t q2 = (B[i] & 0x0f0f0f0fu) | ((H[i] << 2) & 0x30303030u);
        uint32_t q3 = ((A[i] >> 4) & 0x0f0f0f0fu) | (H[i] & 0x30303030u);
        uint32_t q4 = ((B[i] >> 4) & 0x0f0f0f0fu) | ((H[i] >> 2) & 0x30303030u);
        dh[0] = sdot4(q1, X.xh[xd + i], dh[0]);       dl[0] = sdot4(q1, X.xl[xd + i], dl[0]);
        dh[1] = sdot4(q2, X.xh[xd + 8 + i], dh[1]);   dl[1] = sdot4(q2, X.xl[xd + 8 + i], dl[1]);
        dh[2] = sdot4(q3, X.xh[xd + 16 + i], dh[2]);  dl[2] = sdot4(q3, X.xl[xd + 16 + i], dl[2]);
        dh[3] = sdot4(q4, X.xh[xd + 24 + i], dh[3]);  dl[3] = sdot4(q4, X.xl[xd + 24 + i], dl[3]);
    }
    // scales sc[c + 2r], r = 0..3: bytes c, c+2 of scw.x and of scw.y
    int s8 = c * 8;
    float sc0 = (float)(int)(int8_t)((scw.x >> s8) & 0xFF), sc1 = (float)(int)(int8_t)((scw.x >> (s8 + 16)) & 0xFF);
    float sc2 = (float)(int)(int8_t)((scw.y >> s8) & 0xFF), sc3 = (float)(int)(int8_t)((scw.y >> (s8 + 16)) & 0xFF);
    int sbk = 8 * sb + 4 * h;            // x 32-block of run 0
    int bbk = 16 * sb + 8 * h + c;       // x 16-run of run 0
    float acc = sc0 * (X.xs[sbk] * (float)((dh[0] << 7) + dl[0]) - 32.f * X.xb[bbk]);
    acc += sc1 * (X.xs[sbk + 1] * (float)((dh[1] << 7) + dl[1]) - 32.f * X.xb[bbk + 2]);
    acc += sc2 * (X.xs[sbk + 2] * (float)((dh[2] << 7) + dl[2]) - 32.f * X.xb[bbk + 4]);
    acc += sc3 * (X.xs[sbk + 3] * (float)((dh[3] << 7) + dl[3]) - 32.f * X.xb[bbk + 6]);
    return d * acc;
}

// Q8_0 unit u = block u.
__device__ __forceinline__ float unit_q80(const uint8_t *row, int u, const XLds &X) {
    const uint8_t *blk = row + (size_t)u * 34;
    float d = h2f(ld2u(blk));
    uint4 a = ld16u(blk + 2), b = ld16u(blk + 18);
    uint32_t q[8] = { a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w };
    int dh = 0, dl = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        dh = sdot4(q[i], X.xh[8 * u + i], dh);
        dl = sdot4(q[i], X.xl[8 * u + i], dl);
    }
    return d * (X.xs[u] * ((float)dh * 128.f + (float)dl));
}

// Q4_0 unit u = block u.
__device__ __forceinline__ float unit_q40(const uint8_t *row, int u, const XLds &X) {
    const uint8_t *blk = row + (size_t)u * 18;
    float d = h2f(ld2u(blk));
    uint4 a = ld16u(blk + 2);
    uint32_t q[4] = { a.x, a.y, a.z, a.w };
    int dh = 0, dl = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t lo = q[i] & 0x0f0f0f0fu, hi = (q[i] >> 4) & 0x0f0f0f0fu;
        dh = sdot4(lo, X.xh[8 * u + i], dh);
        dl = sdot4(lo, X.xl[8 * u + i], dl);
        dh = sdot4(hi, X.xh[8 * u + 4 + i], dh);
        dl = sdot4(hi, X.xl[8 * u + 4 + i], dl);
    }
    return d * (X.xs[u] * (float)((dh << 7) + dl) - 8.f * (X.xb[2 * u] + X.xb[2 * u + 1]));
}

template <int TYPE> __device__ __forceinline__ float unit_dot(const uint8_t *row, int u, const XLds &X) {
    if (TYPE == RT_GGML_Q4_K) return unit_q4k(row, u, X);
    if (TYPE == RT_GGML_Q6_K) return unit_q6k(row, u, X);
    if (TYPE == RT_GGML_Q8_0) return unit_q80(row, u, X);
    return unit_q40(row, u, X);
}

template <int TYPE>
__device__ __forceinline__ void gemv_rows(const GemvProb &P, int row0, int row1, int m, const XLds &X) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = blockDim.x >> 6;
    const int unit_elems = (TYPE == RT_GGML_Q4_K || TYPE == RT_GGML_Q6_K) ? 64 : 32;
    const int n_units = P.K / unit_elems;
    for (int row = row0 + wave; row < row1; row += nwaves) {
        const uint8_t *rp = P.w + (size_t)row * P.row_bytes;
        float acc = 0.f;
        for (int u = lane; u < n_units; u += 64) acc += unit_dot<TYPE>(rp, u, X);
        acc = wave_sum(acc);
        if (lane == 0) {
            size_t o = (size_t)m * P.N + row;
            P.y[o] = P.res ? P.res[o] + acc : acc;
        }
    }
}

__global__ __launch_bounds__(256) void qgemv_kernel(GemvArgs a) {
    extern __shared__ uint4 lds[];
    int tile = blockIdx.x;
    int pi = 0;
#pragma unroll
    for (int i = 1; i < kMaxGemvProbs; i++)
        if (i < a.n && tile >= a.p[i].tile0) pi = i;
    const GemvProb &P = a.p[pi];
    int t = tile - P.tile0;
    int row0 = t * P.rows_per_tile;
    int row1 = min(P.N, row0 + P.rows_per_tile);
    int m = blockIdx.y;
    size_t K = (size_t)P.K;
    size_t stride = xq_stride(K);
    const uint4 *src = reinterpret_cast<const uint4 *>(P.xq + (size_t)m * stride);
    for (int i = threadIdx.x; i < (int)(stride / 16); i += blockDim.x) lds[i] = src[i];
    __syncthreads();
    const char *base = reinterpret_cast<const char *>(lds);
    XLds X;
    X.xh = reinterpret_cast<const int *>(base);
    X.xl = reinterpret_cast<const int *>(base + K);
    X.xs = reinterpret_cast<const float *>(base + 2 * K);
    X.xb = X.xs + K / 32;
    switch (P.type) {
    case RT_GGML_Q4_K: gemv_rows<RT_GGML_Q4_K>(P, row0, row1, m, X); break;
    case RT_GGML_Q6_K: gemv_rows<RT_GGML_Q6_K>(P, row0, row1, m, X); break;
    case RT_GGML_Q8_0: gemv_rows<RT_GGML_Q8_0>(P, row0, row1, m, X); break;
    case RT_GGML_Q4_0: gemv_rows<RT_GGML_Q4_0>(P, row0, row1, m, X); break;
    }
}

// ------------------------------------------------------------------ RMSNorm
// One block per row.  y = gamma * (x / sqrt(mean(x^2) + eps))  (src/nn/normalization.rs:682-696).
// Writes f32 y when y != nullptr and the xq form when xq != nullptr (needs n % 32 == 0).
__global__ __launch_bounds__(1024) void rmsnorm_kernel(const float *x, const float *gamma, float *y, uint8_t *xq,
                                                       size_t n, float eps) {
    __shared__ float red[16];
    size_t m = blockIdx.x;
    const float *xr = x + m * n;
    float ss = 0.f;
    if ((n & 3) == 0) {
        const float4 *x4 = reinterpret_cast<const float4 *>(xr);
        for (size_t i = threadIdx.x; i < n / 4; i += blockDim.x) {
            float4 v = x4[i];
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    } else {
        for (size_t i = threadIdx.x; i < n; i += blockDim.x) ss += xr[i] * xr[i];
    }
    ss = block_sum(ss, red);
    float rms = sqrtf(ss / (float)n + eps);
    if ((n & 3) == 0) {
        const float4 *x4 = reinterpret_cast<const float4 *>(xr);
        const float4 *g4 = reinterpret_cast<const float4 *>(gamma);
        for (size_t i = threadIdx.x; i < n / 4; i += blockDim.x) {
            float4 v = x4[i], g = g4[i];
            float4 o = make_float4(g.x * (v.x / rms), g.y * (v.y / rms), g.z * (v.z / rms), g.w * (v.w / rms));
            if (y) reinterpret_cast<float4 *>(y + m * n)[i] = o;
            if (xq) quantize_store4(o, i * 4, xq + m * xq_stride(n), n);
        }
    } else {
        for (size_t i = threadIdx.x; i < n; i += blockDim.x) y[m * n + i] = gamma[i] * (xr[i] / rms);
    }
}

// ------------------------------------------------------------------- SwiGLU
// out = up * (gate * 1/(1+exp(-gate)))  (src/nn/activation.rs:404-414 with a = up, b = gate).
__global__ __launch_bounds__(256) void swiglu_kernel(const float *gate, const float *up, float *out, uint8_t *xq,
                                                     size_t n) {
    size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if ((n & 3) == 0) {
        if (i4 * 4 >= n) return;
        float4 g = reinterpret_cast<const float4 *>(gate)[i4], u = reinterpret_cast<const float4 *>(up)[i4];
        float4 o;
        o.x = u.x * (g.x * (1.0f / (1.0f + expf(-g.x))));
        o.y = u.y * (g.y * (1.0f / (1.0f + expf(-g.y))));
        o.z = u.z * (g.z * (1.0f / (1.0f + expf(-g.z))));
        o.w = u.w * (g.w * (1.0f / (1.0f + expf(-g.w))));
        if (out) reinterpret_cast<float4 *>(out)[i4] = o;
        if (xq) quantize_store4(o, i4 * 4, xq, n);
    } else {
        for (size_t i = i4 * 4; i < n && i < i4 * 4 + 4; i++) {
            float b = gate[i];
            out[i] = up[i] * (b * (1.0f / (1.0f + expf(-b))));
        }
    }
}

// --------------------------------------------------------------------- RoPE
// Interleaved pairs: (x[2i], x[2i+1]) turned by pos * inv_freq[i].  One thread per pair.
__global__ void rope_kernel(float *x, int n_heads, int head_dim, const int *pos_dev, int pos, const float *inv_freq,
                            float theta) {
    int half = head_dim / 2;
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_heads * half) return;
    int i = t % half;
    int p = pos_dev ? *pos_dev : pos;
    float f = inv_freq ? inv_freq[i] : (float)pow((double)theta, -2.0 * (double)i / (double)head_dim);
    float ang = (float)p * f;
    float s, c;
    sincosf(ang, &s, &c);
    float2 v = reinterpret_cast<float2 *>(x)[t];
    reinterpret_cast<float2 *>(x)[t] = make_float2(v.x * c - v.y * s, v.x * s + v.y * c);
}

__global__ void kv_append_kernel(uint16_t *cache, const float *v, const int *pos_dev, size_t pos, size_t row_elems) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t p = pos_dev ? (size_t)*pos_dev : pos;
    if (i < row_elems) cache[p * row_elems + i] = f2h_rne(v[i]);
}

// Fused decode-step form: rotate q in place, rotate k and store it and v as fp16 at row *pos_dev.
__global__ void rope_kv_kernel(float *q, const float *k, const float *v, uint16_t *kcache, uint16_t *vcache,
                               const int *pos_dev, int n_heads, int head_dim, const float *inv_freq) {
    int half = head_dim / 2;
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_heads * half) return;
    int i = t % half;
    int p = *pos_dev;
    size_t row = (size_t)n_heads * head_dim;
    float ang = (float)p * inv_freq[i];
    float s, c;
    sincosf(ang, &s, &c);
    float2 qv = reinterpret_cast<float2 *>(q)[t];
    reinterpret_cast<float2 *>(q)[t] = make_float2(qv.x * c - qv.y * s, qv.x * s + qv.y * c);
    float2 kv = reinterpret_cast<const float2 *>(k)[t];
    float k0 = kv.x * c - kv.y * s, k1 = kv.x * s + kv.y * c;
    float2 vv = reinterpret_cast<const float2 *>(v)[t];
    uint32_t kp = (uint32_t)f2h_rne(k0) | ((uint32_t)f2h_rne(k1) << 16);
    uint32_t vp = (uint32_t)f2h_rne(vv.x) | ((uint32_t)f2h_rne(vv.y) << 16);
    reinterpret_cast<uint32_t *>(kcache + (size_t)p * row)[t] = kp;
    reinterpret_cast<uint32_t *>(vcache + (size_t)p * row)[t] = vp;
}

// -------------------------------------------------------- decode attention
// One block (256 threads) per head; cache layout [pos][head][dim], fp16.
// scores = (q . k_j) / sqrt(dim); p = softmax(scores) with max subtraction; out = sum_j p_j v_j
// (example-cli/src/model/architectures/attention.rs:233-338 for one query row).
// EPL = head_dim / 64 (1 or 2).  Dynamic LDS: n_pos floats of scores.
template <int EPL>
__global__ __launch_bounds__(256) void attn_decode_kernel(const float *q, const uint16_t *kc, const uint16_t *vc,
                                                          const int *pos_dev, int n_pos_arg, int n_heads, float *out,
                                                          uint8_t *xq) {
    extern __shared__ float sc[];
    __shared__ float red[4];
    __shared__ __align__(16) float part[256];
    constexpr int HD = 64 * EPL;
    const int n_pos = pos_dev ? *pos_dev + 1 : n_pos_arg;
    const int h = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const size_t row = (size_t)n_heads * HD;
    const float scale = 1.0f / sqrtf((float)HD);
    float qv[EPL];
#pragma unroll
    for (int e = 0; e < EPL; e++) qv[e] = q[(size_t)h * HD + lane * EPL + e];
    for (int j = wave; j < n_pos; j += 4) {
        const uint16_t *kr = kc + (size_t)j * row + (size_t)h * HD + lane * EPL;
        float s = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; e++) s += qv[e] * h2f(kr[e]);
        s = wave_sum(s);
        if (lane == 0) sc[j] = s * scale;
    }
    __syncthreads();
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < n_pos; j += 256) mx = fmaxf(mx, sc[j]);
    mx = block_max(mx, red);
    float sum = 0.f;
    for (int j = threadIdx.x; j < n_pos; j += 256) {
        float e = expf(sc[j] - mx);
        sc[j] = e;
        sum += e;
    }
    sum = block_sum(sum, red);
    for (int j = threadIdx.x; j < n_pos; j += 256) sc[j] = sc[j] / sum;
    __syncthreads();
    const int d = threadIdx.x % HD, grp = threadIdx.x / HD, ngrp = 256 / HD;
    float acc = 0.f;
    for (int j = grp; j < n_pos; j += ngrp) acc += sc[j] * h2f(vc[(size_t)j * row + (size_t)h * HD + d]);
    part[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x < HD) {
        float o = 0.f;
        for (int g = 0; g < ngrp; g++) o += part[g * HD + threadIdx.x];
        part[threadIdx.x] = o;
        if (out) out[(size_t)h * HD + threadIdx.x] = o;
    }
    if (xq) {
        __syncthreads();
        if (threadIdx.x < HD / 4) {
            float4 v = reinterpret_cast<const float4 *>(part)[threadIdx.x];
            quantize_store4(v, (size_t)h * HD + threadIdx.x * 4, xq, row);
        }
    }
}

// ------------------------------------------------------------- small pieces
__global__ void add_kernel(float *x, const float *y, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = x[i] + y[i];
}

// Greedy pick; ties resolve to the lowest index.
__global__ __launch_bounds__(1024) void argmax_kernel(const float *v, size_t n, int *out) {
    __shared__ float bv[1024];
    __shared__ int bi[1024];
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (size_t i = threadIdx.x; i < n; i += blockDim.x) {
        float f = v[i];
        if (f > best) { best = f; idx = (int)i; }
    }
    bv[threadIdx.x] = best;
    bi[threadIdx.x] = idx;
    __syncthreads();
    for (int s = blockDim.x / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            float o = bv[threadIdx.x + s];
            int oi = bi[threadIdx.x + s];
            if (o > bv[threadIdx.x] || (o == bv[threadIdx.x] && oi < bi[threadIdx.x])) {
                bv[threadIdx.x] = o;
                bi[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) *out = bi[0] == 0x7fffffff ? 0 : bi[0];
}

__global__ void set_int_kernel(int *dst, int value) { *dst = value; }

// End of a decode step: record the pick, choose the next input token, advance the position.
__global__ void step_advance_kernel(int *pos_dev, int *token_dev, const int *pick_dev, const int *forced_dev,
                                    int *out_tokens_dev, int *step_dev) {
    int step = *step_dev;
    int pick = *pick_dev;
    if (out_tokens_dev) out_tokens_dev[step] = pick;
    *token_dev = forced_dev ? forced_dev[step] : pick;
    *pos_dev = *pos_dev + 1;
    *step_dev = step + 1;
}

// Dense row-major f32 C[m,n] = A[m,k] . B[k,n], 32x32 tiles through LDS, k summed in ascending order.
__global__ __launch_bounds__(1024) void matmul_f32_kernel(const float *a, const float *b, float *c, size_t m, size_t n,
                                                          size_t k) {
    __shared__ float as[32][33];
    __shared__ float bs[32][33];
    size_t row = (size_t)blockIdx.y * 32 + threadIdx.y, col = (size_t)blockIdx.x * 32 + threadIdx.x;
    float acc = 0.f;
    for (size_t k0 = 0; k0 < k; k0 += 32) {
        as[threadIdx.y][threadIdx.x] = (row < m && k0 + threadIdx.x < k) ? a[row * k + k0 + threadIdx.x] : 0.f;
        bs[threadIdx.y][threadIdx.x] = (col < n && k0 + threadIdx.y < k) ? b[(k0 + threadIdx.y) * n + col] : 0.f;
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 32; kk++) acc += as[threadIdx.y][kk] * bs[kk][threadIdx.x];
        __syncthreads();
    }
    if (row < m && col < n) c[row * n + col] = acc;
}

// ================================================================ launchers

hipError_t launch_quantize_x(hipStream_t s, const float *x, uint8_t *xq, size_t K, size_t batch) {
    dim3 grid((unsigned)((K / 4 + 255) / 256), (unsigned)batch);
    quantize_x_kernel<<<grid, 256, 0, s>>>(x, xq, K);
    return hipGetLastError();
}

hipError_t launch_quantize_group(hipStream_t s, const QuantGroupArgs &a) {
    size_t maxK = 0;
    for (int i = 0; i < a.n; i++) maxK = (size_t)a.K[i] > maxK ? (size_t)a.K[i] : maxK;
    if (a.n == 0 || maxK == 0) return hipSuccess;
    dim3 grid((unsigned)((maxK / 4 + 255) / 256), (unsigned)a.n);
    quantize_group_kernel<<<grid, 256, 0, s>>>(a);
    return hipGetLastError();
}

hipError_t launch_qgemv(hipStream_t s, GemvArgs &a, int batch) {
    size_t total_rows = 0, maxK = 0;
    for (int i = 0; i < a.n; i++) {
        total_rows += (size_t)a.p[i].N;
        if ((size_t)a.p[i].K > maxK) maxK = (size_t)a.p[i].K;
    }
    // aim for ~4 workgroups per CU across the launch; each workgroup re-stages x, so do not go below 8 rows
    int rpt = (int)((total_rows + 1023) / 1024);
    rpt = (rpt + 3) & ~3;
    if (rpt < 8) rpt = 8;
    int tiles = 0;
    for (int i = 0; i < a.n; i++) {
        a.p[i].tile0 = tiles;
        a.p[i].rows_per_tile = rpt;
        tiles += (a.p[i].N + rpt - 1) / rpt;
    }
    size_t lds = xq_stride(maxK);
    dim3 grid((unsigned)tiles, (unsigned)batch);
    qgemv_kernel<<<grid, 256, lds, s>>>(a);
    return hipGetLastError();
}

hipError_t launch_dequant(hipStream_t s, int type, const uint8_t *w, size_t n_rows, size_t n_cols, float *out) {
    size_t total = n_rows * n_cols;
    size_t rb = n_cols / type_block_elems(type) * type_block_bytes(type);
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (blocks == 0) return hipSuccess;
    dequant_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(type, w, rb, n_rows, n_cols, out);
    return hipGetLastError();
}

hipError_t launch_rmsnorm(hipStream_t s, const float *x, const float *gamma, float *y, uint8_t *xq, size_t rows,
                          size_t n, float eps) {
    if (rows == 0) return hipSuccess;
    rmsnorm_kernel<<<dim3((unsigned)rows), 1024, 0, s>>>(x, gamma, y, xq, n, eps);
    return hipGetLastError();
}

hipError_t launch_swiglu(hipStream_t s, const float *gate, const float *up, float *out, uint8_t *xq, size_t n) {
    if (n == 0) return hipSuccess;
    size_t n4 = (n + 3) / 4;
    swiglu_kernel<<<dim3((unsigned)((n4 + 255) / 256)), 256, 0, s>>>(gate, up, out, xq, n);
    return hipGetLastError();
}

hipError_t launch_rope(hipStream_t s, float *x, int n_heads, int head_dim, const int *pos_dev, int pos,
                       const float *inv_freq_dev, float theta) {
    int pairs = n_heads * head_dim / 2;
    if (pairs == 0) return hipSuccess;
    rope_kernel<<<dim3((unsigned)((pairs + 255) / 256)), 256, 0, s>>>(x, n_heads, head_dim, pos_dev, pos, inv_freq_dev,
                                                                      theta);
    return hipGetLastError();
}

hipError_t launch_kv_append(hipStream_t s, uint16_t *cache, const float *v, const int *pos_dev, size_t pos,
                            size_t row_elems) {
    if (row_elems == 0) return hipSuccess;
    kv_append_kernel<<<dim3((unsigned)((row_elems + 255) / 256)), 256, 0, s>>>(cache, v, pos_dev, pos, row_elems);
    return hipGetLastError();
}

hipError_t launch_rope_kv(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kcache,
                          uint16_t *vcache, const int *pos_dev, int n_heads, int head_dim,
                          const float *inv_freq_dev) {
    int pairs = n_heads * head_dim / 2;
    rope_kv_kernel<<<dim3((unsigned)((pairs + 255) / 256)), 256, 0, s>>>(q, k, v, kcache, vcache, pos_dev, n_heads,
                                                                         head_dim, inv_freq_dev);
    return hipGetLastError();
}

hipError_t launch_attn_decode(hipStream_t s, const float *q, const uint16_t *kc, const uint16_t *vc,
                              const int *pos_dev, int n_pos, int n_heads, int head_dim, float *out, uint8_t *xq) {
    size_t lds = (size_t)n_pos * sizeof(float);  // with pos_dev set, n_pos is the upper bound (max_pos)
    if (head_dim == 128)
        attn_decode_kernel<2><<<dim3((unsigned)n_heads), 256, lds, s>>>(q, kc, vc, pos_dev, n_pos, n_heads, out, xq);
    else if (head_dim == 64)
        attn_decode_kernel<1><<<dim3((unsigned)n_heads), 256, lds, s>>>(q, kc, vc, pos_dev, n_pos, n_heads, out, xq);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_add(hipStream_t s, float *x, const float *y, size_t n) {
    if (n == 0) return hipSuccess;
    add_kernel<<<dim3((unsigned)((n + 255) / 256)), 256, 0, s>>>(x, y, n);
    return hipGetLastError();
}

hipError_t launch_argmax(hipStream_t s, const float *v, size_t n, int *out_dev) {
    argmax_kernel<<<1, 1024, 0, s>>>(v, n, out_dev);
    return hipGetLastError();
}

hipError_t launch_embed_row(hipStream_t s, int type, const uint8_t *w, size_t row_bytes, size_t n_cols,
                            const int *token_dev, int vocab, float *out) {
    embed_row_kernel<<<dim3((unsigned)((n_cols + 255) / 256)), 256, 0, s>>>(type, w, row_bytes, n_cols, token_dev,
                                                                            vocab, out);
    return hipGetLastError();
}

hipError_t launch_matmul_f32(hipStream_t s, const float *a, const float *b, float *c, size_t m, size_t n, size_t k) {
    if (m == 0 || n == 0) return hipSuccess;
    dim3 grid((unsigned)((n + 31) / 32), (unsigned)((m + 31) / 32));
    matmul_f32_kernel<<<grid, dim3(32, 32), 0, s>>>(a, b, c, m, n, k);
    return hipGetLastError();
}

hipError_t launch_set_int(hipStream_t s, int *dst, int value) {
    set_int_kernel<<<1, 1, 0, s>>>(dst, value);
    return hipGetLastError();
}

hipError_t launch_step_advance(hipStream_t s, int *pos_dev, int *token_dev, const int *pick_dev,
                               const int *forced_dev, int *out_tokens_dev, int *step_dev) {
    step_advance_kernel<<<1, 1, 0, s>>>(pos_dev, token_dev, pick_dev, forced_dev, out_tokens_dev, step_dev);
    return hipGetLastError();
}

}  // namespace rt
