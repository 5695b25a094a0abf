// Device side of the dequant-fused GEMV (decode): shared by the stand-alone kernel and the persistent
// decode-step kernel.
//
// The computation is HBM-bound: every weight byte is read once with 16-byte loads and consumed by integer
// dot products (v_dot4_i32_i8) against the activation vector held in LDS as two int8 planes (16-bit
// block-scaled integers, see rt_internal.h).
//
// Work split: the workgroups that share a problem deal its rows out round-robin, one "row group" (R rows)
// per wave at a time; the 64 lanes of a wave stride the row's "units" (the slice of a row one lane eats:
// 64 elements of Q4_K / Q6_K, one block of Q8_0 / Q4_0).  The loads of the next step are issued before the
// current one is consumed, and the first step is requested before x is staged, so weight bytes are in
// flight while the workgroup waits for its input.  Partial sums are reduced across the wave with DPP.
//
// x is staged once per workgroup into LDS, in an order permuted per weight type so that the 16-byte LDS
// reads of consecutive lanes hit consecutive addresses.  The staging step can also produce x: quantize an
// f32 vector, or RMS-normalise and quantize it (the norm that precedes q/k/v and gate/up in a decoder
// layer).  The epilogue can add a residual or combine a gate row and an up row into up * silu(gate)
// (src/nn/activation.rs:404-414).
//
// COH = true makes every access to activations (x, y, res) a device-coherent one, for the persistent kernel
// where producer and consumer workgroups sit on different XCDs within one launch.
#pragma once

#include "rt_device.h"

namespace rt {

// Units of a row: 64 elements of the super-block formats, one 32-element block of the others, 16 bytes of an
// unquantized row (8 halves or 4 floats).
__device__ __forceinline__ int units_of(int type, int K) {
    if (type == RT_GGML_F16) return K / 8;
    if (type == RT_GGML_F32) return K / 4;
    return (type == RT_GGML_Q2_K || type == RT_GGML_Q3_K || type == RT_GGML_Q4_K || type == RT_GGML_Q5_K || type == RT_GGML_Q6_K) ? K / 64 : K / 32;
}

// dword index inside a plane (xh or xl) of the 4 elements starting at e (e % 4 == 0)
__device__ __forceinline__ int x_slot_dword(int type, int e, int U) {
    int j = e >> 4, w = (e >> 2) & 3;
    int slot;
    if (type == RT_GGML_Q4_K || type == RT_GGML_Q5_K) slot = (j & 3) * U + (j >> 2);
    else if (type == RT_GGML_Q6_K || type == RT_GGML_Q3_K || type == RT_GGML_Q2_K) slot = ((j >> 1) & 3) * U + (2 * (j >> 3) + (j & 1));
    else slot = (j & 1) * U + (j >> 1);
    return slot * 4 + w;
}

// Place 4 quantized elements and the block metadata they carry into the per-type LDS layout.
//   planes: xh at dword 0, xl at dword K/4; floats S from dword K/2:
//   Q4_K, Q5_K : S[4u + {0,1}] = scale of the unit's two 32-blocks, S[4u + {2,3}] = scale * sum of each block
//   Q6_K, Q3_K, Q2_K : S[b] = scale of 32-block b (= 4 * half + run);  S[2U + 4u + r] = scale * sum of the unit's run r
//   Q8_0 : S[u] = scale;   Q4_0 : S[2u] = scale, S[2u+1] = scale * sum of the block
__device__ __forceinline__ void stage_store(int type, int K, int U, uint32_t *lds, int e, uint32_t hi, uint32_t lo,
                                            float s, float bsum16, float bsum32) {
    int d = x_slot_dword(type, e, U);
    lds[d] = hi;
    lds[K / 4 + d] = lo;
    float *S = reinterpret_cast<float *>(lds + K / 2);
    if (type == RT_GGML_Q4_K || type == RT_GGML_Q5_K) {
        if ((e & 31) == 0) {
            int b = e >> 5, u = b >> 1, half = b & 1;
            S[4 * u + half] = s;
            S[4 * u + 2 + half] = bsum32;
        }
    } else if (type == RT_GGML_Q6_K || type == RT_GGML_Q3_K || type == RT_GGML_Q2_K) {
        if ((e & 31) == 0) S[e >> 5] = s;
        if ((e & 15) == 0) {
            int i16 = e >> 4;
            int u = 2 * (i16 >> 3) + (i16 & 1), r = (i16 >> 1) & 3;
            S[2 * U + 4 * u + r] = bsum16;
        }
    } else if (type == RT_GGML_Q8_0 || type == RT_GGML_Q8_1) {
        if ((e & 31) == 0) S[e >> 5] = s;
    } else {
        if ((e & 31) == 0) {
            S[2 * (e >> 5)] = s;
            S[2 * (e >> 5) + 1] = bsum32;
        }
    }
}

template <bool COH>
__device__ __forceinline__ void stage_x(const GemvProb &P, int m, uint32_t *lds, float *red) {
    const int K = P.K, U = units_of(P.type, K), type = P.type;
    const int n4 = K / 4;
    if (P.stage == kStageXq) {
        const uint8_t *xq = reinterpret_cast<const uint8_t *>(P.x) + (size_t)m * xq_stride((size_t)K);
        const uint32_t *qh = reinterpret_cast<const uint32_t *>(xq);
        const uint32_t *ql = reinterpret_cast<const uint32_t *>(xq + K);
        const float *xs = reinterpret_cast<const float *>(xq + 2 * (size_t)K);
        const float *xb = xs + K / 32;
        if (gemv_float_weights(type)) {
            // unquantized weights take x back as f32: x = s * (128 * high part + low part)
            float4 *xf = reinterpret_cast<float4 *>(lds);
            for (int i = threadIdx.x; i < n4; i += (int)blockDim.x) {
                const float s = xs[i >> 3];
                const uint32_t hi = qh[i], lo = ql[i];
                xf[i] = make_float4(s * (float)(((int)(int8_t)(hi & 0xFF) << 7) + (int)(lo & 127)),
                                    s * (float)(((int)(int8_t)((hi >> 8) & 0xFF) << 7) + (int)((lo >> 8) & 127)),
                                    s * (float)(((int)(int8_t)((hi >> 16) & 0xFF) << 7) + (int)((lo >> 16) & 127)),
                                    s * (float)(((int)(int8_t)(hi >> 24) << 7) + (int)((lo >> 24) & 127)));
            }
        } else
        for (int i = threadIdx.x; i < n4; i += (int)blockDim.x) {
            int e = 4 * i;
            float s = 0.f, b16 = 0.f, b32 = 0.f;
            if ((e & 15) == 0) {
                s = xs[e >> 5];
                b16 = xb[e >> 4];
                if ((e & 31) == 0) b32 = b16 + xb[(e >> 4) + 1];
            }
            stage_store(type, K, U, lds, e, qh[i], ql[i], s, b16, b32);
        }
    } else {
        const float *x = reinterpret_cast<const float *>(P.x) + (size_t)m * K;
        float rms = 1.f;
        if (P.stage == kStageRms) {
            float ss = 0.f;
            for (int i = threadIdx.x; i < n4; i += (int)blockDim.x) {
                float4 v = ld_f4<COH>(x + 4 * i);
                ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
            }
            ss = block_sum(ss, red);
            rms = sqrtf(ss / (float)K + P.eps);
        }
        const float4 *g4 = reinterpret_cast<const float4 *>(P.gamma);
        // K % 32 == 0 and blockDim.x % 8 == 0: the 8 lanes of a 32-block enter and leave this loop together
        for (int i = threadIdx.x; i < n4; i += (int)blockDim.x) {
            float4 v = ld_f4<COH>(x + 4 * i);
            if (P.stage == kStageRms) {
                float4 g = g4[i];
                v = make_float4(g.x * (v.x / rms), g.y * (v.y / rms), g.z * (v.z / rms), g.w * (v.w / rms));
            }
            if (gemv_float_weights(type)) {
                reinterpret_cast<float4 *>(lds)[i] = v;
                continue;
            }
            Q4Pack p = quantize4(v);
            stage_store(type, K, U, lds, 4 * i, p.hi, p.lo, p.s, p.s * (float)p.sum16, p.s * (float)p.sum32);
        }
    }
    __syncthreads();
}

// ---- per-type register images of one unit of one weight row, of the matching x slice, and their dot ----

template <int TYPE> struct WRegs;
template <int TYPE> struct XRegs;

template <> struct WRegs<RT_GGML_Q4_K> { uint4 hdr, qa, qb; };
template <> struct XRegs<RT_GGML_Q4_K> { uint4 h[4], l[4]; float4 sv; };
template <> struct WRegs<RT_GGML_Q5_K> { uint4 hdr, ha, hb, qa, qb; };     // header, the 32 bytes of fifth bits, the unit's 32 nibble bytes
template <> struct XRegs<RT_GGML_Q5_K> : XRegs<RT_GGML_Q4_K> {};              // same 64-element units, same x slice
template <> struct WRegs<RT_GGML_Q6_K> { uint4 A, B, H; uint2 sc; uint32_t d; };
template <> struct XRegs<RT_GGML_Q6_K> { uint4 h[4], l[4]; float4 xs, xb; };
template <> struct WRegs<RT_GGML_Q8_0> { uint4 a, b; uint32_t d; };
template <> struct XRegs<RT_GGML_Q8_0> { uint4 h[2], l[2]; float s; };
template <> struct WRegs<RT_GGML_Q4_0> { uint4 a; uint32_t d; };
// Q8_1: a Q8_0 block with a second half word (d * sum of the quants) between the scale and the quants: same registers, same x slice
template <> struct WRegs<RT_GGML_Q8_1> : WRegs<RT_GGML_Q8_0> {};
template <> struct XRegs<RT_GGML_Q8_1> : XRegs<RT_GGML_Q8_0> {};
template <> struct XRegs<RT_GGML_Q4_0> { uint4 h[2], l[2]; float2 sv; };
// Q3_K: a unit is, as for Q6_K, 16 byte positions x 4 runs of one half of a super-block (element 128 n + 32 j + 16 c + i):
// the same x slice; 16 bytes of 2-bit fields, 16 bytes of third bits, the 12 scale bytes, d
template <> struct WRegs<RT_GGML_Q3_K> { uint4 Q, H; uint2 s01; uint32_t s2, d; };
template <> struct XRegs<RT_GGML_Q3_K> : XRegs<RT_GGML_Q6_K> {};
// Q2_K: the same unit and x slice again; 16 bytes of 2-bit fields, the eight scale bytes of the half, d | dmin << 16
template <> struct WRegs<RT_GGML_Q2_K> { uint4 Q; uint2 sc; uint32_t dm; };
template <> struct XRegs<RT_GGML_Q2_K> : XRegs<RT_GGML_Q6_K> {};
// unquantized rows: 16 bytes of weights per unit against the f32 x in LDS
template <> struct WRegs<RT_GGML_F16> { uint4 q; };
template <> struct XRegs<RT_GGML_F16> { float4 a, b; };
template <> struct WRegs<RT_GGML_F32> { uint4 q; };
template <> struct XRegs<RT_GGML_F32> { float4 a; };
// Q4_1 / Q5_0 / Q5_1: 32-element blocks like Q4_0 (same x slice), with an offset m and / or a word of fifth bits
template <> struct WRegs<RT_GGML_Q4_1> { uint4 a; uint32_t dm; };           // d | m << 16
template <> struct WRegs<RT_GGML_Q5_0> { uint4 a; uint32_t d, qh; };
template <> struct WRegs<RT_GGML_Q5_1> { uint4 a; uint32_t dm, qh; };
template <> struct XRegs<RT_GGML_Q4_1> : XRegs<RT_GGML_Q4_0> {};
template <> struct XRegs<RT_GGML_Q5_0> : XRegs<RT_GGML_Q4_0> {};
template <> struct XRegs<RT_GGML_Q5_1> : XRegs<RT_GGML_Q4_0> {};

// Weight loads go through a buffer resource made for the piece of the matrix a wave step may read (a row, or one pass of
// a row): the resource starts at the piece's first byte and its num_records is the piece's length, so the hardware's range
// check holds every lane inside the piece whatever its 32-bit vector offset turns out to be -- a lane that is out of range
// reads zeros (a failed comparison in a test) instead of touching memory that may not be mapped.  The piece itself is
// placed by wave-uniform scalar arithmetic and clamped to the tensor, so no load of these kernels can leave the tensor.
// No 64-bit address arithmetic per load: the lane's place in the piece is the vector offset.
//
// The start is rounded down to a multiple of four bytes (rows of Q6_K at K = 11008 are 9030 bytes: only 2-byte aligned)
// and the remainder goes into the scalar offset, with num_records lengthened by it: whether the range check counts the
// scalar offset or not, every in-range lane passes it.  num_records is lengthened by kWindowSlack more, so that no rule a
// range check may follow (the access as a whole, dword by dword, sub-dword loads widened to a dword) can refuse the last
// bytes of a piece that is not a whole number of dwords -- a 2-byte scale at offset 9028 of a 9030-byte row.  A lane that
// is out of range can then get kWindowSlack + 3 bytes past the piece and no further: inside the 64 bytes every upload
// leaves behind a tensor.  (The CPU build of these sources sets the slack to zero: there a load ends the run the moment it
// leaves the piece.)
#ifdef RT_EMULATED
constexpr uint32_t kWindowSlack = 0;
#else
constexpr uint32_t kWindowSlack = 16;
#endif
struct WRow {
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t soff;      // 0..3: what the rounding of the start took off
};
// w: the tensor; nbytes: its size (N * row_bytes < 4 GB, checked at launch); start: byte offset of the piece; span: its length
// (nbytes >= span).  All arguments wave-uniform.
__device__ __forceinline__ WRow weight_window(const uint8_t *w, uint32_t nbytes, uint32_t start, uint32_t span) {
    start = min(start, nbytes - span);      // unsigned: a start that went wrong in any direction lands inside the tensor
    const uint32_t rem = start & 3u;
    // raw buffer (stride 0), dword 3 as for 32-bit data
    return WRow{ __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(w) + (start - rem), 0, (int)(span + rem + kWindowSlack), 0x00020000), rem };
}
__device__ __forceinline__ uint4 bld16(WRow r, uint32_t off) {
    return __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(r.rsrc, off, r.soff, 0));
}
__device__ __forceinline__ uint2 bld8(WRow r, uint32_t off) {
    return __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(r.rsrc, off, r.soff, 0));
}
__device__ __forceinline__ uint32_t bld4(WRow r, uint32_t off) {
    return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r.rsrc, off, r.soff, 0);
}
__device__ __forceinline__ uint32_t bld2(WRow r, uint32_t off) {
    return (uint32_t)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r.rsrc, off, r.soff, 0);
}

__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q4_K> &w, WRow row, int u) {
    uint32_t off = (uint32_t)(u >> 2) * 144u, g = (uint32_t)(u & 3);
    w.hdr = bld16(row, off);
    w.qa = bld16(row, off + 16u + 32u * g);
    w.qb = bld16(row, off + 32u + 32u * g);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q5_K> &w, WRow row, int u) {
    uint32_t off = (uint32_t)(u >> 2) * 176u, g = (uint32_t)(u & 3);
    w.hdr = bld16(row, off);
    w.ha = bld16(row, off + 16u);
    w.hb = bld16(row, off + 32u);
    w.qa = bld16(row, off + 48u + 32u * g);
    w.qb = bld16(row, off + 64u + 32u * g);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q6_K> &w, WRow row, int u) {
    uint32_t off = (uint32_t)(u >> 2) * 210u, h = (uint32_t)((u >> 1) & 1), c = (uint32_t)(u & 1);
    w.A = bld16(row, off + 64u * h + 16u * c);
    w.B = bld16(row, off + 64u * h + 32u + 16u * c);
    w.H = bld16(row, off + 128u + 32u * h + 16u * c);
    w.sc = bld8(row, off + 192u + 8u * h);
    w.d = bld2(row, off + 208u);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q2_K> &w, WRow row, int u) {
    uint32_t off = (uint32_t)(u >> 2) * 84u, n = (uint32_t)((u >> 1) & 1), c = (uint32_t)(u & 1);
    w.sc = bld8(row, off + 8u * n);
    w.Q = bld16(row, off + 16u + 32u * n + 16u * c);
    w.dm = bld4(row, off + 80u);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q3_K> &w, WRow row, int u) {
    uint32_t off = (uint32_t)(u >> 2) * 110u, n = (uint32_t)((u >> 1) & 1), c = (uint32_t)(u & 1);
    w.H = bld16(row, off + 16u * c);
    w.Q = bld16(row, off + 32u + 32u * n + 16u * c);
    w.s01 = bld8(row, off + 96u);
    w.s2 = bld2(row, off + 104u) | (bld2(row, off + 106u) << 16);
    w.d = bld2(row, off + 108u);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q8_0> &w, WRow row, int u) {
    uint32_t off = (uint32_t)u * 34u;
    w.d = bld2(row, off);
    w.a = bld16(row, off + 2u);
    w.b = bld16(row, off + 18u);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q8_1> &w, WRow row, int u) {
    uint32_t off = (uint32_t)u * 36u;
    w.d = bld2(row, off);
    w.a = bld16(row, off + 4u);
    w.b = bld16(row, off + 20u);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q4_0> &w, WRow row, int u) {
    uint32_t off = (uint32_t)u * 18u;
    w.d = bld2(row, off);
    w.a = bld16(row, off + 2u);
}

__device__ __forceinline__ void load_w(WRegs<RT_GGML_F16> &w, WRow row, int u) { w.q = bld16(row, (uint32_t)u * 16u); }
__device__ __forceinline__ void load_w(WRegs<RT_GGML_F32> &w, WRow row, int u) { w.q = bld16(row, (uint32_t)u * 16u); }
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q4_1> &w, WRow row, int u) {
    uint32_t off = (uint32_t)u * 20u;
    w.dm = bld4(row, off);
    w.a = bld16(row, off + 4u);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q5_0> &w, WRow row, int u) {
    uint32_t off = (uint32_t)u * 22u;
    w.d = bld2(row, off);
    w.qh = bld2(row, off + 2u) | (bld2(row, off + 4u) << 16);
    w.a = bld16(row, off + 6u);
}
__device__ __forceinline__ void load_w(WRegs<RT_GGML_Q5_1> &w, WRow row, int u) {
    uint32_t off = (uint32_t)u * 24u;
    w.dm = bld4(row, off);
    w.qh = bld4(row, off + 4u);
    w.a = bld16(row, off + 8u);
}

__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q4_K> &x, const uint32_t *lds, int u, int U, int K) {
    const uint4 *XH = reinterpret_cast<const uint4 *>(lds);
    const uint4 *XL = XH + K / 16;
#pragma unroll
    for (int c = 0; c < 4; c++) { x.h[c] = XH[c * U + u]; x.l[c] = XL[c * U + u]; }
    x.sv = reinterpret_cast<const float4 *>(lds + K / 2)[u];
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q5_K> &x, const uint32_t *lds, int u, int U, int K) {
    load_x(static_cast<XRegs<RT_GGML_Q4_K> &>(x), lds, u, U, K);
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q6_K> &x, const uint32_t *lds, int u, int U, int K) {
    const uint4 *XH = reinterpret_cast<const uint4 *>(lds);
    const uint4 *XL = XH + K / 16;
#pragma unroll
    for (int r = 0; r < 4; r++) { x.h[r] = XH[r * U + u]; x.l[r] = XL[r * U + u]; }
    const float *S = reinterpret_cast<const float *>(lds + K / 2);
    x.xs = reinterpret_cast<const float4 *>(S)[u >> 1];
    x.xb = reinterpret_cast<const float4 *>(S + 2 * U)[u];
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q2_K> &x, const uint32_t *lds, int u, int U, int K) {
    load_x(static_cast<XRegs<RT_GGML_Q6_K> &>(x), lds, u, U, K);
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q3_K> &x, const uint32_t *lds, int u, int U, int K) {
    load_x(static_cast<XRegs<RT_GGML_Q6_K> &>(x), lds, u, U, K);
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q8_0> &x, const uint32_t *lds, int u, int U, int K) {
    const uint4 *XH = reinterpret_cast<const uint4 *>(lds);
    const uint4 *XL = XH + K / 16;
    x.h[0] = XH[u]; x.h[1] = XH[U + u]; x.l[0] = XL[u]; x.l[1] = XL[U + u];
    x.s = reinterpret_cast<const float *>(lds + K / 2)[u];
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q8_1> &x, const uint32_t *lds, int u, int U, int K) {
    load_x(static_cast<XRegs<RT_GGML_Q8_0> &>(x), lds, u, U, K);
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q4_0> &x, const uint32_t *lds, int u, int U, int K) {
    const uint4 *XH = reinterpret_cast<const uint4 *>(lds);
    const uint4 *XL = XH + K / 16;
    x.h[0] = XH[u]; x.h[1] = XH[U + u]; x.l[0] = XL[u]; x.l[1] = XL[U + u];
    x.sv = reinterpret_cast<const float2 *>(lds + K / 2)[u];
}

__device__ __forceinline__ void load_x(XRegs<RT_GGML_F16> &x, const uint32_t *lds, int u, int, int) {
    x.a = reinterpret_cast<const float4 *>(lds)[2 * u];
    x.b = reinterpret_cast<const float4 *>(lds)[2 * u + 1];
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_F32> &x, const uint32_t *lds, int u, int, int) {
    x.a = reinterpret_cast<const float4 *>(lds)[u];
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q4_1> &x, const uint32_t *lds, int u, int U, int K) {
    load_x(static_cast<XRegs<RT_GGML_Q4_0> &>(x), lds, u, U, K);
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q5_0> &x, const uint32_t *lds, int u, int U, int K) {
    load_x(static_cast<XRegs<RT_GGML_Q4_0> &>(x), lds, u, U, K);
}
__device__ __forceinline__ void load_x(XRegs<RT_GGML_Q5_1> &x, const uint32_t *lds, int u, int U, int K) {
    load_x(static_cast<XRegs<RT_GGML_Q4_0> &>(x), lds, u, U, K);
}

#define RT_W4(v) { (v).x, (v).y, (v).z, (v).w }

// The float tails of the dot products are written with explicit fused operations and contraction off, so
// that every instantiation (one or two rows per step, any staging mode) rounds the same way: a row's result
// does not depend on which code path computed it.
#pragma clang fp contract(off)

__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q4_K> &w, const XRegs<RT_GGML_Q4_K> &x, int u) {
    const int g = u & 3;
    uint32_t scw, mw;
    if (g < 2) {
        scw = w.hdr.y & 0x3f3f3f3fu;
        mw = w.hdr.z & 0x3f3f3f3fu;
    } else {
        scw = (w.hdr.w & 0x0f0f0f0fu) | ((w.hdr.y >> 2) & 0x30303030u);
        mw = ((w.hdr.w >> 4) & 0x0f0f0f0fu) | ((w.hdr.z >> 2) & 0x30303030u);
    }
    const int sh = (g & 1) * 16;
    scw >>= sh;
    mw >>= sh;
    float sc0 = (float)(scw & 0xFF), sc1 = (float)((scw >> 8) & 0xFF);
    float m0 = (float)(mw & 0xFF), m1 = (float)((mw >> 8) & 0xFF);
    float d = h2f(w.hdr.x & 0xFFFF), dmin = h2f(w.hdr.x >> 16);
    const uint32_t q[8] = { w.qa.x, w.qa.y, w.qa.z, w.qa.w, w.qb.x, w.qb.y, w.qb.z, w.qb.w };
    const uint32_t hlo[8] = { x.h[0].x, x.h[0].y, x.h[0].z, x.h[0].w, x.h[1].x, x.h[1].y, x.h[1].z, x.h[1].w };
    const uint32_t hhi[8] = { x.h[2].x, x.h[2].y, x.h[2].z, x.h[2].w, x.h[3].x, x.h[3].y, x.h[3].z, x.h[3].w };
    const uint32_t llo[8] = { x.l[0].x, x.l[0].y, x.l[0].z, x.l[0].w, x.l[1].x, x.l[1].y, x.l[1].z, x.l[1].w };
    const uint32_t lhi[8] = { x.l[2].x, x.l[2].y, x.l[2].z, x.l[2].w, x.l[3].x, x.l[3].y, x.l[3].z, x.l[3].w };
    int dh0 = 0, dl0 = 0, dh1 = 0, dl1 = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint32_t lo = q[i] & 0x0f0f0f0fu, hi = (q[i] >> 4) & 0x0f0f0f0fu;
        dh0 = sdot4(lo, (int)hlo[i], dh0);
        dl0 = sdot4(lo, (int)llo[i], dl0);
        dh1 = sdot4(hi, (int)hhi[i], dh1);
        dl1 = sdot4(hi, (int)lhi[i], dl1);
    }
    float t0 = (float)((dh0 << 7) + dl0), t1 = (float)((dh1 << 7) + dl1);
    const float pos = __builtin_fmaf(sc0, x.sv.x * t0, sc1 * (x.sv.y * t1)), neg = __builtin_fmaf(m0, x.sv.z, m1 * x.sv.w);
    return __builtin_fmaf(d, pos, -(dmin * neg));
}

// Q5_K: the Q4_K unit with the fifth bit of every element taken from qh (bit 2g of byte l for the low-nibble
// sub-block of unit g, bit 2g+1 for the high-nibble one); values 0..31, the -min term as in Q4_K.
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q5_K> &w, const XRegs<RT_GGML_Q5_K> &x, int u) {
    const int g = u & 3;
    uint32_t scw, mw;
    if (g < 2) {
        scw = w.hdr.y & 0x3f3f3f3fu;
        mw = w.hdr.z & 0x3f3f3f3fu;
    } else {
        scw = (w.hdr.w & 0x0f0f0f0fu) | ((w.hdr.y >> 2) & 0x30303030u);
        mw = ((w.hdr.w >> 4) & 0x0f0f0f0fu) | ((w.hdr.z >> 2) & 0x30303030u);
    }
    const int sh = (g & 1) * 16;
    scw >>= sh;
    mw >>= sh;
    float sc0 = (float)(scw & 0xFF), sc1 = (float)((scw >> 8) & 0xFF);
    float m0 = (float)(mw & 0xFF), m1 = (float)((mw >> 8) & 0xFF);
    float d = h2f(w.hdr.x & 0xFFFF), dmin = h2f(w.hdr.x >> 16);
    const uint32_t q[8] = { w.qa.x, w.qa.y, w.qa.z, w.qa.w, w.qb.x, w.qb.y, w.qb.z, w.qb.w };
    const uint32_t hb[8] = { w.ha.x, w.ha.y, w.ha.z, w.ha.w, w.hb.x, w.hb.y, w.hb.z, w.hb.w };
    const uint32_t hlo[8] = { x.h[0].x, x.h[0].y, x.h[0].z, x.h[0].w, x.h[1].x, x.h[1].y, x.h[1].z, x.h[1].w };
    const uint32_t hhi[8] = { x.h[2].x, x.h[2].y, x.h[2].z, x.h[2].w, x.h[3].x, x.h[3].y, x.h[3].z, x.h[3].w };
    const uint32_t llo[8] = { x.l[0].x, x.l[0].y, x.l[0].z, x.l[0].w, x.l[1].x, x.l[1].y, x.l[1].z, x.l[1].w };
    const uint32_t lhi[8] = { x.l[2].x, x.l[2].y, x.l[2].z, x.l[2].w, x.l[3].x, x.l[3].y, x.l[3].z, x.l[3].w };
    int dh0 = 0, dl0 = 0, dh1 = 0, dl1 = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t bits = hb[i] >> (2 * g);      // bit 0 of each byte: fifth bit of the low-nibble element, bit 1: of the high-nibble one
        uint32_t lo = (q[i] & 0x0f0f0f0fu) | ((bits << 4) & 0x10101010u);
        uint32_t hi = ((q[i] >> 4) & 0x0f0f0f0fu) | ((bits << 3) & 0x10101010u);
        dh0 = sdot4(lo, (int)hlo[i], dh0);
        dl0 = sdot4(lo, (int)llo[i], dl0);
        dh1 = sdot4(hi, (int)hhi[i], dh1);
        dl1 = sdot4(hi, (int)lhi[i], dl1);
    }
    float t0 = (float)((dh0 << 7) + dl0), t1 = (float)((dh1 << 7) + dl1);
    const float pos = __builtin_fmaf(sc0, x.sv.x * t0, sc1 * (x.sv.y * t1)), neg = __builtin_fmaf(m0, x.sv.z, m1 * x.sv.w);
    return __builtin_fmaf(d, pos, -(dmin * neg));
}

__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q6_K> &w, const XRegs<RT_GGML_Q6_K> &x, int u) {
    const int s8 = (u & 1) * 8;
    const uint32_t A[4] = RT_W4(w.A), B[4] = RT_W4(w.B), H[4] = RT_W4(w.H);
    const uint32_t h0[4] = RT_W4(x.h[0]), h1[4] = RT_W4(x.h[1]), h2[4] = RT_W4(x.h[2]), h3[4] = RT_W4(x.h[3]);
    const uint32_t l0[4] = RT_W4(x.l[0]), l1[4] = RT_W4(x.l[1]), l2[4] = RT_W4(x.l[2]), l3[4] = RT_W4(x.l[3]);
    int dh[4] = { 0, 0, 0, 0 }, dl[4] = { 0, 0, 0, 0 };
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t q1 = (A[i] & 0x0f0f0f0fu) | ((H[i] << 4) & 0x30303030u);
        uint32_t q2 = (B[i] & 0x0f0f0f0fu) | ((H[i] << 2) & 0x30303030u);
        uint32_t q3 = ((A[i] >> 4) & 0x0f0f0f0fu) | (H[i] & 0x30303030u);
        uint32_t q4 = ((B[i] >> 4) & 0x0f0f0f0fu) | ((H[i] >> 2) & 0x30303030u);
        dh[0] = sdot4(q1, (int)h0[i], dh[0]);  dl[0] = sdot4(q1, (int)l0[i], dl[0]);
        dh[1] = sdot4(q2, (int)h1[i], dh[1]);  dl[1] = sdot4(q2, (int)l1[i], dl[1]);
        dh[2] = sdot4(q3, (int)h2[i], dh[2]);  dl[2] = sdot4(q3, (int)l2[i], dl[2]);
        dh[3] = sdot4(q4, (int)h3[i], dh[3]);  dl[3] = sdot4(q4, (int)l3[i], dl[3]);
    }
    uint32_t s01 = w.sc.x >> s8, s23 = w.sc.y >> s8;
    float sc0 = (float)(int)(int8_t)(s01 & 0xFF), sc1 = (float)(int)(int8_t)((s01 >> 16) & 0xFF);
    float sc2 = (float)(int)(int8_t)(s23 & 0xFF), sc3 = (float)(int)(int8_t)((s23 >> 16) & 0xFF);
    float a = sc0 * __builtin_fmaf(x.xs.x, (float)((dh[0] << 7) + dl[0]), -32.f * x.xb.x);
    a = __builtin_fmaf(sc1, __builtin_fmaf(x.xs.y, (float)((dh[1] << 7) + dl[1]), -32.f * x.xb.y), a);
    a = __builtin_fmaf(sc2, __builtin_fmaf(x.xs.z, (float)((dh[2] << 7) + dl[2]), -32.f * x.xb.z), a);
    a = __builtin_fmaf(sc3, __builtin_fmaf(x.xs.w, (float)((dh[3] << 7) + dl[3]), -32.f * x.xb.w), a);
    return h2f(w.d) * a;
}

// Q2_K: run j of the unit holds the 2-bit fields j of 16 bytes; its scale byte is number 2 j + c of the half's eight
// (low nibble: scale, high nibble: minimum).  y = d * scale * q - dmin * minimum.
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q2_K> &w, const XRegs<RT_GGML_Q2_K> &x, int u) {
    const int c = u & 1;
    const uint32_t Q[4] = RT_W4(w.Q);
    const uint32_t h0[4] = RT_W4(x.h[0]), h1[4] = RT_W4(x.h[1]), h2[4] = RT_W4(x.h[2]), h3[4] = RT_W4(x.h[3]);
    const uint32_t l0[4] = RT_W4(x.l[0]), l1[4] = RT_W4(x.l[1]), l2[4] = RT_W4(x.l[2]), l3[4] = RT_W4(x.l[3]);
    int dh[4] = { 0, 0, 0, 0 }, dl[4] = { 0, 0, 0, 0 };
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t q0 = Q[i] & 0x03030303u, q1 = (Q[i] >> 2) & 0x03030303u, q2 = (Q[i] >> 4) & 0x03030303u, q3 = (Q[i] >> 6) & 0x03030303u;
        dh[0] = sdot4(q0, (int)h0[i], dh[0]);  dl[0] = sdot4(q0, (int)l0[i], dl[0]);
        dh[1] = sdot4(q1, (int)h1[i], dh[1]);  dl[1] = sdot4(q1, (int)l1[i], dl[1]);
        dh[2] = sdot4(q2, (int)h2[i], dh[2]);  dl[2] = sdot4(q2, (int)l2[i], dl[2]);
        dh[3] = sdot4(q3, (int)h3[i], dh[3]);  dl[3] = sdot4(q3, (int)l3[i], dl[3]);
    }
    const uint32_t b01 = w.sc.x >> (8 * c), b23 = w.sc.y >> (8 * c);      // bytes c, c + 2 of each word: runs 0, 1 | 2, 3
    const float s0 = (float)(b01 & 0xFu), s1 = (float)((b01 >> 16) & 0xFu), s2 = (float)(b23 & 0xFu), s3 = (float)((b23 >> 16) & 0xFu);
    const float m0 = (float)((b01 >> 4) & 0xFu), m1 = (float)((b01 >> 20) & 0xFu), m2 = (float)((b23 >> 4) & 0xFu), m3 = (float)((b23 >> 20) & 0xFu);
    float pos = s0 * (x.xs.x * (float)((dh[0] << 7) + dl[0]));
    pos = __builtin_fmaf(s1, x.xs.y * (float)((dh[1] << 7) + dl[1]), pos);
    pos = __builtin_fmaf(s2, x.xs.z * (float)((dh[2] << 7) + dl[2]), pos);
    pos = __builtin_fmaf(s3, x.xs.w * (float)((dh[3] << 7) + dl[3]), pos);
    float neg = m0 * x.xb.x;
    neg = __builtin_fmaf(m1, x.xb.y, neg);
    neg = __builtin_fmaf(m2, x.xb.z, neg);
    neg = __builtin_fmaf(m3, x.xb.w, neg);
    return __builtin_fmaf(h2f(w.dm & 0xFFFFu), pos, -(h2f(w.dm >> 16) * neg));
}

// Run j of the unit: stored value v = 2-bit field j of the byte | third bit (bit 4 n + j of the hmask byte) << 2, element = v - 4;
// its scale is number 8 n + 2 j + c of the 16: low four bits in nibble n of scale byte 2 j + c, high two in bits
// 2 (2 n + j / 2) .. of scale byte 8 + (2 j + c) % 4.
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q3_K> &w, const XRegs<RT_GGML_Q3_K> &x, int u) {
    const int n = (u >> 1) & 1, c = u & 1;
    const uint32_t Q[4] = RT_W4(w.Q), H[4] = RT_W4(w.H);
    const uint32_t h0[4] = RT_W4(x.h[0]), h1[4] = RT_W4(x.h[1]), h2[4] = RT_W4(x.h[2]), h3[4] = RT_W4(x.h[3]);
    const uint32_t l0[4] = RT_W4(x.l[0]), l1[4] = RT_W4(x.l[1]), l2[4] = RT_W4(x.l[2]), l3[4] = RT_W4(x.l[3]);
    int dh[4] = { 0, 0, 0, 0 }, dl[4] = { 0, 0, 0, 0 };
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t hb = H[i] >> (4 * n);
        uint32_t q0 = (Q[i] & 0x03030303u) | ((hb << 2) & 0x04040404u);
        uint32_t q1 = ((Q[i] >> 2) & 0x03030303u) | ((hb << 1) & 0x04040404u);
        uint32_t q2 = ((Q[i] >> 4) & 0x03030303u) | (hb & 0x04040404u);
        uint32_t q3 = ((Q[i] >> 6) & 0x03030303u) | ((hb >> 1) & 0x04040404u);
        dh[0] = sdot4(q0, (int)h0[i], dh[0]);  dl[0] = sdot4(q0, (int)l0[i], dl[0]);
        dh[1] = sdot4(q1, (int)h1[i], dh[1]);  dl[1] = sdot4(q1, (int)l1[i], dl[1]);
        dh[2] = sdot4(q2, (int)h2[i], dh[2]);  dl[2] = sdot4(q2, (int)l2[i], dl[2]);
        dh[3] = sdot4(q3, (int)h3[i], dh[3]);  dl[3] = sdot4(q3, (int)l3[i], dl[3]);
    }
    // scale bytes 2 j + c for j = 0..3: bytes c, c + 2 of the first word, then of the second; the high bits come from
    // bytes c, c + 2, c, c + 2 of the third word
    const uint32_t b01 = w.s01.x >> (8 * c), b23 = w.s01.y >> (8 * c), bh = w.s2 >> (8 * c);
    const uint32_t lo_a = (b01 >> (4 * n)) & 0x000f000fu, lo_b = (b23 >> (4 * n)) & 0x000f000fu;     // scales j = 0, 1 | 2, 3 in bytes 0 and 2
    const uint32_t hi_a = (bh >> (4 * n)) & 0x00030003u, hi_b = (bh >> (4 * n + 2)) & 0x00030003u;
    const uint32_t s_a = lo_a | (hi_a << 4), s_b = lo_b | (hi_b << 4);
    const float sc[4] = { (float)((int)(s_a & 0xFFu) - 32), (float)((int)(s_a >> 16) - 32), (float)((int)(s_b & 0xFFu) - 32),
                          (float)((int)(s_b >> 16) - 32) };
    float a = sc[0] * __builtin_fmaf(x.xs.x, (float)((dh[0] << 7) + dl[0]), -4.f * x.xb.x);
    a = __builtin_fmaf(sc[1], __builtin_fmaf(x.xs.y, (float)((dh[1] << 7) + dl[1]), -4.f * x.xb.y), a);
    a = __builtin_fmaf(sc[2], __builtin_fmaf(x.xs.z, (float)((dh[2] << 7) + dl[2]), -4.f * x.xb.z), a);
    a = __builtin_fmaf(sc[3], __builtin_fmaf(x.xs.w, (float)((dh[3] << 7) + dl[3]), -4.f * x.xb.w), a);
    return h2f(w.d) * a;
}

__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q8_0> &w, const XRegs<RT_GGML_Q8_0> &x, int) {
    const uint32_t q[8] = { w.a.x, w.a.y, w.a.z, w.a.w, w.b.x, w.b.y, w.b.z, w.b.w };
    const uint32_t xh[8] = { x.h[0].x, x.h[0].y, x.h[0].z, x.h[0].w, x.h[1].x, x.h[1].y, x.h[1].z, x.h[1].w };
    const uint32_t xl[8] = { x.l[0].x, x.l[0].y, x.l[0].z, x.l[0].w, x.l[1].x, x.l[1].y, x.l[1].z, x.l[1].w };
    int dh = 0, dl = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        dh = sdot4(q[i], (int)xh[i], dh);
        dl = sdot4(q[i], (int)xl[i], dl);
    }
    return h2f(w.d) * (x.s * __builtin_fmaf((float)dh, 128.f, (float)dl));
}

__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q8_1> &w, const XRegs<RT_GGML_Q8_1> &x, int u) {
    return dot_unit(static_cast<const WRegs<RT_GGML_Q8_0> &>(w), static_cast<const XRegs<RT_GGML_Q8_0> &>(x), u);
}
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q4_0> &w, const XRegs<RT_GGML_Q4_0> &x, int) {
    const uint32_t q[4] = RT_W4(w.a);
    const uint32_t hlo[4] = RT_W4(x.h[0]), hhi[4] = RT_W4(x.h[1]), llo[4] = RT_W4(x.l[0]), lhi[4] = RT_W4(x.l[1]);
    int dh = 0, dl = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t lo = q[i] & 0x0f0f0f0fu, hi = (q[i] >> 4) & 0x0f0f0f0fu;
        dh = sdot4(lo, (int)hlo[i], dh);
        dl = sdot4(lo, (int)llo[i], dl);
        dh = sdot4(hi, (int)hhi[i], dh);
        dl = sdot4(hi, (int)lhi[i], dl);
    }
    return h2f(w.d) * __builtin_fmaf(x.sv.x, (float)((dh << 7) + dl), -8.f * x.sv.y);
}
// Unquantized rows: products in element order, one fused multiply-add each.
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_F16> &w, const XRegs<RT_GGML_F16> &x, int) {
    const uint32_t q[4] = RT_W4(w.q);
    float a = h2f(q[0] & 0xFFFFu) * x.a.x;
    a = __builtin_fmaf(h2f(q[0] >> 16), x.a.y, a);
    a = __builtin_fmaf(h2f(q[1] & 0xFFFFu), x.a.z, a);
    a = __builtin_fmaf(h2f(q[1] >> 16), x.a.w, a);
    a = __builtin_fmaf(h2f(q[2] & 0xFFFFu), x.b.x, a);
    a = __builtin_fmaf(h2f(q[2] >> 16), x.b.y, a);
    a = __builtin_fmaf(h2f(q[3] & 0xFFFFu), x.b.z, a);
    a = __builtin_fmaf(h2f(q[3] >> 16), x.b.w, a);
    return a;
}
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_F32> &w, const XRegs<RT_GGML_F32> &x, int) {
    float a = __uint_as_float(w.q.x) * x.a.x;
    a = __builtin_fmaf(__uint_as_float(w.q.y), x.a.y, a);
    a = __builtin_fmaf(__uint_as_float(w.q.z), x.a.z, a);
    a = __builtin_fmaf(__uint_as_float(w.q.w), x.a.w, a);
    return a;
}

// The integer sums of a 32-element block against the two planes of x: nibbles of the 16 bytes, optionally with the
// fifth bits of qh (bit j: element j; the low nibbles are elements 0..15, the high ones 16..31).  Four bits of qh
// reach bit 4 of four bytes through one multiplication: bit k lands on 8k + 4 (and on places the mask drops).
template <bool FIFTH>
__device__ __forceinline__ int block32_dot(const uint4 &a, uint32_t qh, const XRegs<RT_GGML_Q4_0> &x) {
    const uint32_t q[4] = RT_W4(a);
    const uint32_t hlo[4] = RT_W4(x.h[0]), hhi[4] = RT_W4(x.h[1]), llo[4] = RT_W4(x.l[0]), lhi[4] = RT_W4(x.l[1]);
    int dh = 0, dl = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t lo = q[i] & 0x0f0f0f0fu, hi = (q[i] >> 4) & 0x0f0f0f0fu;
        if (FIFTH) {
            lo |= (((qh >> (4 * i)) & 15u) * 0x02040810u) & 0x10101010u;
            hi |= (((qh >> (16 + 4 * i)) & 15u) * 0x02040810u) & 0x10101010u;
        }
        dh = sdot4(lo, (int)hlo[i], dh);
        dl = sdot4(lo, (int)llo[i], dl);
        dh = sdot4(hi, (int)hhi[i], dh);
        dl = sdot4(hi, (int)lhi[i], dl);
    }
    return (dh << 7) + dl;      // below 2^24 in magnitude (32 elements x 31 x 127 x 128 + ...): exact as a float
}
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q4_1> &w, const XRegs<RT_GGML_Q4_1> &x, int) {
    const float t = x.sv.x * (float)block32_dot<false>(w.a, 0u, x);
    return __builtin_fmaf(h2f(w.dm & 0xFFFFu), t, h2f(w.dm >> 16) * x.sv.y);
}
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q5_0> &w, const XRegs<RT_GGML_Q5_0> &x, int) {
    return h2f(w.d) * __builtin_fmaf(x.sv.x, (float)block32_dot<true>(w.a, w.qh, x), -16.f * x.sv.y);
}
__device__ __forceinline__ float dot_unit(const WRegs<RT_GGML_Q5_1> &w, const XRegs<RT_GGML_Q5_1> &x, int) {
    const float t = x.sv.x * (float)block32_dot<true>(w.a, w.qh, x);
    return __builtin_fmaf(h2f(w.dm & 0xFFFFu), t, h2f(w.dm >> 16) * x.sv.y);
}
#pragma clang fp contract(fast)

// A wave walks "steps": step s = (row group s / n_iter, unit pass s % n_iter); a row group is R rows (with the
// SwiGLU epilogue: R/2 gate rows and their up rows).  Row groups are dealt round-robin over all waves that work
// on the problem.  The weight registers of step s+1 are requested before step s is consumed.
template <int TYPE, int R, bool COH>
struct Walker {
    const GemvProb &P;
    const uint32_t *lds;
    int m, U, n_iter, lane, gw, n_gw, n_groups, rows_per_group;
    bool dual;
    const uint8_t *w1, *w2;     // the matrix, and the second one of the gate / up pair form (else the same)
    uint32_t nbytes;            // size of a matrix

    // A step is (row group g, unit pass p); steps are walked in order, so the position is advanced, not divided out.
    struct Pos { int g, p; };
    __device__ __forceinline__ Pos first() const { return Pos{ gw, 0 }; }
    __device__ __forceinline__ Pos next(Pos q) const { return q.p + 1 == n_iter ? Pos{ q.g + n_gw, 0 } : Pos{ q.g, q.p + 1 }; }
    __device__ __forceinline__ int group_of(Pos q) const { return q.g; }
    __device__ __forceinline__ int unit_of(Pos q) const { return lane + 64 * q.p; }

    // rv: the residual values of the step's rows, requested with the weights so that the row end has no load
    // of its own to wait for (a wait for the youngest load would also wait for every prefetch before it)
    __device__ __forceinline__ void request(WRegs<TYPE> *w, float *rv, Pos s) const {
        const int g = group_of(s);
        const int u = min(unit_of(s), U - 1);  // lanes past the end of the row reread the last unit; masked later
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = dual ? g * rows_per_group + (r >> 1) : g * rows_per_group + r;
            row = min(row, P.N - 1);  // ragged tail: reread the last row, the store is skipped
            // a tensor is below 4 GB (checked at launch), so the row's byte offset fits 32 bits
            load_w(w[r], weight_window((dual && (r & 1)) ? w2 : w1, nbytes, (uint32_t)row * (uint32_t)P.row_bytes, (uint32_t)P.row_bytes), u);
            if (!dual && P.res) rv[r] = ld_f<COH>(&P.res[(size_t)m * P.N + row]);
        }
    }

    // x slice of the unit a lane works on in step s (rows of <= 64 units: the same slice in every step)
    __device__ __forceinline__ void fetch_x(XRegs<TYPE> &x, Pos s) const { load_x(x, lds, min(unit_of(s), U - 1), U, P.K); }

    __device__ __forceinline__ void consume(const WRegs<TYPE> *w, const float *rv, const XRegs<TYPE> &x, Pos s, float *acc) const {
        const int u = unit_of(s);
        const int uc = min(u, U - 1);
        const float live = u < U ? 1.f : 0.f;
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = __builtin_fmaf(live, dot_unit(w[r], x, uc), acc[r]);
        if (s.p != n_iter - 1) return;
        const int g = group_of(s);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = wave_sum_dpp(acc[r]);
        if (dual) {
#pragma unroll
            for (int r = 0; r < R / 2; r++) {
                int row = g * rows_per_group + r;
                if (lane == r && row < P.N) {
                    float gate = acc[2 * r], up = acc[2 * r + 1];
                    st_f<COH>(&P.y[(size_t)m * P.N + row], up * (gate * (1.0f / (1.0f + expf(-gate)))));
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < R; r++) {
                int row = g * rows_per_group + r;
                if (lane == r && row < P.N) {
                    size_t o = (size_t)m * P.N + row;
                    st_f<COH>(&P.y[o], P.res ? rv[r] + acc[r] : acc[r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0.f;
    }
};


// All rows of problem P that fall to workgroup `wg` of the `n_wg` workgroups sharing it.
template <int TYPE, int R, bool COH>
__device__ __forceinline__ void gemv_problem(const GemvProb &P, int wg, int n_wg, int m, uint32_t *lds, float *red) {
    const int waves = (int)(blockDim.x >> 6);
    Walker<TYPE, R, COH> W{ P, lds, m, units_of(TYPE, P.K), 0, (int)(threadIdx.x & 63), 0, 0, 0, 0, P.epi == kEpiSwiglu,
                            P.w, P.epi == kEpiSwiglu ? P.w2 : P.w, (uint32_t)P.N * (uint32_t)P.row_bytes };
    W.n_iter = (W.U + 63) / 64;
    W.rows_per_group = W.dual ? R / 2 : R;
    W.n_groups = (P.N + W.rows_per_group - 1) / W.rows_per_group;
    W.gw = wg * waves + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // wave-uniform: row addresses stay scalar
    W.n_gw = n_wg * waves;
    const int my_groups = W.gw < W.n_groups ? (W.n_groups - W.gw + W.n_gw - 1) / W.n_gw : 0;
    const int steps = my_groups * W.n_iter;
    WRegs<TYPE> a[R], b[R];
    float ra[R], rb[R];
#pragma unroll
    for (int r = 0; r < R; r++) ra[r] = rb[r] = 0.f;
    using Pos = typename Walker<TYPE, R, COH>::Pos;
    Pos pa = W.first(), pb = W.next(pa);     // positions of the steps held in a and b
    if (steps > 0) W.request(a, ra, pa);     // in flight while x is being staged
    stage_x<COH>(P, m, lds, red);
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
    XRegs<TYPE> x;
    if (R == 1 && W.n_iter == 1) {
        // every step of this lane meets the same x slice: keep it in registers, LDS is read once
        W.fetch_x(x, pa);
        for (int s = 0; s < steps; s += 2) {
            if (s + 1 < steps) W.request(b, rb, pb);
            W.consume(a, ra, x, pa, acc);
            pa = W.next(pb);
            if (s + 1 < steps) {
                if (s + 2 < steps) W.request(a, ra, pa);
                W.consume(b, rb, x, pb, acc);
                pb = W.next(pa);
            }
        }
    } else {
        for (int s = 0; s < steps; s += 2) {
            if (s + 1 < steps) W.request(b, rb, pb);
            W.fetch_x(x, pa);
            W.consume(a, ra, x, pa, acc);
            pa = W.next(pb);
            if (s + 1 < steps) {
                if (s + 2 < steps) W.request(a, ra, pa);
                W.fetch_x(x, pb);
                W.consume(b, rb, x, pb, acc);
                pb = W.next(pa);
            }
        }
    }
}

// Dispatch on the block format.  R2 picks two rows per wave step (always used by the SwiGLU epilogue).
template <bool COH, bool ALLOW_R2>
__device__ __forceinline__ void gemv_dispatch(const GemvProb &P, int wg, int n_wg, int m, bool r2, uint32_t *lds, float *red) {
    // Q5_K, Q3_K and Q2_K run one row per step (with a two-row form of any of them the kernel as a whole spills); the launcher
    // refuses the gate / up pair form for them, the caller issues gate and up as two problems and a separate SwiGLU
    if (P.type == RT_GGML_Q5_K) {
        gemv_problem<RT_GGML_Q5_K, 1, COH>(P, wg, n_wg, m, lds, red);
    } else if (P.type == RT_GGML_Q3_K) {
        gemv_problem<RT_GGML_Q3_K, 1, COH>(P, wg, n_wg, m, lds, red);
    } else if (P.type == RT_GGML_Q2_K) {
        gemv_problem<RT_GGML_Q2_K, 1, COH>(P, wg, n_wg, m, lds, red);
    } else if ((ALLOW_R2 && r2) || P.epi == kEpiSwiglu) {
        switch (P.type) {
        case RT_GGML_Q4_K: gemv_problem<RT_GGML_Q4_K, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q6_K: gemv_problem<RT_GGML_Q6_K, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q8_0: gemv_problem<RT_GGML_Q8_0, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q8_1: gemv_problem<RT_GGML_Q8_1, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q4_0: gemv_problem<RT_GGML_Q4_0, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q4_1: gemv_problem<RT_GGML_Q4_1, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q5_0: gemv_problem<RT_GGML_Q5_0, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q5_1: gemv_problem<RT_GGML_Q5_1, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_F16: gemv_problem<RT_GGML_F16, 2, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_F32: gemv_problem<RT_GGML_F32, 2, COH>(P, wg, n_wg, m, lds, red); break;
        }
    } else {
        switch (P.type) {
        case RT_GGML_Q4_K: gemv_problem<RT_GGML_Q4_K, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q6_K: gemv_problem<RT_GGML_Q6_K, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q8_0: gemv_problem<RT_GGML_Q8_0, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q8_1: gemv_problem<RT_GGML_Q8_1, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q4_0: gemv_problem<RT_GGML_Q4_0, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q4_1: gemv_problem<RT_GGML_Q4_1, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q5_0: gemv_problem<RT_GGML_Q5_0, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q5_1: gemv_problem<RT_GGML_Q5_1, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_F16: gemv_problem<RT_GGML_F16, 1, COH>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_F32: gemv_problem<RT_GGML_F32, 1, COH>(P, wg, n_wg, m, lds, red); break;
        }
    }
}

// The problem a workgroup of the grouped launch belongs to, as a local copy chosen by a chain of selects over the argument
// structure's fixed slots.  (Indexing the by-value argument with a run-time index, or handing it to a function by
// reference, makes the compiler copy all of it to private memory as soon as the kernel grows past some size; a private
// frame in this kernel slows every launch of it.)
#define RT_GEMV_PICK_PROBLEM(args, wg, P)                             \
    rt::GemvProb P = (args).p[0];                                     \
    _Pragma("unroll") for (int i_ = 1; i_ < rt::kMaxGemvProbs; i_++)  \
        if (i_ < (args).n && (wg) >= (args).p[i_].tile0) P = (args).p[i_]

}  // namespace rt
