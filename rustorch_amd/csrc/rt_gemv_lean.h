// The decode GEMV's own code path for the four block formats of the benchmark (Q4_K, Q6_K, Q8_0, Q4_0).
//
// Same x layout in LDS and the same dot-product arithmetic per unit as the general path in rt_gemv_device.h.  A row of one
// pass (up to 4096 elements of the K-quants) has the general path's bits; a longer row is the sum, in pass order, of
// its passes' wave sums (the general path sums each lane's passes first), whichever way the launch deals the passes out.
// Everything that does not depend on the row is taken out of the loop:
//   * what a lane needs to decode its unit -- the byte selector of its two 6-bit scales and minima, the
//     masks of the two packings of a Q4_K header, the scale bytes of its Q6_K runs -- is a lane constant
//     (a lane's unit index changes by 64 from pass to pass, so u & 3 never changes), and the decode is
//     branch-free: one byte permute per header word instead of a divergent if / else per row;
//   * the byte offset of the lane's unit inside a row is a lane constant plus a per-pass stride, the row
//     is a scalar offset of the buffer load: no address arithmetic per load;
// Only these formats are instantiated here, so their register budget is not set by the widest of the
// other eight.
#pragma once

#include "rt_gemv_device.h"

// What a wave does with a unit's registers; a timing harness may substitute a function that only touches them
// (loads, staging and stores kept, arithmetic dropped) to measure the memory side alone.
#ifndef RT_LEAN_DOT
#define RT_LEAN_DOT(lane_consts, w, x) lean_dot(lane_consts, w, x)
#endif

namespace rt {

// After x has been staged, once per problem: wait for every outstanding load.  The two weight requests that are in flight
// went out before the staging and its barrier, so they have landed or nearly.  What the wait buys is in the steady-state loop: the
// compiler's wait-count bookkeeping follows every path through the staging code at once, ends up holding some staging
// register for possibly still in flight, and -- where the loop reuses that register -- waits for *all* loads there, the
// prefetch just issued included (seen in the generated code of the Q6_K loops: vmcnt(0) in the first of the two steps and no wait
// in the second, against vmcnt(7), (6), (5) per step with this wait in place).
__device__ __forceinline__ void lean_settle_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }      // vmcnt(0), the other counters untouched

// The first product of an integer sum and the following ones.  (Through the compiler's own dot4, not inline assembly: the
// result of a dot instruction may only be read by another kind of vector instruction a few issue slots later, and the
// compiler keeps that distance only for instructions it can see.)
__device__ __forceinline__ int sdot4_first(uint32_t a, uint32_t b) { return __builtin_amdgcn_sdot4((int)a, (int)b, 0, false); }
__device__ __forceinline__ int sdot4_acc(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }

template <int TYPE> struct LeanLane;

// ---- Q4_K: unit = 64 elements = sub-blocks 2g, 2g+1 of a super-block (g = u & 3)
template <> struct LeanLane<RT_GGML_Q4_K> {
    uint32_t off_h, off_q;     // byte offsets inside the row of the header and of the 32 nibble bytes, pass 0
    uint32_t sel, mA, mB, mC;
    static constexpr uint32_t kPassBytes = 16u * 144u;     // 64 units further on
    __device__ __forceinline__ void init(int lane) {
        const uint32_t g = (uint32_t)lane & 3u, h = g & 1u;
        off_h = ((uint32_t)lane >> 2) * 144u;
        off_q = off_h + 16u + 32u * g;
        sel = 0x05040100u + 0x02020202u * h;              // bytes 2h, 2h+1 of the second operand, then of the first
        mA = g < 2 ? 0x3f3f3f3fu : 0u;
        mB = g < 2 ? 0u : 0x0f0f0f0fu;
        mC = g < 2 ? 0u : 0x30303030u;
    }
    __device__ __forceinline__ void load(WRegs<RT_GGML_Q4_K> &w, WRow row, uint32_t pass_off) const {
        w.hdr = bld16(row, off_h + pass_off);
        w.qa = bld16(row, off_q + pass_off);
        w.qb = bld16(row, off_q + pass_off + 16u);
    }
};

#pragma clang fp contract(off)
__device__ __forceinline__ float lean_dot(const LeanLane<RT_GGML_Q4_K> &c, const WRegs<RT_GGML_Q4_K> &w, const XRegs<RT_GGML_Q4_K> &x) {
    // header words: y = scales[0..3], z = scales[4..7], wd = scales[8..11].  For sub-blocks j < 4: sc = y_j & 63,
    // m = z_j & 63; for j >= 4: sc = (wd_{j-4} & 15) | (y_{j-4} >> 6) << 4, m = (wd_{j-4} >> 4) | (z_{j-4} >> 6) << 4.
    const uint32_t P = __builtin_amdgcn_perm(w.hdr.z, w.hdr.y, c.sel);                 // y_2h, y_2h+1, z_2h, z_2h+1
    const uint32_t Wx = __builtin_amdgcn_perm(w.hdr.w >> 4, w.hdr.w, c.sel);           // wd_2h, wd_2h+1, (wd >> 4)_2h, (wd >> 4)_2h+1
    const uint32_t S = (P & c.mA) | (Wx & c.mB) | ((P >> 2) & c.mC);                   // sc0, sc1, m0, m1
    const float sc0 = (float)(S & 0xFFu), sc1 = (float)((S >> 8) & 0xFFu), m0 = (float)((S >> 16) & 0xFFu), m1 = (float)(S >> 24);
    const float d = h2f(w.hdr.x & 0xFFFFu), dmin = h2f(w.hdr.x >> 16);
    const uint32_t q[8] = { w.qa.x, w.qa.y, w.qa.z, w.qa.w, w.qb.x, w.qb.y, w.qb.z, w.qb.w };
    const uint32_t hlo[8] = { x.h[0].x, x.h[0].y, x.h[0].z, x.h[0].w, x.h[1].x, x.h[1].y, x.h[1].z, x.h[1].w };
    const uint32_t hhi[8] = { x.h[2].x, x.h[2].y, x.h[2].z, x.h[2].w, x.h[3].x, x.h[3].y, x.h[3].z, x.h[3].w };
    const uint32_t llo[8] = { x.l[0].x, x.l[0].y, x.l[0].z, x.l[0].w, x.l[1].x, x.l[1].y, x.l[1].z, x.l[1].w };
    const uint32_t lhi[8] = { x.l[2].x, x.l[2].y, x.l[2].z, x.l[2].w, x.l[3].x, x.l[3].y, x.l[3].z, x.l[3].w };
    int dh0, dl0, dh1, dl1;
    {
        const uint32_t lo = q[0] & 0x0f0f0f0fu, hi = (q[0] >> 4) & 0x0f0f0f0fu;
        dh0 = sdot4_first(lo, hlo[0]);
        dl0 = sdot4_first(lo, llo[0]);
        dh1 = sdot4_first(hi, hhi[0]);
        dl1 = sdot4_first(hi, lhi[0]);
    }
#pragma unroll
    for (int i = 1; i < 8; i++) {
        const uint32_t lo = q[i] & 0x0f0f0f0fu, hi = (q[i] >> 4) & 0x0f0f0f0fu;
        dh0 = sdot4_acc(lo, hlo[i], dh0);
        dl0 = sdot4_acc(lo, llo[i], dl0);
        dh1 = sdot4_acc(hi, hhi[i], dh1);
        dl1 = sdot4_acc(hi, lhi[i], dl1);
    }
    const float t0 = (float)((dh0 << 7) + dl0), t1 = (float)((dh1 << 7) + dl1);
    const float pos = __builtin_fmaf(sc0, x.sv.x * t0, sc1 * (x.sv.y * t1)), neg = __builtin_fmaf(m0, x.sv.z, m1 * x.sv.w);
    return __builtin_fmaf(d, pos, -(dmin * neg));
}
#pragma clang fp contract(fast)

// ---- Q6_K: unit = 16 byte positions x 4 runs of one half of a super-block (u & 3 = 2 * half + c)
template <> struct LeanLane<RT_GGML_Q6_K> {
    uint32_t off_a, off_h, off_s, off_d;
    uint32_t sel;
    static constexpr uint32_t kPassBytes = 16u * 210u;
    __device__ __forceinline__ void init(int lane) {
        const uint32_t h = ((uint32_t)lane >> 1) & 1u, c = (uint32_t)lane & 1u, blk = ((uint32_t)lane >> 2) * 210u;
        off_a = blk + 64u * h + 16u * c;
        off_h = blk + 128u + 32u * h + 16u * c;
        off_s = blk + 192u + 8u * h;
        off_d = blk + 208u;
        sel = 0x06040200u + 0x01010101u * c;              // bytes c, c+2 of the second operand, then of the first
    }
    __device__ __forceinline__ void load(WRegs<RT_GGML_Q6_K> &w, WRow row, uint32_t pass_off) const {
        w.A = bld16(row, off_a + pass_off);
        w.B = bld16(row, off_a + pass_off + 32u);
        w.H = bld16(row, off_h + pass_off);
        w.sc = bld8(row, off_s + pass_off);
        w.d = bld2(row, off_d + pass_off);
    }
};

#pragma clang fp contract(off)
__device__ __forceinline__ float lean_dot(const LeanLane<RT_GGML_Q6_K> &c, const WRegs<RT_GGML_Q6_K> &w, const XRegs<RT_GGML_Q6_K> &x) {
    const uint32_t A[4] = RT_W4(w.A), B[4] = RT_W4(w.B), H[4] = RT_W4(w.H);
    const uint32_t h0[4] = RT_W4(x.h[0]), h1[4] = RT_W4(x.h[1]), h2[4] = RT_W4(x.h[2]), h3[4] = RT_W4(x.h[3]);
    const uint32_t l0[4] = RT_W4(x.l[0]), l1[4] = RT_W4(x.l[1]), l2[4] = RT_W4(x.l[2]), l3[4] = RT_W4(x.l[3]);
    int dh[4], dl[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t q1 = (A[i] & 0x0f0f0f0fu) | ((H[i] << 4) & 0x30303030u);
        const uint32_t q2 = (B[i] & 0x0f0f0f0fu) | ((H[i] << 2) & 0x30303030u);
        const uint32_t q3 = ((A[i] >> 4) & 0x0f0f0f0fu) | (H[i] & 0x30303030u);
        const uint32_t q4 = ((B[i] >> 4) & 0x0f0f0f0fu) | ((H[i] >> 2) & 0x30303030u);
        if (i == 0) {
            dh[0] = sdot4_first(q1, h0[0]);  dl[0] = sdot4_first(q1, l0[0]);
            dh[1] = sdot4_first(q2, h1[0]);  dl[1] = sdot4_first(q2, l1[0]);
            dh[2] = sdot4_first(q3, h2[0]);  dl[2] = sdot4_first(q3, l2[0]);
            dh[3] = sdot4_first(q4, h3[0]);  dl[3] = sdot4_first(q4, l3[0]);
        } else {
            dh[0] = sdot4_acc(q1, h0[i], dh[0]);  dl[0] = sdot4_acc(q1, l0[i], dl[0]);
            dh[1] = sdot4_acc(q2, h1[i], dh[1]);  dl[1] = sdot4_acc(q2, l1[i], dl[1]);
            dh[2] = sdot4_acc(q3, h2[i], dh[2]);  dl[2] = sdot4_acc(q3, l2[i], dl[2]);
            dh[3] = sdot4_acc(q4, h3[i], dh[3]);  dl[3] = sdot4_acc(q4, l3[i], dl[3]);
        }
    }
    // the scale of run r is byte c + 2 r of the half's eight
    const uint32_t S = __builtin_amdgcn_perm(w.sc.y, w.sc.x, c.sel);
    const float sc0 = (float)(int)(int8_t)(S & 0xFFu), sc1 = (float)(int)(int8_t)((S >> 8) & 0xFFu);
    const float sc2 = (float)(int)(int8_t)((S >> 16) & 0xFFu), sc3 = (float)(int)(int8_t)(S >> 24);
    float a = sc0 * __builtin_fmaf(x.xs.x, (float)((dh[0] << 7) + dl[0]), -32.f * x.xb.x);
    a = __builtin_fmaf(sc1, __builtin_fmaf(x.xs.y, (float)((dh[1] << 7) + dl[1]), -32.f * x.xb.y), a);
    a = __builtin_fmaf(sc2, __builtin_fmaf(x.xs.z, (float)((dh[2] << 7) + dl[2]), -32.f * x.xb.z), a);
    a = __builtin_fmaf(sc3, __builtin_fmaf(x.xs.w, (float)((dh[3] << 7) + dl[3]), -32.f * x.xb.w), a);
    return h2f(w.d) * a;
}
#pragma clang fp contract(fast)

// ---- Q8_0 / Q4_0: unit = one 32-element block
template <> struct LeanLane<RT_GGML_Q8_0> {
    uint32_t off;
    static constexpr uint32_t kPassBytes = 64u * 34u;
    __device__ __forceinline__ void init(int lane) { off = (uint32_t)lane * 34u; }
    __device__ __forceinline__ void load(WRegs<RT_GGML_Q8_0> &w, WRow row, uint32_t pass_off) const {
        w.d = bld2(row, off + pass_off);
        w.a = bld16(row, off + pass_off + 2u);
        w.b = bld16(row, off + pass_off + 18u);
    }
};
template <> struct LeanLane<RT_GGML_Q4_0> {
    uint32_t off;
    static constexpr uint32_t kPassBytes = 64u * 18u;
    __device__ __forceinline__ void init(int lane) { off = (uint32_t)lane * 18u; }
    __device__ __forceinline__ void load(WRegs<RT_GGML_Q4_0> &w, WRow row, uint32_t pass_off) const {
        w.d = bld2(row, off + pass_off);
        w.a = bld16(row, off + pass_off + 2u);
    }
};
__device__ __forceinline__ float lean_dot(const LeanLane<RT_GGML_Q8_0> &, const WRegs<RT_GGML_Q8_0> &w, const XRegs<RT_GGML_Q8_0> &x) {
    return dot_unit(w, x, 0);
}
__device__ __forceinline__ float lean_dot(const LeanLane<RT_GGML_Q4_0> &, const WRegs<RT_GGML_Q4_0> &w, const XRegs<RT_GGML_Q4_0> &x) {
    return dot_unit(w, x, 0);
}

// Staging of x in two halves.  `issue` sends the loads of the activation vector out before the first weight requests and
// `finish` writes LDS after them: a wave's loads complete in issue order, so x can be waited for while two steps of
// weights stay in flight behind it (requested the other way round, the wait for x would also be a wait for them, and
// nothing would be on its way while the workgroup stages).  Values, arithmetic and LDS layout are those of stage_x.
struct LeanStage {
    // 4 and 2 trips hold a whole row of up to 8192 elements with 512 threads (10 240 with 640); longer rows finish in the
    // loops below.  With 6 and 3 the kernel without the pair form needs 100 registers, with 4 and 2 it needs 91: under the 96
    // that five waves per SIMD leave each wave.
    static constexpr int NBQ = 4;      // trips of the ready-made form held in registers (5 words each)
    static constexpr int NBF = 2;      // trips of the f32 forms (a float4 of x and one of gamma each)
    uint32_t h[NBQ], l[NBQ];
    float s[NBQ], b0[NBQ], b1[NBQ];
    float4 v[NBF], g[NBF];

    __device__ __forceinline__ void issue(const GemvProb &P, int m) {
        const int K = P.K, n4 = K / 4, T = (int)blockDim.x, t = (int)threadIdx.x;
        if (P.stage == kStageXq) {
            const uint8_t *xq = reinterpret_cast<const uint8_t *>(P.x) + (size_t)m * xq_stride((size_t)K);
            const uint32_t *qh = reinterpret_cast<const uint32_t *>(xq), *ql = reinterpret_cast<const uint32_t *>(xq + K);
            const float *xs = reinterpret_cast<const float *>(xq + 2 * (size_t)K), *xb = xs + K / 32;
#pragma unroll
            for (int j = 0; j < NBQ; j++) {
                const int i = t + j * T;
                if (i < n4) { h[j] = qh[i]; l[j] = ql[i]; s[j] = xs[i >> 3]; b0[j] = xb[i >> 2]; b1[j] = xb[(i >> 2) | 1]; }
            }
        } else {
            const float4 *x4 = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(P.x) + (size_t)m * K);
            const float4 *g4 = reinterpret_cast<const float4 *>(P.gamma);
#pragma unroll
            for (int j = 0; j < NBF; j++) {
                const int i = t + j * T;
                if (i < n4) { v[j] = x4[i]; if (P.stage == kStageRms) g[j] = g4[i]; }
            }
        }
    }

    template <int TYPE>
    __device__ __forceinline__ void finish(const GemvProb &P, int m, uint32_t *lds, float *red) {
        const int K = P.K, U = units_of(TYPE, K), n4 = K / 4, T = (int)blockDim.x, t = (int)threadIdx.x;
        if (P.stage == kStageXq) {
#pragma unroll
            for (int j = 0; j < NBQ; j++) {
                const int i = t + j * T;
                if (i < n4) stage_store(TYPE, K, U, lds, 4 * i, h[j], l[j], s[j], b0[j], b0[j] + b1[j]);
            }
            if (n4 > NBQ * T) {
                const uint8_t *xq = reinterpret_cast<const uint8_t *>(P.x) + (size_t)m * xq_stride((size_t)K);
                const uint32_t *qh = reinterpret_cast<const uint32_t *>(xq), *ql = reinterpret_cast<const uint32_t *>(xq + K);
                const float *xs = reinterpret_cast<const float *>(xq + 2 * (size_t)K), *xb = xs + K / 32;
                for (int i = t + NBQ * T; i < n4; i += T) {
                    const float c0 = xb[i >> 2];
                    stage_store(TYPE, K, U, lds, 4 * i, qh[i], ql[i], xs[i >> 3], c0, c0 + xb[(i >> 2) | 1]);
                }
            }
        } else {
            const float4 *x4 = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(P.x) + (size_t)m * K);
            const float4 *g4 = reinterpret_cast<const float4 *>(P.gamma);
            float rms = 1.f;
            if (P.stage == kStageRms) {
                // the sum of squares in the order of stage_x: a thread's trips one after the other, then the block
                float ss = 0.f;
#pragma unroll
                for (int j = 0; j < NBF; j++) {
                    const int i = t + j * T;
                    if (i < n4) ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
                }
                for (int i = t + NBF * T; i < n4; i += T) {
                    const float4 w = x4[i];
                    ss += w.x * w.x + w.y * w.y + w.z * w.z + w.w * w.w;
                }
                ss = block_sum(ss, red);
                rms = sqrtf(ss / (float)K + P.eps);
            }
            // K % 32 == 0 and blockDim.x % 8 == 0: the 8 lanes of a 32-block take every branch here together
            auto put = [&](int i, float4 w, float4 gm) {
                if (P.stage == kStageRms) w = make_float4(gm.x * (w.x / rms), gm.y * (w.y / rms), gm.z * (w.z / rms), gm.w * (w.w / rms));
                const Q4Pack p = quantize4(w);
                stage_store(TYPE, K, U, lds, 4 * i, p.hi, p.lo, p.s, p.s * (float)p.sum16, p.s * (float)p.sum32);
            };
#pragma unroll
            for (int j = 0; j < NBF; j++) {
                const int i = t + j * T;
                if (i < n4) put(i, v[j], g[j]);
            }
            for (int i = t + NBF * T; i < n4; i += T) put(i, x4[i], P.stage == kStageRms ? g4[i] : make_float4(0.f, 0.f, 0.f, 0.f));
        }
        __syncthreads();
    }
};

// All rows of problem P that fall to workgroup `wg` of the `n_wg` workgroups sharing it.  R rows per wave step
// (DUAL: R / 2 gate rows and their up rows, combined into up * silu(gate)).
template <int TYPE, int R, bool DUAL, bool EXACT>
__device__ __forceinline__ void lean_problem_t(const GemvProb &P, int wg, int n_wg, int m, uint32_t *lds, float *red) {
    constexpr int RG = DUAL ? R / 2 : R;                       // output rows per row group
    const int lane = (int)(threadIdx.x & 63);
    const int waves = (int)(blockDim.x >> 6);
    const int U = units_of(TYPE, P.K), n_iter = (U + 63) >> 6;
    const int N = P.N;
    const int n_groups = (N + RG - 1) / RG;
    const int gw = wg * waves + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int n_gw = n_wg * waves;
    const int my_groups = gw < n_groups ? (n_groups - gw + n_gw - 1) / n_gw : 0;
    const int steps = my_groups * n_iter;
    const uint32_t row_bytes = (uint32_t)P.row_bytes, nbytes = (uint32_t)N * row_bytes;
    const uint8_t *const w1 = P.w, *const w2 = DUAL ? P.w2 : P.w;
    // a residual is taken only in place (res == y; the launcher sends other cases to the general path): the row end is then
    // one returnless floating-point add to memory, with no load to wait for and no register held for it
    const bool add_to_y = !DUAL && P.res != nullptr;
    float *y = P.y + (size_t)m * N;

    LeanLane<TYPE> L;
    L.init(lane);

    // position of a step: row group g, pass p
    struct Pos { int g, p; };
    auto next = [&](Pos q) { return q.p + 1 == n_iter ? Pos{ q.g + n_gw, 0 } : Pos{ q.g, q.p + 1 }; };
    // EXACT: the row is a whole number of passes, every lane has a unit in every pass, and the window the loads go
    // through (weight_window) is the pass.  Otherwise the window is the row, the pass is part of the lane's offset, and the
    // lanes past the end of the row in its last pass reread the unit 64 before theirs (same u & 3, so the lane constants
    // hold; U >= 64 whenever a row has more than one pass); their products are masked.  Offsets are unsigned: nothing here
    // may go below the start of the row -- and if it did, the window's range check would turn the load into zeros.
    auto request = [&](WRegs<TYPE> *w, Pos s) {
        uint32_t so = 0, vo = 0;
        if (EXACT) so = (uint32_t)s.p * LeanLane<TYPE>::kPassBytes;
        else vo = (uint32_t)(s.p - ((n_iter > 1 && lane + 64 * s.p >= U) ? 1 : 0)) * LeanLane<TYPE>::kPassBytes;
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = s.g * RG + (DUAL ? (r >> 1) : r);
            row = min(row, N - 1);                                         // ragged tail: reread the last row, the store is skipped
            L.load(w[r], weight_window((DUAL && (r & 1)) ? w2 : w1, nbytes, (uint32_t)row * row_bytes + so,
                                       EXACT ? LeanLane<TYPE>::kPassBytes : row_bytes), vo);
        }
    };

    WRegs<TYPE> a[R], b[R];
    Pos pa{ gw, 0 }, pb = next(pa);
    if (!EXACT && U < 64 && lane >= U) L.init(0);       // rows shorter than one pass: the spare lanes reread unit 0 (masked)
    // x first, then two steps of weights, which stay in flight while x is being staged.  Both requests go out whatever the
    // number of steps (a wave with fewer rereads a row group of its own: a wait placed after a conditional request would
    // have to assume that nothing younger than x is outstanding, and so wait for everything)
    LeanStage S;
#ifndef RT_LEAN_NO_STAGE
    S.issue(P, m);
#endif
    request(a, steps > 0 ? pa : Pos{ gw % n_groups, 0 });
    request(b, steps > 1 ? pb : (steps > 0 ? pa : Pos{ gw % n_groups, 0 }));
#ifndef RT_LEAN_NO_STAGE
    S.finish<TYPE>(P, m, lds, red);
#endif
    lean_settle_loads();
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;

    constexpr bool kPasswise = !DUAL && R == 1;
    float row_sum = 0.f;
    auto consume = [&](const WRegs<TYPE> *w, Pos s) {
        const int u = lane + 64 * s.p;
        XRegs<TYPE> x;
        if (EXACT) {
            load_x(x, lds, u, U, P.K);
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] += RT_LEAN_DOT(L, w[r], x);
        } else {
            const float live = u < U ? 1.f : 0.f;
            load_x(x, lds, min(u, U - 1), U, P.K);
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] = __builtin_fmaf(live, RT_LEAN_DOT(L, w[r], x), acc[r]);
        }
        if (kPasswise) {
            // One row per step: a row's result is the sum, in pass order, of its passes' wave sums -- the same value, bit
            // for bit, that the split form builds through LDS, so a launch's shape never changes a result.
            row_sum += wave_sum_dpp(acc[0]);
            acc[0] = 0.f;
            if (s.p != n_iter - 1) return;
            acc[0] = row_sum;
            row_sum = 0.f;
        } else {
            if (s.p != n_iter - 1) return;
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] = wave_sum_dpp(acc[r]);
        }
        if (DUAL) {
#pragma unroll
            for (int r = 0; r < RG; r++) {
                const int row = s.g * RG + r;
                if (lane == r && row < N) {
                    const float gate = acc[2 * r], up = acc[2 * r + 1];
                    y[row] = up * (gate * (1.0f / (1.0f + expf(-gate))));
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int row = s.g * RG + r;
                if (lane == r && row < N) {
                    if (add_to_y) unsafeAtomicAdd(&y[row], acc[r]);
                    else y[row] = acc[r];
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0.f;
    };

    // a holds step s, b step s + 1 (requested).  In the steady state every consume is followed by the request that refills
    // its registers, unconditionally: a request inside an `if` would make the compiler wait, at the join, for the
    // loads of the path that has fewer of them outstanding -- that is, for the prefetch it has just issued.  The last one
    // to three steps are written out per case for the same reason.
    int s = 0;
    while (s + 3 < steps) {
        consume(a, pa);
        pa = next(pb);
        request(a, pa);
        consume(b, pb);
        pb = next(pa);
        request(b, pb);
        s += 2;
    }
    const int left = steps - s;
    if (left == 3) {
        consume(a, pa);
        pa = next(pb);
        request(a, pa);
        consume(b, pb);
        consume(a, pa);
    } else if (left > 0) {
        consume(a, pa);
        if (left == 2) consume(b, pb);
    }
}

// Rows of more than one pass with the planner's ksplit: the unit of work is one pass of one row.  The workgroup owns the
// rows wg, wg + n_wg, ...; their passes, in row order, are dealt out round-robin to its waves (so neighbouring waves read
// neighbouring pieces of one row at the same time); every pass is reduced over its wave on its own and left in LDS behind
// x; at the end the workgroup adds the passes of each row in pass order and stores.  A wave's work is then a multiple of
// a third of a long row instead of whole rows -- a launch ends with its slowest wave, and a wave streams a 9 KB row in
// about 6 us -- and a row's result does not depend on how the launch was cut: each (row, pass) sum is the same 64 lanes.
template <int TYPE, bool EXACT>
__device__ __forceinline__ void lean_problem_split(const GemvProb &P, int wg, int n_wg, int m, uint32_t *lds, float *red) {
    const int lane = (int)(threadIdx.x & 63);
    const int waves = (int)(blockDim.x >> 6);
    const int U = units_of(TYPE, P.K), n_iter = (U + 63) >> 6;
    const int N = P.N;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int rows_wg = wg < N ? (N - wg + n_wg - 1) / n_wg : 0;
    const int items = rows_wg * n_iter;
    const int steps = w < items ? (items - w + waves - 1) / waves : 0;
    const uint32_t row_bytes = (uint32_t)P.row_bytes, nbytes = (uint32_t)N * row_bytes;
    const bool add_to_y = P.res != nullptr;
    float *y = P.y + (size_t)m * N;
    float *part = reinterpret_cast<float *>(lds) + ((gemv_lds_bytes(TYPE, (size_t)P.K) + 15) >> 4) * 4;      // [rows_wg][n_iter]

    LeanLane<TYPE> L;
    L.init(lane);

    // item = (j: which of the workgroup's rows, p: pass); a wave moves on by `waves` items
    struct Pos { int j, p; };
    const int dj = waves / n_iter, dp = waves % n_iter;
    auto next = [&](Pos q) {
        Pos r{ q.j + dj, q.p + dp };
        if (r.p >= n_iter) { r.p -= n_iter; r.j++; }
        return r;
    };
    auto request = [&](WRegs<TYPE> &wr, Pos s) {
        uint32_t so = 0, vo = 0;
        if (EXACT) so = (uint32_t)s.p * LeanLane<TYPE>::kPassBytes;
        else vo = (uint32_t)(s.p - ((lane + 64 * s.p >= U) ? 1 : 0)) * LeanLane<TYPE>::kPassBytes;      // n_iter > 1 here: U >= 64
        const int row = min(wg + n_wg * s.j, N - 1);
        L.load(wr, weight_window(P.w, nbytes, (uint32_t)row * row_bytes + so, EXACT ? LeanLane<TYPE>::kPassBytes : row_bytes), vo);
    };

    WRegs<TYPE> a, b;
    Pos pa{ w / n_iter, w % n_iter }, pb = next(pa);
    // x first, then two steps of weights (both whatever the number of steps: a wave with fewer rereads the first pass of the
    // workgroup's first row, see lean_problem_t)
    LeanStage S;
#ifndef RT_LEAN_NO_STAGE
    S.issue(P, m);
#endif
    request(a, steps > 0 ? pa : Pos{ 0, 0 });
    request(b, steps > 1 ? pb : (steps > 0 ? pa : Pos{ 0, 0 }));
#ifndef RT_LEAN_NO_STAGE
    S.finish<TYPE>(P, m, lds, red);
#endif
    lean_settle_loads();

    auto consume = [&](const WRegs<TYPE> &wr, Pos s) {
        const int u = lane + 64 * s.p;
        XRegs<TYPE> x;
        float d;
        if (EXACT) {
            load_x(x, lds, u, U, P.K);
            d = RT_LEAN_DOT(L, wr, x);
        } else {
            const float live = u < U ? 1.f : 0.f;
            load_x(x, lds, min(u, U - 1), U, P.K);
            d = live * RT_LEAN_DOT(L, wr, x);
        }
        d = wave_sum_dpp(d);
        if (lane == 0) part[s.j * n_iter + s.p] = d;
    };

    int s = 0;
    while (s + 3 < steps) {
        consume(a, pa);
        pa = next(pb);
        request(a, pa);
        consume(b, pb);
        pb = next(pa);
        request(b, pb);
        s += 2;
    }
    const int left = steps - s;
    if (left == 3) {
        consume(a, pa);
        pa = next(pb);
        request(a, pa);
        consume(b, pb);
        consume(a, pa);
    } else if (left > 0) {
        consume(a, pa);
        if (left == 2) consume(b, pb);
    }
    __syncthreads();
    for (int j = (int)threadIdx.x; j < rows_wg; j += (int)blockDim.x) {
        float sum = part[j * n_iter];
        for (int p = 1; p < n_iter; p++) sum += part[j * n_iter + p];
        const int row = wg + n_wg * j;
        if (add_to_y) unsafeAtomicAdd(&y[row], sum);
        else y[row] = sum;
    }
}

template <int TYPE, int R, bool DUAL>
__device__ __forceinline__ void lean_problem(const GemvProb &P, int wg, int n_wg, int m, uint32_t *lds, float *red) {
    const bool exact = (units_of(TYPE, P.K) & 63) == 0;
    if (!DUAL && R == 1 && P.ksplit) {
        if (exact) lean_problem_split<TYPE, true>(P, wg, n_wg, m, lds, red);
        else lean_problem_split<TYPE, false>(P, wg, n_wg, m, lds, red);
    } else if (exact) lean_problem_t<TYPE, R, DUAL, true>(P, wg, n_wg, m, lds, red);
    else lean_problem_t<TYPE, R, DUAL, false>(P, wg, n_wg, m, lds, red);
}

__device__ __forceinline__ bool lean_type(int type) {
    return type == RT_GGML_Q4_K || type == RT_GGML_Q6_K || type == RT_GGML_Q8_0 || type == RT_GGML_Q4_0;
}

// PAIR = false leaves the gate / up pair form out of the kernel (the launcher picks it when no problem of the launch has
// the SwiGLU epilogue): the pair form holds two rows of weights twice over and sets the register budget of a kernel that
// contains it, whether a launch reaches it or not.
template <int R, bool PAIR>
__device__ __forceinline__ void lean_dispatch(const GemvProb &P, int wg, int n_wg, int m, uint32_t *lds, float *red) {
    if (PAIR && P.epi == kEpiSwiglu) {
        switch (P.type) {
        case RT_GGML_Q4_K: lean_problem<RT_GGML_Q4_K, 2, true>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q6_K: lean_problem<RT_GGML_Q6_K, 2, true>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q8_0: lean_problem<RT_GGML_Q8_0, 2, true>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q4_0: lean_problem<RT_GGML_Q4_0, 2, true>(P, wg, n_wg, m, lds, red); break;
        }
    } else {
        switch (P.type) {
        case RT_GGML_Q4_K: lean_problem<RT_GGML_Q4_K, R, false>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q6_K: lean_problem<RT_GGML_Q6_K, R, false>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q8_0: lean_problem<RT_GGML_Q8_0, R, false>(P, wg, n_wg, m, lds, red); break;
        case RT_GGML_Q4_0: lean_problem<RT_GGML_Q4_0, R, false>(P, wg, n_wg, m, lds, red); break;
        }
    }
}

}  // namespace rt
