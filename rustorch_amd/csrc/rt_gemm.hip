// Prefill contraction Y[M,N] = X[M,K] . dequant(W)^T on the matrix cores (gfx950 MFMA, fp16 in / f32 out).
//
// Roofline: for M >= 64 this is a dense contraction bounded by MFMA throughput, not by HBM.  The weights
// stay in their raw GGUF blocks; a wave reads the bytes of its 32-row fragment straight from global memory
// (16 bytes per lane and k-tile for Q4_K), expands them to fp16 in registers with two packed operations
// per pair of elements, and feeds v_mfma_f32_32x32x16_f16.  Dequantized weights never touch LDS or HBM.
//
// Operands
//   A = 32 weight rows x 16 k   (expanded in registers)
//   B = 16 k x 32 tokens        (X, fp16, staged through LDS in 64-k tiles, double buffered)
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
// Work split: a workgroup (4 waves) owns a BM x BN tile of Y; when the grid would leave CUs idle the k
// range is split across workgroups and partial tiles are added into Y with f32 atomics.
#include "rt_device.h"

#include <cstring>

namespace rt {

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x4 ldg16(const uint8_t *p) { u32x4 v; __builtin_memcpy(&v, p, 16); return v; }
__device__ __forceinline__ u32x4 ldg16a(const uint8_t *p) { return *reinterpret_cast<const u32x4 *>(p); }
__device__ __forceinline__ u32x2 ldg8(const uint8_t *p) { u32x2 v; __builtin_memcpy(&v, p, 8); return v; }

constexpr int kBK = 64;          // k per tile

// ---- pre-pass: X f32 [M,K] -> fp16, row-scaled, k-permuted; inv_scale[m] undoes the row scale
__global__ __launch_bounds__(256) void xprep_kernel(const float *X, size_t K, _Float16 *Xp, float *inv_scale) {
    __shared__ float red[4];
    const size_t m = blockIdx.x;
    const float *x = X + m * K;
    float amax = 0.f;
    for (size_t i = threadIdx.x; i < K / 4; i += blockDim.x) {
        float4 v = reinterpret_cast<const float4 *>(x)[i];
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
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
    const int perm[8] = { 0, 2, 1, 3, 4, 6, 5, 7 };
    for (size_t g = threadIdx.x; g < K / 8; g += blockDim.x) {
        size_t kt = g >> 3;
        int sh = (int)(g & 7), s = sh >> 1, h = sh & 1;
        size_t src = 64 * kt + 32 * (size_t)(s >> 1) + 16 * (size_t)h + 8 * (size_t)(s & 1);
        float4 a = reinterpret_cast<const float4 *>(x + src)[0], b = reinterpret_cast<const float4 *>(x + src)[1];
        const float v[8] = { a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w };
        half8v o;
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = (_Float16)(v[perm[i]] * scale);
        *reinterpret_cast<half8v *>(Xp + m * K + 8 * g) = o;
    }
}

// ---- raw weight bytes of one lane for one k-tile
template <int TYPE> struct WTile;
template <> struct WTile<RT_GGML_Q4_K> { u32x4 hdr, qs; };
template <> struct WTile<RT_GGML_Q6_K> { u32x4 A, B, H; u32x2 sc; uint32_t d; };

// lane half h takes l in [16h, 16h+16) of the tile's group (Q4_K) / half super-block (Q6_K)
__device__ __forceinline__ void load_tile(WTile<RT_GGML_Q4_K> &w, const uint8_t *row, int kt, int h) {
    const uint8_t *blk = row + (size_t)(kt >> 2) * 144;
    w.hdr = ldg16a(blk);
    w.qs = ldg16a(blk + 16 + 32 * (kt & 3) + 16 * h);
}
__device__ __forceinline__ void load_tile(WTile<RT_GGML_Q6_K> &w, const uint8_t *row, int kt, int h) {
    const uint8_t *blk = row + (size_t)(kt >> 2) * 210;
    const int hf = (kt >> 1) & 1;
    w.A = ldg16(blk + 64 * hf + 16 * h);
    w.B = ldg16(blk + 64 * hf + 32 + 16 * h);
    w.H = ldg16(blk + 128 + 32 * hf + 16 * h);
    w.sc = ldg8(blk + 192 + 8 * hf);
    w.d = ld2u(blk + 208);
}

__device__ __forceinline__ half2v splat(float f) {
    _Float16 v = (_Float16)f;
    return half2v{ v, v };
}
__device__ __forceinline__ half2v as_h2(uint32_t u) { return __builtin_bit_cast(half2v, u); }

// Per-tile constants of one weight fragment: everything of the expansion that does not depend on the MFMA step.
template <int TYPE> struct TileK;
template <> struct TileK<RT_GGML_Q4_K> { half2v a[2], c[2]; };   // [low nibbles, high nibbles]: 16*d*sc and -dmin*m
template <> struct TileK<RT_GGML_Q6_K> { half2v a[2]; int sh_l, sh_h[2]; };   // 64*d*sc of the tile's two runs

__device__ __forceinline__ void prep(TileK<RT_GGML_Q4_K> &k, const WTile<RT_GGML_Q4_K> &w, int kt, int) {
    const int g = kt & 3;
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
    float d = 16.f * h2f(w.hdr.x & 0xFFFF), dmin = -h2f(w.hdr.x >> 16);
    // (1 + q/16) - 1 is exact in fp16, so the only roundings are those of the scale, of the min and of the result
    k.a[0] = splat(d * (float)(scw & 0xFF));
    k.a[1] = splat(d * (float)((scw >> 8) & 0xFF));
    k.c[0] = splat(dmin * (float)(mw & 0xFF));
    k.c[1] = splat(dmin * (float)((mw >> 8) & 0xFF));
}

// Packed pair u (k slots 2u, 2u+1 of this lane's row) of the fp16 A operand for MFMA step s of the tile.
// A step's operand is four such pairs; they are produced one at a time so that each can be issued behind
// one matrix instruction.
__device__ __forceinline__ half2v expand_unit(const WTile<RT_GGML_Q4_K> &w, const TileK<RT_GGML_Q4_K> &k, int s, int u) {
    const int hi = s >> 1;
    const uint32_t q = (s & 1) ? ((u & 2) ? w.qs.w : w.qs.z) : ((u & 2) ? w.qs.y : w.qs.x);
    const uint32_t M = 0x03C003C0u, G = 0x3C003C00u;
    // low nibbles of bytes (0,2) / (1,3) sit at bits 3:0 / 11:8 (and +16); high nibbles 4 bits further up
    const int sh = (u & 1) * 8 + hi * 4;    // nibble position to bring to bit 6
    const uint32_t p = (sh <= 6 ? (q << (6 - sh)) : (q >> (sh - 6)));
    return (as_h2((p & M) | G) - splat(1.f)) * k.a[hi] + k.c[hi];
}

__device__ __forceinline__ void prep(TileK<RT_GGML_Q6_K> &k, const WTile<RT_GGML_Q6_K> &w, int kt, int h) {
    // tile parity p: runs 0,1 (low nibbles) or 2,3 (high nibbles) of the half super-block; run r = 2p + s/2;
    // the 16 elements of a run this lane holds share scale sc[2r + h] of the half's 8 scales
    const int p = kt & 1;
    const float d = 64.f * h2f(w.d);
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int si = 2 * (2 * p + j) + h;
        uint32_t sw = si < 4 ? w.sc.x : w.sc.y;
        k.a[j] = splat(d * (float)(int)(int8_t)((sw >> (8 * (si & 3))) & 0xFF));
        k.sh_h[j] = 2 * (2 * p + j);
    }
    k.sh_l = 4 * p;
}

__device__ __forceinline__ half2v expand_unit(const WTile<RT_GGML_Q6_K> &w, const TileK<RT_GGML_Q6_K> &k, int s, int u) {
    const int j = s >> 1, t = s & 1;
    const u32x4 L = j ? w.B : w.A;    // run parity = j: even runs read ql[l], odd runs ql[l + 32]
    const uint32_t l = t ? ((u & 2) ? L.w : L.z) : ((u & 2) ? L.y : L.x);
    const uint32_t hq = t ? ((u & 2) ? w.H.w : w.H.z) : ((u & 2) ? w.H.y : w.H.x);
    // 6-bit values, one per byte
    const uint32_t v = ((l >> k.sh_l) & 0x0f0f0f0fu) | (((hq >> k.sh_h[j]) & 0x03030303u) << 4);
    // fp16 value 1 + v/64 is the bit pattern 0x3C00 | v << 4;  (1 + v/64) - 1.5 = (v - 32)/64 exactly,
    // so w = 64*dsc * ((1 + v/64) - 1.5) carries only the rounding of the scale and of the product
    const uint32_t M = 0x03F003F0u, G = 0x3C003C00u;
    const uint32_t p = (u & 1) ? (v >> 4) : (v << 4);
    return (as_h2((p & M) | G) - splat(1.5f)) * k.a[j];
}

template <int TYPE>
__device__ __forceinline__ half8v expand(const WTile<TYPE> &w, const TileK<TYPE> &k, int s) {
    half2v r0 = expand_unit(w, k, s, 0), r1 = expand_unit(w, k, s, 1), r2 = expand_unit(w, k, s, 2), r3 = expand_unit(w, k, s, 3);
    return half8v{ r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1] };
}

// s_waitcnt that only constrains the vector-memory counter (gfx9 encoding: vmcnt in bits 3:0 and 15:14;
// lgkmcnt = 15 and expcnt = 7 mean no constraint).
template <int N> __device__ __forceinline__ void wait_vmcnt_c() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// WM waves along m (4 / WM along n); a wave owns MF x NF fragments of 32 x 32.
//
// X tiles (BM rows x 64 k, fp16) go from global memory straight into a ring of NS LDS stages with 16-byte
// LDS-DMA loads, issued NS-1 tiles ahead; weight bytes go to registers two tiles ahead.  One barrier per k-tile.
// LDS stage: row m holds 8 chunks of 16 bytes, chunk c at position c ^ ((m >> 1) & 7), so that the 16 lanes
// that read the same chunk index of 16 consecutive rows fall on distinct banks.
// Grid: 1-D and XCD-aware.  Tiles are ordered by (m-tile, k-split) "slab" first, n-tile second; workgroup b
// runs on XCD b % 8 (round-robin dispatch), and XCD x is given a contiguous run of that order, so the
// workgroups that share an L2 share an X slab and the slab is read from HBM once.
template <int TYPE, int WM, int MF, int NF>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void qgemm_kernel(const uint8_t *W, size_t row_bytes, int N, int K, const _Float16 *Xp,
                                                    const float *inv_scale, int M, float *Y, const float *res,
                                                    int ktiles_per_split, int ksplit, int tiles_n, int n_tiles_total,
                                                    int per_xcd) {
    constexpr int WN = 4 / WM, BM = WM * MF * 32, BN = WN * NF * 32, XV = BM / 32, NS = 4;
    constexpr int WL = TYPE == RT_GGML_Q4_K ? 2 : 5;   // global loads per weight fragment and k-tile
    constexpr int kStageHalves = BM * kBK;   // halves per stage (no padding: swizzled)
    RT_DYN_LDS(_Float16, xs);                // [NS][BM][64]
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, nl = lane & 31, h = lane >> 5;
    const int wm = wave % WM, wn = wave / WM;
    // tile of this workgroup
    const int t = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || t >= n_tiles_total) return;
    const int slab = t / tiles_n, nt = t - slab * tiles_n;
    const int mt = slab / ksplit, kz = slab - mt * ksplit;
    const int n0 = nt * BN, m0 = mt * BM;
    const int ktiles = K / kBK;
    const int kt0 = kz * ktiles_per_split, kt1 = min(ktiles, kt0 + ktiles_per_split);
    if (kt0 >= kt1) return;

    const uint8_t *rp[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) rp[f] = W + (size_t)min(n0 + (wn * NF + f) * 32 + nl, N - 1) * row_bytes;

    // LDS-DMA: instruction i of this wave fills LDS rows (wave*XV + i)*8 .. +8 of a stage; lane L lands at
    // row + L/8, position L%8, which must hold chunk (L%8) ^ ((row >> 1) & 7) of that X row.
    const _Float16 *xsrc[XV];
#pragma unroll
    for (int i = 0; i < XV; i++) {
        int row = (wave * XV + i) * 8 + (lane >> 3);
        int c = (lane & 7) ^ ((row >> 1) & 7);
        xsrc[i] = Xp + (size_t)min(m0 + row, M - 1) * K + 8 * c;
    }
    auto issue_x = [&](int kt) {
        const int st = (kt - kt0) % NS;
#pragma unroll
        for (int i = 0; i < XV; i++) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xsrc[i] + (size_t)kt * kBK),
                                             (__attribute__((address_space(3))) void *)(xs + (size_t)st * kStageHalves + (size_t)(wave * XV + i) * 8 * kBK),
                                             16, 0, 0);
        }
    };

    float16v acc[MF][NF];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][f][r] = 0.f;

    // B fragment address pieces: lane (token nl of fragment i, half h) reads chunk 2s+h of row (wm*MF+i)*32 + nl
    int brow[MF], bsw[MF];
#pragma unroll
    for (int i = 0; i < MF; i++) {
        brow[i] = (wm * MF + i) * 32 + nl;
        bsw[i] = (brow[i] >> 1) & 7;
    }

    auto compute = [&](int kt, const WTile<TYPE> *wc) {
        const _Float16 *stage = xs + (size_t)((kt - kt0) % NS) * kStageHalves;
        TileK<TYPE> tk[NF];
#pragma unroll
        for (int f = 0; f < NF; f++) prep(tk[f], wc[f], kt, h);
        half8v a[NF], b[MF];
#pragma unroll
        for (int f = 0; f < NF; f++) a[f] = expand(wc[f], tk[f], 0);
#pragma unroll
        for (int i = 0; i < MF; i++)
            b[i] = *reinterpret_cast<const half8v *>(stage + (size_t)brow[i] * kBK + 8 * (h ^ bsw[i]));
#pragma unroll
        for (int s = 0; s < 4; s++) {
            // Operands of the next step are fetched (LDS) at the top of this step and expanded (VALU) one packed
            // pair behind each matrix instruction of this step; the order below is pinned for the scheduler.
            constexpr int UPM = (4 + MF - 1) / MF;    // expansion pairs issued behind each matrix instruction
            half8v bn[MF];
            half2v an[NF][4];
            if (s < 3) {
#pragma unroll
                for (int i = 0; i < MF; i++)
                    bn[i] = *reinterpret_cast<const half8v *>(stage + (size_t)brow[i] * kBK + 8 * ((2 * (s + 1) + h) ^ bsw[i]));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < MF * NF; j++) {
                const int i = j / NF, f = j % NF;
                acc[i][f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[f], b[i], acc[i][f], 0, 0, 0);
                if (s < 3) {
#pragma unroll
                    for (int q = j * UPM; q < (j + 1) * UPM && q < 4 * NF; q++)
                        an[q / 4][q % 4] = expand_unit(wc[q / 4], tk[q / 4], s + 1, q % 4);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (s < 3) {
#pragma unroll
                for (int f = 0; f < NF; f++)
                    a[f] = half8v{ an[f][0][0], an[f][0][1], an[f][1][0], an[f][1][1], an[f][2][0], an[f][2][1], an[f][3][0], an[f][3][1] };
#pragma unroll
                for (int i = 0; i < MF; i++) b[i] = bn[i];
            }
        }
    };

    WTile<TYPE> w0[NF], w1[NF], w2[NF];
    // prologue: X tiles kt0 .. kt0+NS-2 and weight tiles kt0, kt0+1 in flight
#pragma unroll
    for (int d = 0; d < NS - 1; d++)
        if (kt0 + d < kt1) issue_x(kt0 + d);
#pragma unroll
    for (int f = 0; f < NF; f++) load_tile(w0[f], rp[f], kt0, h);
    if (kt0 + 1 < kt1) {
#pragma unroll
        for (int f = 0; f < NF; f++) load_tile(w1[f], rp[f], kt0 + 1, h);
    }

    // one iteration: tile kt is computed from `wc`; tile kt+2's weights are requested into `wl`, tile kt+NS-1's X into LDS
#define RT_GEMM_STEP(KT, wc, wl)                                                                   \
    if ((KT) < kt1) {                                                                              \
        /* loads complete in order: once only the previous iteration's requests (X tile KT+2,    */  \
        /* weights KT+1) may be outstanding, X tile KT and weights KT have landed                  */  \
        if ((KT) == kt0) wait_vmcnt_c<0>();                                                        \
        else if ((KT) + 2 < kt1) wait_vmcnt_c<XV + WL * NF>();                                     \
        else if ((KT) + 1 < kt1) wait_vmcnt_c<WL * NF>();                                          \
        else wait_vmcnt_c<0>();                                                                    \
        __syncthreads();                                                                           \
        if ((KT) + NS - 1 < kt1) issue_x((KT) + NS - 1);                                           \
        if ((KT) + 2 < kt1) {                                                                      \
            _Pragma("unroll") for (int f = 0; f < NF; f++) load_tile(wl[f], rp[f], (KT) + 2, h);   \
        }                                                                                          \
        compute((KT), wc);                                                                         \
    }
    for (int kt = kt0; kt < kt1; kt += 3) {
        RT_GEMM_STEP(kt, w0, w2)
        RT_GEMM_STEP(kt + 1, w1, w0)
        RT_GEMM_STEP(kt + 2, w2, w1)
    }
#undef RT_GEMM_STEP

    // D[i][j]: j (token) = lane % 32; i (weight row) = 8*(r/4) + 4*(lane/32) + r%4
    const int use_atomic = ksplit > 1;
#pragma unroll
    for (int i = 0; i < MF; i++) {
        const int m = m0 + (wm * MF + i) * 32 + nl;
        if (m >= M) continue;
        const float inv = inv_scale[m];
#pragma unroll
        for (int f = 0; f < NF; f++) {
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                const int n = n0 + (wn * NF + f) * 32 + 8 * g4 + 4 * h;
                if (n >= N) continue;   // N is a multiple of 4: a group of 4 rows is inside or outside as a whole
                float4 v = make_float4(acc[i][f][4 * g4] * inv, acc[i][f][4 * g4 + 1] * inv, acc[i][f][4 * g4 + 2] * inv,
                                       acc[i][f][4 * g4 + 3] * inv);
                float *yp = Y + (size_t)m * N + n;
                if (res && kz == 0) {
                    float4 rv = *reinterpret_cast<const float4 *>(res + (size_t)m * N + n);
                    v.x += rv.x; v.y += rv.y; v.z += rv.z; v.w += rv.w;
                }
                if (use_atomic) {
                    atomicAdd(yp, v.x); atomicAdd(yp + 1, v.y); atomicAdd(yp + 2, v.z); atomicAdd(yp + 3, v.w);
                } else {
                    *reinterpret_cast<float4 *>(yp) = v;
                }
            }
        }
    }
}

template <int TYPE, int WM, int MF, int NF>
hipError_t launch_cfg(hipStream_t s, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const _Float16 *Xp,
                      const float *inv_scale, size_t M, float *Y, const float *res) {
    constexpr int WN = 4 / WM, BM = WM * MF * 32, BN = WN * NF * 32, NS = 4;
    const size_t lds = (size_t)NS * BM * kBK * sizeof(_Float16);
    auto kern = qgemm_kernel<TYPE, WM, MF, NF>;
    static bool attr_set = false;
    if (!attr_set && lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN), ktiles = (int)(K / kBK);
    // fill the 256 CUs: split k until there are enough workgroups, keeping at least 8 tiles per split
    int ksplit = 1;
    while (tiles_m * tiles_n * ksplit < 256 && ktiles / (ksplit * 2) >= 8) ksplit *= 2;
    const int per = (ktiles + ksplit - 1) / ksplit;
    ksplit = (ktiles + per - 1) / per;
    if (ksplit > 1) {
        // partial tiles are added into Y: start from zero (the residual is added by split 0)
        hipError_t e = hipMemsetAsync(Y, 0, M * N * sizeof(float), s);
        if (e != hipSuccess) return e;
    }
    const int total = tiles_m * ksplit * tiles_n;
    const int per_xcd = (total + 7) / 8;
    kern<<<dim3((unsigned)(8 * per_xcd)), 256, lds, s>>>(w, row_bytes, (int)N, (int)K, Xp, inv_scale, (int)M, Y, res, per, ksplit,
                                                        tiles_n, total, per_xcd);
    return hipGetLastError();
}

template <int TYPE>
hipError_t launch_type(hipStream_t s, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const _Float16 *Xp,
                       const float *inv_scale, size_t M, float *Y, const float *res) {
    if (M >= 192) return launch_cfg<TYPE, 2, 4, 2>(s, w, N, K, row_bytes, Xp, inv_scale, M, Y, res);   // 256 x 128
    if (M >= 96) return launch_cfg<TYPE, 1, 4, 2>(s, w, N, K, row_bytes, Xp, inv_scale, M, Y, res);    // 128 x 256
    return launch_cfg<TYPE, 1, 2, 2>(s, w, N, K, row_bytes, Xp, inv_scale, M, Y, res);                 //  64 x 256
}

bool mfma_path(int type, size_t N, size_t K, size_t M) {
    return (type == RT_GGML_Q4_K || type == RT_GGML_Q6_K) && M >= 16 && K % 256 == 0 && N % 4 == 0;
}

}  // namespace

size_t qgemm_scratch_bytes(size_t M, size_t K) {
    size_t xp = (M * K * sizeof(_Float16) + 255) & ~(size_t)255;
    return xp + M * sizeof(float);
}

// res (optional, may alias Y only when it is not Y's own storage being zeroed: see below) is added to the result.
hipError_t launch_qgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes,
                        const float *X, size_t M, float *Y, const float *res, void *scratch, size_t scratch_bytes) {
    if (mfma_path(type, N, K, M) && res != Y) {
        if (scratch_bytes < qgemm_scratch_bytes(M, K)) return hipErrorInvalidValue;
        _Float16 *Xp = reinterpret_cast<_Float16 *>(scratch);
        float *inv_scale = reinterpret_cast<float *>(reinterpret_cast<char *>(scratch) + ((M * K * sizeof(_Float16) + 255) & ~(size_t)255));
        xprep_kernel<<<dim3((unsigned)M), 256, 0, s>>>(X, K, Xp, inv_scale);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        if (type == RT_GGML_Q4_K) return launch_type<RT_GGML_Q4_K>(s, w, N, K, row_bytes, Xp, inv_scale, M, Y, res);
        return launch_type<RT_GGML_Q6_K>(s, w, N, K, row_bytes, Xp, inv_scale, M, Y, res);
    }
    // Row-by-row form (small M, Q8_0 / Q4_0, in-place residual): the GEMV kernel, one grid slice per row of X.
    GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = 1;
    a.p[0].w = w; a.p[0].x = X; a.p[0].stage = kStageF32; a.p[0].y = Y; a.p[0].res = res; a.p[0].row_bytes = row_bytes;
    a.p[0].type = type; a.p[0].N = (int)N; a.p[0].K = (int)K;
    return launch_qgemv(s, a, (int)M);
}

}  // namespace rt
