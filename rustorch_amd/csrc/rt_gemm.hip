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

constexpr int kBK = 64;          // k per tile
constexpr int kMaxSplit = 8;     // most k splits of one launch

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

// ---- raw weight bytes of one lane (weight row nl, k half h) for one super-block of 256 k
template <int TYPE> struct WSb;
template <> struct WSb<RT_GGML_Q4_K> { u32x4 hdr; u32x4 qs[4]; };                 // d|dmin, 12 scale bytes; 16 bytes per 64-k tile
template <> struct WSb<RT_GGML_Q6_K> { u32x4 A[2], B[2], H[2], sc; uint32_t d; };  // per 128-k half: ql[l], ql[l+32], qh[l]
template <int TYPE> struct WLoads;
template <> struct WLoads<RT_GGML_Q4_K> { static constexpr int n = 5; };
template <> struct WLoads<RT_GGML_Q6_K> { static constexpr int n = 8; };

__device__ __forceinline__ void load_sb(WSb<RT_GGML_Q4_K> &w, const uint8_t *row, int sb, int h) {
    const uint8_t *blk = row + (size_t)sb * 144;
    w.hdr = ldg16a(blk);
#pragma unroll
    for (int t = 0; t < 4; t++) w.qs[t] = ldg16a(blk + 16 + 32 * t + 16 * h);
}
__device__ __forceinline__ void load_sb(WSb<RT_GGML_Q6_K> &w, const uint8_t *row, int sb, int h) {
    const uint8_t *blk = row + (size_t)sb * 210;
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
        w.A[hf] = ldg16(blk + 64 * hf + 16 * h);
        w.B[hf] = ldg16(blk + 64 * hf + 32 + 16 * h);
        w.H[hf] = ldg16(blk + 128 + 32 * hf + 16 * h);
    }
    w.sc = ldg16(blk + 192);
    w.d = ld2u(blk + 208);
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

// Per-super-block constants of one lane's weight row: everything of the expansion that does not depend on the
// MFMA step.  One register holds the pair the two halves of a tile need; the fma picks the half.
template <int TYPE> struct SbK;
template <> struct SbK<RT_GGML_Q4_K> { half2v a[4], c[4]; };   // tile t: (16*d*sc, -dmin*m) of sub-blocks 2t (low nibbles) and 2t+1
template <> struct SbK<RT_GGML_Q6_K> { half2v a[4]; };         // tile t: 64*d*sc of the tile's two 16-element runs of this lane

// bytes 0 and 1 of v as two exact fp16 numbers: 0x6400 | b is 1024 + b
__device__ __forceinline__ half2v byte_pair(uint32_t v) {
    return as_h2((v & 0xFFu) | ((v & 0xFF00u) << 8) | 0x64006400u) - splat(1024.f);
}

__device__ __forceinline__ void prep(SbK<RT_GGML_Q4_K> &k, const WSb<RT_GGML_Q4_K> &w, int) {
    const uint32_t y = w.hdr.y, z = w.hdr.z, x = w.hdr.w;
    const uint32_t sc_lo = y & 0x3f3f3f3fu, m_lo = z & 0x3f3f3f3fu;
    const uint32_t sc_hi = (x & 0x0f0f0f0fu) | ((y >> 2) & 0x30303030u);
    const uint32_t m_hi = ((x >> 4) & 0x0f0f0f0fu) | ((z >> 2) & 0x30303030u);
    // fp16 products of an 11-bit and a 6-bit number round once: the same value as the f32 product rounded to fp16
    const half2v d16 = splat_h(h_bits(w.hdr.x & 0xFFFF)) * splat(16.f);
    const half2v nmin = -splat_h(h_bits(w.hdr.x >> 16));
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const uint32_t scw = t < 2 ? sc_lo : sc_hi, mw = t < 2 ? m_lo : m_hi;
        k.a[t] = byte_pair(scw >> (16 * (t & 1))) * d16;
        k.c[t] = byte_pair(mw >> (16 * (t & 1))) * nmin;
    }
}

// Packed pair u (k slots 2u, 2u+1 of this lane's row) of the fp16 A operand for MFMA step s of tile t.
// A step's operand is four such pairs; they are produced one at a time so that each can be issued behind
// one matrix instruction.
__device__ __forceinline__ half2v expand_unit(const WSb<RT_GGML_Q4_K> &w, const SbK<RT_GGML_Q4_K> &k, int t, int s, int u, uint32_t G) {
    const int hi = s >> 1;
    const u32x4 qs = w.qs[t];
    const uint32_t q = (s & 1) ? ((u & 2) ? qs.w : qs.z) : ((u & 2) ? qs.y : qs.x);
    // low nibbles of bytes (0,2) / (1,3) sit at bits 3:0 / 11:8 (and +16); high nibbles 4 bits further up
    const int sh = (u & 1) * 8 + hi * 4;    // nibble position to bring to bit 6
    const uint32_t p = (sh <= 6 ? (q << (6 - sh)) : (q >> (sh - 6)));
    const half2v a = splat_h(k.a[t][hi]), c = splat_h(k.c[t][hi]);
    return (as_h2(and_or(p, 0x03C003C0u, G)) - splat(1.f)) * a + c;
}

__device__ __forceinline__ void prep(SbK<RT_GGML_Q6_K> &k, const WSb<RT_GGML_Q6_K> &w, int h) {
    // tile t = 2*hf + p: half hf of the super-block, runs 2p and 2p+1 of that half; of a run's 32 elements this
    // lane holds 16 with scale index 2*run + h among the half's 8 scales, i.e. bytes h and h+2 of word 2*hf + p
    const half2v d64 = splat_h(h_bits(w.d)) * splat(64.f);
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const uint32_t v = w.sc[t] >> (8 * h);
        // int8 b -> fp16: 0x6400 | (b ^ 0x80) is 1024 + b + 128
        k.a[t] = (as_h2((((v & 0xFFu) | (v & 0x00FF0000u)) ^ 0x00800080u) | 0x64006400u) - splat(1152.f)) * d64;
    }
}

__device__ __forceinline__ half2v expand_unit(const WSb<RT_GGML_Q6_K> &w, const SbK<RT_GGML_Q6_K> &k, int t, int s, int u, uint32_t G) {
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
    // fp16 value 1 + v/64 is the bit pattern 0x3C00 | v << 4;  (1 + v/64) - 1.5 = (v - 32)/64 exactly,
    // so w = 64*dsc * ((1 + v/64) - 1.5) carries only the rounding of the scale and of the product
    const uint32_t pp = (u & 1) ? (v >> 4) : (v << 4);
    return (as_h2(and_or(pp, 0x03F003F0u, G)) - splat(1.5f)) * splat_h(k.a[t][j]);
}

// s_waitcnt that only constrains the vector-memory counter (gfx9 encoding: vmcnt in bits 3:0 and 15:14;
// lgkmcnt = 15 and expcnt = 7 mean no constraint).
template <int N> __device__ __forceinline__ void wait_vmcnt_c() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// One super-block (256 k = 4 tiles x 4 MFMA steps) of a wave's 32 rows x 32*MF tokens.
//
// X tiles (BM rows x 64 k, fp16) go from global memory straight into a ring of 4 LDS stages with 16-byte
// LDS-DMA loads, issued 3 tiles ahead; since a split starts on a super-block boundary, tile t of every
// super-block lives in stage t.  One barrier per tile.  LDS stage: row m holds 8 chunks of 16 bytes, chunk c
// at position c ^ ((m >> 1) & 7), so that the 16 lanes that read the same chunk index of 16 consecutive
// rows fall on distinct banks.
//
// Vector-memory operations complete in order, so "at most n outstanding" pins which have landed.  Issue order
// per super-block: weights of the next super-block (WL loads), then one X tile (XI loads) after each barrier.
// Before tile t the operations younger than its own X tile are two more X tiles and, for t < 3, the weight
// prefetch.  LAST: no prefetch, and only tile 0 still has an X tile to request.
template <int TYPE, int MF, int XI, bool LAST, class IssueX>
__device__ __forceinline__ void superblock(float16v (&acc)[MF], const WSb<TYPE> &w, const _Float16 *xs, int stage_halves,
                                           const int (&brow)[MF], const int (&bsw)[MF], int h, uint32_t G, int kt, IssueX issue_x) {
    constexpr int WL = WLoads<TYPE>::n;
    constexpr int UPM = (4 + MF - 1) / MF;    // expansion pairs issued behind each matrix instruction
    SbK<TYPE> k;
    prep(k, w, h);
    half8v a;
    {
        half2v r0 = expand_unit(w, k, 0, 0, 0, G), r1 = expand_unit(w, k, 0, 0, 1, G), r2 = expand_unit(w, k, 0, 0, 2, G),
               r3 = expand_unit(w, k, 0, 0, 3, G);
        a = half8v{ r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1] };
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
        if (!LAST) {
            if (t < 3) wait_vmcnt_c<2 * XI + WL>(); else wait_vmcnt_c<2 * XI>();
        } else {
            if (t < 2) wait_vmcnt_c<2 * XI>(); else if (t == 2) wait_vmcnt_c<XI>(); else wait_vmcnt_c<0>();
        }
        __builtin_amdgcn_s_barrier();
        if (!LAST || t == 0) issue_x(kt + t + 3, (t + 3) & 3);
        const _Float16 *stage = xs + (size_t)t * stage_halves;
        half8v b[MF];
#pragma unroll
        for (int i = 0; i < MF; i++) b[i] = *reinterpret_cast<const half8v *>(stage + (size_t)brow[i] * kBK + 8 * (h ^ bsw[i]));
#pragma unroll
        for (int s = 0; s < 4; s++) {
            // Operands of the next step are fetched (LDS) at the top of this step and expanded (VALU) one packed
            // pair behind each matrix instruction of this step; the order below is pinned for the scheduler.
            const bool more_b = s < 3, more_a = s < 3 || t < 3;
            const int tn = s < 3 ? t : t + 1, sn = (s + 1) & 3;
            half8v bn[MF];
            half2v an[4];
            if (more_b) {
#pragma unroll
                for (int i = 0; i < MF; i++)
                    bn[i] = *reinterpret_cast<const half8v *>(stage + (size_t)brow[i] * kBK + 8 * ((2 * (s + 1) + h) ^ bsw[i]));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < MF; j++) {
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b[j], acc[j], 0, 0, 0);
                if (more_a) {
#pragma unroll
                    for (int q = j * UPM; q < (j + 1) * UPM && q < 4; q++) an[q] = expand_unit(w, k, tn, sn, q, G);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (more_a) a = half8v{ an[0][0], an[0][1], an[1][0], an[1][1], an[2][0], an[2][1], an[3][0], an[3][1] };
            if (more_b) {
#pragma unroll
                for (int i = 0; i < MF; i++) b[i] = bn[i];
            }
        }
    }
}

// Grid: 1-D and XCD-aware.  Tiles are ordered by (m-tile, k-split) "slab" first, n-tile second; workgroup b
// runs on XCD b % 8 (round-robin dispatch), and XCD x is given a contiguous run of that order, so the
// workgroups that share an L2 share an X slab and the slab is read from HBM once.
// Y_out: Y itself (ksplit == 1; res, when given, is added) or the first of ksplit partial planes of
// plane_stride floats each.
template <int TYPE, int NW, int MF>
__global__ __launch_bounds__(64 * NW) void qgemm_kernel(const uint8_t *W, size_t row_bytes, int N, int K, const _Float16 *Xp,
                                                        const float *inv_scale, int M, float *Y_out, size_t plane_stride,
                                                        const float *res, int sb_per_split, int ksplit, int tiles_n,
                                                        int n_tiles_total, int per_xcd) {
    constexpr int BM = 32 * MF, BN = 32 * NW, XI = BM / 8 / NW;
    static_assert(XI >= 1 && XI * 8 * NW == BM, "every wave issues whole 8-row LDS-DMA loads");
    constexpr int kStageHalves = BM * kBK;   // halves per stage (no padding: swizzled)
    RT_DYN_LDS(_Float16, xs);                // [4][BM][64]
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, nl = lane & 31, h = lane >> 5;
    // tile of this workgroup
    const int t = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || t >= n_tiles_total) return;
    const int slab = t / tiles_n, nt = t - slab * tiles_n;
    const int mt = slab / ksplit, kz = slab - mt * ksplit;
    const int n0 = nt * BN, m0 = mt * BM;
    const int sb0 = kz * sb_per_split, sb1 = min(K / 256, sb0 + sb_per_split);
    if (sb0 >= sb1) return;      // the launcher sizes the splits so that none is empty

    const uint8_t *rp = W + (size_t)min(n0 + wave * 32 + nl, N - 1) * row_bytes;

    // LDS-DMA: instruction i of this wave fills LDS rows (wave*XI + i)*8 .. +8 of a stage; lane L lands at
    // row + L/8, position L%8, which must hold chunk (L%8) ^ ((row >> 1) & 7) of that X row.
    const _Float16 *xsrc[XI];
#pragma unroll
    for (int i = 0; i < XI; i++) {
        int row = (wave * XI + i) * 8 + (lane >> 3);
        int c = (lane & 7) ^ ((row >> 1) & 7);
        xsrc[i] = Xp + (size_t)min(m0 + row, M - 1) * K + 8 * c;
    }
    auto issue_x = [&](int kt, int st) {
#pragma unroll
        for (int i = 0; i < XI; i++) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xsrc[i] + (size_t)kt * kBK),
                                             (__attribute__((address_space(3))) void *)(xs + (size_t)st * kStageHalves + (size_t)(wave * XI + i) * 8 * kBK),
                                             16, 0, 0);
        }
    };

    float16v acc[MF];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.f;

    // B fragment address pieces: lane (token nl of fragment i, half h) reads chunk 2s+h of row i*32 + nl
    int brow[MF], bsw[MF];
#pragma unroll
    for (int i = 0; i < MF; i++) {
        brow[i] = i * 32 + nl;
        bsw[i] = (brow[i] >> 1) & 7;
    }
    // the exponent pattern of the expansion, kept in a vector register (operand of v_and_or_b32)
    uint32_t G;
    asm volatile("v_mov_b32 %0, 0x3c003c00" : "=v"(G));

    WSb<TYPE> wc, wn;
    const int kt0 = 4 * sb0;
    issue_x(kt0, 0);
    issue_x(kt0 + 1, 1);
    issue_x(kt0 + 2, 2);
    load_sb(wc, rp, sb0, h);
    for (int sb = sb0; sb < sb1 - 1; sb++) {
        load_sb(wn, rp, sb + 1, h);
        superblock<TYPE, MF, XI, false>(acc, wc, xs, kStageHalves, brow, bsw, h, G, 4 * sb, issue_x);
        wc = wn;
    }
    superblock<TYPE, MF, XI, true>(acc, wc, xs, kStageHalves, brow, bsw, h, G, 4 * (sb1 - 1), issue_x);

    // D[i][j]: j (token) = lane % 32; i (weight row) = 8*(r/4) + 4*(lane/32) + r%4
    float *Yp = Y_out + (size_t)kz * plane_stride;
#pragma unroll
    for (int i = 0; i < MF; i++) {
        const int m = m0 + i * 32 + nl;
        if (m >= M) continue;
        const float inv = inv_scale[m];
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
            const int n = n0 + wave * 32 + 8 * g4 + 4 * h;
            if (n >= N) continue;   // N is a multiple of 4: a group of 4 rows is inside or outside as a whole
            float4 v = make_float4(acc[i][4 * g4] * inv, acc[i][4 * g4 + 1] * inv, acc[i][4 * g4 + 2] * inv, acc[i][4 * g4 + 3] * inv);
            if (res && ksplit == 1) {
                float4 rv = *reinterpret_cast<const float4 *>(res + (size_t)m * N + n);
                v.x += rv.x; v.y += rv.y; v.z += rv.z; v.w += rv.w;
            }
            *reinterpret_cast<float4 *>(Yp + (size_t)m * N + n) = v;
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

struct GemmPlan { int nw, mf, ksplit, sb_per_split; };

// Shape of the launch: waves per workgroup (tile 32*mf tokens x 32*nw rows) and k splits.
GemmPlan gemm_plan(size_t M, size_t N, size_t K) {
    GemmPlan p;
    p.mf = M > 64 ? 4 : 2;
    const size_t bm = 32 * (size_t)p.mf, tiles_m = (M + bm - 1) / bm, nsb = K / 256;
    const size_t t8 = tiles_m * ((N + 255) / 256), t4 = tiles_m * ((N + 127) / 128);
    p.ksplit = 1;
    if (t8 >= 224) {
        p.nw = 8;                 // one 8-wave workgroup per CU already fills the chip
    } else {
        p.nw = 4;                 // two 4-wave workgroups per CU: split k until the 512 slots are taken
        while (t4 * p.ksplit * 2 <= 512 && nsb / (p.ksplit * 2) >= 2 && p.ksplit < kMaxSplit) p.ksplit *= 2;
    }
    p.sb_per_split = (int)((nsb + p.ksplit - 1) / p.ksplit);
    p.ksplit = (int)((nsb + p.sb_per_split - 1) / p.sb_per_split);     // no empty split
    return p;
}

template <int TYPE, int NW, int MF>
hipError_t launch_cfg(hipStream_t s, const GemmPlan &p, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const _Float16 *Xp,
                      const float *inv_scale, size_t M, float *Y, const float *res, float *partial) {
    constexpr int BM = 32 * MF, BN = 32 * NW;
    const size_t lds = (size_t)4 * BM * kBK * sizeof(_Float16);
    auto kern = qgemm_kernel<TYPE, NW, MF>;
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    const int total = tiles_m * p.ksplit * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const size_t plane = M * N;
    kern<<<dim3((unsigned)(8 * per_xcd)), 64 * NW, lds, s>>>(w, row_bytes, (int)N, (int)K, Xp, inv_scale, (int)M, p.ksplit > 1 ? partial : Y,
                                                             plane, res, p.sb_per_split, p.ksplit, tiles_n, total, per_xcd);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || p.ksplit == 1) return e;
    const size_t n4 = plane / 4;
    const unsigned grid = (unsigned)std::min<size_t>((n4 + 255) / 256, 2048);
    splitk_reduce_kernel<<<grid, 256, 0, s>>>(partial, plane, p.ksplit, res, Y, n4);
    return hipGetLastError();
}

template <int TYPE>
hipError_t launch_type(hipStream_t s, const GemmPlan &p, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const _Float16 *Xp,
                       const float *inv_scale, size_t M, float *Y, const float *res, float *partial) {
    if (p.nw == 8 && p.mf == 4) return launch_cfg<TYPE, 8, 4>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial);
    if (p.nw == 4 && p.mf == 4) return launch_cfg<TYPE, 4, 4>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial);
    if (p.nw == 8 && p.mf == 2) return launch_cfg<TYPE, 8, 2>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial);
    return launch_cfg<TYPE, 4, 2>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial);
}

bool mfma_path(int type, size_t N, size_t K, size_t M) {
    return (type == RT_GGML_Q4_K || type == RT_GGML_Q6_K) && M >= 16 && K % 256 == 0 && N % 4 == 0;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

// workspace: fp16 X, one f32 per row of X, and the partial planes of a k-split launch
size_t qgemm_scratch_bytes(int type, size_t M, size_t N, size_t K) {
    if (!mfma_path(type, N, K, M)) return 0;
    GemmPlan p = gemm_plan(M, N, K);
    return align256(M * K * sizeof(_Float16)) + align256(M * sizeof(float)) + (p.ksplit > 1 ? (size_t)p.ksplit * M * N * sizeof(float) : 0);
}

// res (optional) is added to the result; it may be Y itself only on the row-by-row path.
hipError_t launch_qgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes,
                        const float *X, size_t M, float *Y, const float *res, void *scratch, size_t scratch_bytes) {
    if (mfma_path(type, N, K, M) && res != Y) {
        if (scratch_bytes < qgemm_scratch_bytes(type, M, N, K)) return hipErrorInvalidValue;
        const GemmPlan p = gemm_plan(M, N, K);
        char *base = reinterpret_cast<char *>(scratch);
        _Float16 *Xp = reinterpret_cast<_Float16 *>(base);
        float *inv_scale = reinterpret_cast<float *>(base + align256(M * K * sizeof(_Float16)));
        float *partial = reinterpret_cast<float *>(base + align256(M * K * sizeof(_Float16)) + align256(M * sizeof(float)));
        xprep_kernel<<<dim3((unsigned)M), 256, 0, s>>>(X, K, Xp, inv_scale);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        if (type == RT_GGML_Q4_K) return launch_type<RT_GGML_Q4_K>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial);
        return launch_type<RT_GGML_Q6_K>(s, p, w, N, K, row_bytes, Xp, inv_scale, M, Y, res, partial);
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
