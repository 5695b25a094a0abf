// Dequant-fused GEMV for up to 8 activation rows at once on the integer matrix cores (Q4_K and Q6_K weights; the callers
// send batches of 3 and more here).
//
// The one-row GEMV kernel runs a batch as grid.y passes over the weights; here the weights are streamed once.
// A wave owns 16 weight rows and a share of the super-blocks along k.  The 8 activation rows, quantized to the
// 15 bits as in the one-row kernel (per token and 32 elements a scale, and of every element a signed high plane
// q >> 7 and a low plane q & 127), are the A operand of v_mfma_i32_16x16x32_i8: matrix row i = 8 * plane + token.  The raw
// quants of 16 weight rows are the B operand (column j = weight row), so a lane's four results belong to the
// weight row whose block header that lane itself holds, and the block scales are applied lane-locally.
//
// Weights reach the lanes in two steps.  A wave loads the 16 block images of its rows with consecutive lanes on
// consecutive 16-byte pieces (a few cache lines per load instruction; lane-per-row addressing costs one line look-up per
// lane and was measured at a third of the rate), writes them to an LDS slot of its own and reads the operand
// layout back from there.
//
// Operand layout of v_mfma_i32_16x16x32_i8 (lane l, c = l / 16): A holds row l % 16, k = 8c .. 8c+7; B holds
// column l % 16, k = 8c .. 8c+7; D holds column l % 16, rows 4c .. 4c+3.
#include "rt_internal.h"
#include "rt_device.h"

#include <cstring>

namespace rt {

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kMbThreads = 512;            // 8 waves: 8 / S groups of 16 weight rows, each group's k dealt out to S waves
constexpr int kMbWaves = kMbThreads / 64;
constexpr size_t kMbLdsMax = 32 * 1024;     // the x scales (Q4_K: and block sums) in LDS: 8 tokens x 4 bytes per block of 32, i.e. K bytes each

// Quantizes up to 8 activation rows into the operand form, with the quantization step of the one-row kernel: per
// token and 32-element block a scale s = amax / 16383 (xs[block][token]) and the 15-bit values q = round(x / s) as a
// signed high plane q >> 7 and a low plane q & 127.  Per block 512 bytes in the order the lanes load them:
// [k chunk c = 0..3][matrix row i = 8 * plane + token][8 bytes], i.e. lane 16 c + i owns bytes 8 (16 c + i) .. + 7.
// xb[block][token] = s * (sum of the block's q), the x side of the -min term of Q4_K.  Tokens past `batch` are zero.
__global__ __launch_bounds__(256) void xq8_prep_kernel(const float *__restrict__ X, int batch, int K, uint8_t *__restrict__ xq,
                                                       float *__restrict__ xs, float *__restrict__ xb) {
    const int t = blockIdx.y;
    const int i4 = blockIdx.x * 256 + threadIdx.x;         // four elements per lane, eight lanes per block
    if (4 * i4 >= K) return;                               // K % 32 == 0: the lanes of a block leave together
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (t < batch) v = *reinterpret_cast<const float4 *>(X + (size_t)t * K + 4 * (size_t)i4);
    xq8_store4(v, i4, t, Xq8Work{ xq, xs, xb });
}

constexpr int kMbMaxProbs = 4;             // weight matrices of one format that meet the same prepared rows in one launch

struct MbProbDev {
    const uint8_t *w;
    size_t row_bytes;
    float *y;                              // [batch][N]
    const float *res;                      // optional, added to y; may alias y
    int N;                                 // rows
    int wg0;                               // first workgroup of the problem
};

struct MbArgs {
    MbProbDev p[kMbMaxProbs];
    int n;
    int nsb;                               // super-blocks of 256 along k
    const uint8_t *xq;
    const float *xs, *xb;                  // [K / 32][8] each
    int batch;
    int ksplit;                            // S: 1, 2, 4 or 8
};

__device__ __forceinline__ uint2 ld8(const uint8_t *p) {
    uint2 v;
    __builtin_memcpy(&v, p, 8);
    return v;
}
__device__ __forceinline__ long pack8(uint32_t lo, uint32_t hi) { return (long)(((unsigned long)hi << 32) | lo); }
__device__ __forceinline__ int mad24(int a, int b, int c) { return __mul24(a, b) + c; }
__device__ __forceinline__ float4 ldf4(const float *p) { return *reinterpret_cast<const float4 *>(p); }

// The lane's A operands of one super-block: 8 bytes of each of its 8 blocks of 32.
struct XOps {
    uint2 v[8];
};
__device__ __forceinline__ void x_load(XOps &x, const uint8_t *xq_lane, int sb) {
    const uint8_t *p = xq_lane + (size_t)sb * 4096;        // one address, eight constant offsets
#pragma unroll
    for (int b = 0; b < 8; b++) x.v[b] = ld8(p + 512 * b);
}

// Copies n floats (a multiple of 4) into LDS with the whole workgroup.
__device__ __forceinline__ void stage_floats(float *dst, const float *src, int n) {
    for (int i = 4 * threadIdx.x; i < n; i += 4 * kMbThreads) *reinterpret_cast<float4 *>(dst + i) = ldf4(src + i);
}

__device__ __forceinline__ void wave_lds_fence() {     // orders one wave's own LDS writes and reads (no workgroup barrier)
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// The images of one super-block of 16 rows as a wave loads them: 16-byte piece p = lane + 64 i is piece p % PIECES of
// row p / PIECES, and piece p of the wave's LDS slot; the last half words of 210-byte blocks follow the pieces, one
// dword per row.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <int BLOCK, int PIECES, bool TAIL> struct MbFmt {
    static constexpr int kBlock = BLOCK, kPieces = PIECES, kStride = 16 * PIECES;
    static constexpr int kLoads = (16 * PIECES + 63) / 64, kLast = 16 * PIECES - 64 * (kLoads - 1);   // lanes of the last load
    static constexpr bool kTail = TAIL;            // a last half word per row (BLOCK = 16 PIECES + 2)
    static constexpr int kSlotWords = 64 * PIECES + (TAIL ? 16 : 0);
};
using FmtQ4K = MbFmt<144, 9, false>;
using FmtQ6K = MbFmt<210, 13, true>;

template <class F> struct WImg {
    u32x4 w[F::kLoads];
    uint32_t tail;
};
template <class F> struct WOffs {
    uint32_t g[F::kLoads];                         // byte offset from the group's first row in memory
    uint32_t gt;
};
template <class F> __device__ __forceinline__ void img_offsets(WOffs<F> &o, int group, int N, size_t row_bytes) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i < F::kLoads; i++) {
        const int p = min(lane + 64 * i, 16 * F::kPieces - 1), r = p / F::kPieces, w = p % F::kPieces;
        const int rr = min(group * 16 + r, N - 1) - group * 16;        // rows past the end read the last row
        o.g[i] = (uint32_t)(rr * row_bytes) + 16 * w;
    }
    const int rt = min(group * 16 + (lane & 15), N - 1) - group * 16;
    o.gt = (uint32_t)(rt * row_bytes) + 16 * F::kPieces;
}
template <class F> __device__ __forceinline__ void img_load(WImg<F> &r, const uint8_t *blk0, const WOffs<F> &o) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i < F::kLoads; i++)
        if (i + 1 < F::kLoads || lane < F::kLast) __builtin_memcpy(&r.w[i], blk0 + o.g[i], 16);
    if (F::kTail) {
        uint16_t t;
        __builtin_memcpy(&t, blk0 + o.gt, 2);
        r.tail = t;
    }
}
template <class F> __device__ __forceinline__ void img_store(uint32_t *slot, const WImg<F> &r) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i < F::kLoads; i++)
        if (i + 1 < F::kLoads || lane < F::kLast) *reinterpret_cast<u32x4 *>(slot + 4 * (lane + 64 * i)) = r.w[i];
    if (F::kTail && lane < 16) slot[64 * F::kPieces + lane] = r.tail;
}
__device__ __forceinline__ uint2 lds8(const uint32_t *slot, int byte_off) { return *reinterpret_cast<const uint2 *>(slot + byte_off / 4); }

// The wave's place: problem, row group (16 weight rows) of it and k slice.
struct MbPlace {
    int prob, wg;                          // problem, workgroup within it
    int group, ks;
    bool live;
};
__device__ __forceinline__ MbPlace mb_place(const MbArgs &a) {
    const int wv = threadIdx.x >> 6, per_wg = kMbWaves / a.ksplit;
    MbPlace p;
    p.prob = 0;
#pragma unroll
    for (int i = 1; i < kMbMaxProbs; i++)
        if (i < a.n && (int)blockIdx.x >= a.p[i].wg0) p.prob = i;
    p.wg = blockIdx.x - a.p[p.prob].wg0;
    p.group = p.wg * per_wg + wv / a.ksplit;
    p.ks = wv % a.ksplit;
    p.live = p.group * 16 < a.p[p.prob].N;
    return p;
}

// Folds the two planes (lanes l and l ^ 32 hold the same weight row and tokens), then the k slices, and writes y.
__device__ __forceinline__ void mb_finish(const MbArgs &a, const MbPlace &pl, float (&acc)[4], float (*part)[16][8]) {
    const MbProbDev &P = a.p[pl.prob];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int j = lane & 15, c = lane >> 4;
#pragma unroll
    for (int r = 0; r < 4; r++) acc[r] += __shfl_xor(acc[r], 32, 64);
    if (c < 2) {
#pragma unroll
        for (int r = 0; r < 4; r++) part[wv][j][4 * c + r] = acc[r];
    }
    __syncthreads();
    const int per_wg = kMbWaves / a.ksplit;
    for (int e = threadIdx.x; e < 128 * per_wg; e += kMbThreads) {     // 16 rows x 8 tokens per group: up to 1024 results
        const int gl = e >> 7, jj = (e >> 3) & 15, t = e & 7;
        const int n = (pl.wg * per_wg + gl) * 16 + jj;
        float s = 0.f;
        for (int k = 0; k < a.ksplit; k++) s += part[gl * a.ksplit + k][jj][t];
        if (n < P.N && t < a.batch) {
            const size_t o = (size_t)t * P.N + n;
            if (P.res) s += P.res[o];
            P.y[o] = s;
        }
    }
}

// ---- Q4_K: 144-byte super-block = d, dmin (fp16), 12 bytes of 6-bit scales and mins, 128 bytes of nibbles;
// unit g (64 elements) = bytes 32g..32g+31, low nibbles = sub-block 2g, high nibbles = sub-block 2g+1.
struct Q4kRegs {
    uint4 hdr;
    uint2 q[4];
};
__device__ __forceinline__ void q4k_read(Q4kRegs &r, const uint32_t *slot, int j, int c) {
    const int base = j * FmtQ4K::kStride;
    const uint2 h0 = lds8(slot, base), h1 = lds8(slot, base + 8);
    r.hdr = make_uint4(h0.x, h0.y, h1.x, h1.y);
#pragma unroll
    for (int g = 0; g < 4; g++) r.q[g] = lds8(slot, base + 16 + 32 * g + 8 * c);
}

__global__ __launch_bounds__(kMbThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void qgemv_mb_q4k_kernel(MbArgs a) {
    RT_DYN_LDS(float4, lds4);                  // xs[K / 32][8], xb[K / 32][8]
    __shared__ float part[kMbWaves][16][8];
    __shared__ __align__(16) uint32_t slots[kMbWaves][FmtQ4K::kSlotWords];
    float *xs = reinterpret_cast<float *>(lds4), *xb = xs + a.nsb * 64;
    const int lane = threadIdx.x & 63;
    const int j = lane & 15, c = lane >> 4;
    uint32_t *slot = slots[threadIdx.x >> 6];
    const MbPlace pl = mb_place(a);
    const MbProbDev &P = a.p[pl.prob];
    const uint8_t *wrow = P.w + (size_t)pl.group * 16 * P.row_bytes;     // the group's first row (only read when live)
    const float pf = c < 2 ? 128.f : 1.f;      // weight of the plane this lane's results belong to
    const float mf = c < 2 ? 1.f : 0.f;        // the -min term is counted once, with the high plane
    const int tok4 = 4 * (c & 1);
    const uint8_t *xq_lane = a.xq + 8 * lane;
    float acc[4] = { 0.f, 0.f, 0.f, 0.f };
    WOffs<FmtQ4K> offs;
    img_offsets(offs, pl.group, P.N, P.row_bytes);
    WImg<FmtQ4K> img;
    Q4kRegs cur;
    XOps xc, xn;
    int sb = pl.live ? pl.ks : a.nsb;
    if (sb < a.nsb) {
        img_load(img, wrow + (size_t)sb * 144, offs);
        x_load(xc, xq_lane, sb);
    }
    stage_floats(xs, a.xs, a.nsb * 64);
    stage_floats(xb, a.xb, a.nsb * 64);
    __syncthreads();
    for (; sb < a.nsb; sb += a.ksplit) {
        const int sbn = min(sb + a.ksplit, a.nsb - 1);     // past the end a super-block is requested again: no branch around the loads
        wave_lds_fence();                      // the previous super-block's operand reads come first
        img_store(slot, img);
        wave_lds_fence();
        img_load(img, wrow + (size_t)sbn * 144, offs);   // the next image into the registers just written out
        x_load(xn, xq_lane, sbn);
        q4k_read(cur, slot, j, c);
        const float d = h2f(cur.hdr.x & 0xFFFF), dmin = h2f(cur.hdr.x >> 16);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            uint32_t scw, mw;
            if (g < 2) {
                scw = cur.hdr.y & 0x3f3f3f3fu;
                mw = cur.hdr.z & 0x3f3f3f3fu;
            } else {
                scw = (cur.hdr.w & 0x0f0f0f0fu) | ((cur.hdr.y >> 2) & 0x30303030u);
                mw = ((cur.hdr.w >> 4) & 0x0f0f0f0fu) | ((cur.hdr.z >> 2) & 0x30303030u);
            }
            scw >>= (g & 1) * 16;
            mw >>= (g & 1) * 16;
            const float wa = d * (float)(scw & 0xFF) * pf, wb = d * (float)((scw >> 8) & 0xFF) * pf;
            const float na = dmin * (float)(mw & 0xFF) * mf, nb = dmin * (float)((mw >> 8) & 0xFF) * mf;
            const long xa = pack8(xc.v[2 * g].x, xc.v[2 * g].y), xbv = pack8(xc.v[2 * g + 1].x, xc.v[2 * g + 1].y);
            const long wlo = pack8(cur.q[g].x & 0x0f0f0f0fu, cur.q[g].y & 0x0f0f0f0fu);
            const long whi = pack8((cur.q[g].x >> 4) & 0x0f0f0f0fu, (cur.q[g].y >> 4) & 0x0f0f0f0fu);
            const i32x4 z = { 0, 0, 0, 0 };
            const i32x4 da = __builtin_amdgcn_mfma_i32_16x16x32_i8(xa, wlo, z, 0, 0, 0);
            const i32x4 db = __builtin_amdgcn_mfma_i32_16x16x32_i8(xbv, whi, z, 0, 0, 0);
            const int ba = (8 * sb + 2 * g) * 8 + tok4;
            const float4 sa = ldf4(xs + ba), sbv = ldf4(xs + ba + 8), ma = ldf4(xb + ba), mb = ldf4(xb + ba + 8);
            acc[0] += (wa * sa.x) * (float)da[0] + (wb * sbv.x) * (float)db[0] - (na * ma.x + nb * mb.x);
            acc[1] += (wa * sa.y) * (float)da[1] + (wb * sbv.y) * (float)db[1] - (na * ma.y + nb * mb.y);
            acc[2] += (wa * sa.z) * (float)da[2] + (wb * sbv.z) * (float)db[2] - (na * ma.z + nb * mb.z);
            acc[3] += (wa * sa.w) * (float)da[3] + (wb * sbv.w) * (float)db[3] - (na * ma.w + nb * mb.w);
        }
        xc = xn;
    }
    mb_finish(a, pl, acc, part);
}

// ---- Q6_K: 210-byte super-block = ql[128], qh[64], int8 scales[16], d (fp16).  Element 128h + 32r + l
// (half h, run r, l = 0..31) = nibble (low for r < 2) of ql[64h + 32(r & 1) + l] | bits 2r..2r+1 of
// qh[32h + l] << 4, minus 32; scale index 8h + 2r + l / 16.
struct Q6kRegs {
    uint2 ql[4], qh[2];                    // ql[2h + (r & 1)], qh[h]: the lane's 8 byte positions
    uint32_t sc[4];
    uint32_t d;
};
__device__ __forceinline__ void q6k_read(Q6kRegs &r, const uint32_t *slot, int j, int c) {
    const int base = j * FmtQ6K::kStride;
#pragma unroll
    for (int i = 0; i < 4; i++) r.ql[i] = lds8(slot, base + 32 * i + 8 * c);
#pragma unroll
    for (int h = 0; h < 2; h++) r.qh[h] = lds8(slot, base + 128 + 32 * h + 8 * c);
    const uint2 s0 = lds8(slot, base + 192), s1 = lds8(slot, base + 200);
    r.sc[0] = s0.x; r.sc[1] = s0.y; r.sc[2] = s1.x; r.sc[3] = s1.y;
    r.d = slot[64 * FmtQ6K::kPieces + j];
}

// Four 6-bit values of run r (nibbles of ql, bit pairs of qh) as signed bytes -32..31: bytes 0..63 plus 0x60 do not
// carry into the next byte, and flipping bit 7 then takes off 0x80.
template <int R> __device__ __forceinline__ uint32_t q6k_bytes(uint32_t ql, uint32_t qh) {
    const uint32_t lo = (R < 2 ? ql : ql >> 4) & 0x0f0f0f0fu, hi = (qh >> (2 * R)) & 0x03030303u;
    return (((hi << 4) | lo) + 0x60606060u) ^ 0x80808080u;
}

template <int H, int R>
__device__ __forceinline__ void q6k_run(const Q6kRegs &w, const XOps &x, uint32_t keep0, const float *xs_blk, float (&acc)[4]) {
    const uint32_t vx = q6k_bytes<R>(w.ql[2 * H + (R & 1)].x, w.qh[H].x), vy = q6k_bytes<R>(w.ql[2 * H + (R & 1)].y, w.qh[H].y);
    // The two 16-element runs of a 32-element block have their own scale.  One matrix instruction over the whole block
    // (S0 + S1) and one with the second run's k positions (lanes c >= 2) zeroed in the weight operand (S0):
    // s0 S0 + s1 S1 = (s0 - s1) S0 + s1 (S0 + S1).
    const long wall = pack8(vx, vy), w0 = pack8(vx & keep0, vy & keep0);
    const long xa = pack8(x.v[4 * H + R].x, x.v[4 * H + R].y);
    const i32x4 z = { 0, 0, 0, 0 };
    const i32x4 dall = __builtin_amdgcn_mfma_i32_16x16x32_i8(xa, wall, z, 0, 0, 0);
    const i32x4 d0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(xa, w0, z, 0, 0, 0);
    // scales 8H + 2R (first run) and 8H + 2R + 1 (second run), signed bytes; |s d| < 2^24
    const uint32_t word = w.sc[2 * H + R / 2];
    const int s0 = (int)(word << (24 - 16 * (R & 1))) >> 24, s1 = (int)(word << (16 - 16 * (R & 1))) >> 24;
    const int sd = s0 - s1;
    const float4 sx = ldf4(xs_blk + (4 * H + R) * 8);
    acc[0] += sx.x * (float)mad24(sd, d0[0], __mul24(s1, dall[0]));
    acc[1] += sx.y * (float)mad24(sd, d0[1], __mul24(s1, dall[1]));
    acc[2] += sx.z * (float)mad24(sd, d0[2], __mul24(s1, dall[2]));
    acc[3] += sx.w * (float)mad24(sd, d0[3], __mul24(s1, dall[3]));
}

__global__ __launch_bounds__(kMbThreads) void qgemv_mb_q6k_kernel(MbArgs a) {
    RT_DYN_LDS(float4, lds4);                  // xs[K / 32][8]
    __shared__ float part[kMbWaves][16][8];
    __shared__ __align__(16) uint32_t slots[kMbWaves][FmtQ6K::kSlotWords];
    float *xs = reinterpret_cast<float *>(lds4);
    const int lane = threadIdx.x & 63;
    const int j = lane & 15, c = lane >> 4;
    uint32_t *slot = slots[threadIdx.x >> 6];
    const MbPlace pl = mb_place(a);
    const MbProbDev &P = a.p[pl.prob];
    const uint8_t *wrow = P.w + (size_t)pl.group * 16 * P.row_bytes;     // the group's first row (only read when live)
    const float pf = c < 2 ? 128.f : 1.f;
    const int tok4 = 4 * (c & 1);
    const uint32_t keep0 = c < 2 ? 0xFFFFFFFFu : 0u;
    const uint8_t *xq_lane = a.xq + 8 * lane;
    float acc[4] = { 0.f, 0.f, 0.f, 0.f };
    WOffs<FmtQ6K> offs;
    img_offsets(offs, pl.group, P.N, P.row_bytes);
    WImg<FmtQ6K> img;
    Q6kRegs cur;
    XOps xc, xn;
    int sb = pl.live ? pl.ks : a.nsb;
    if (sb < a.nsb) {
        img_load(img, wrow + (size_t)sb * 210, offs);
        x_load(xc, xq_lane, sb);
    }
    stage_floats(xs, a.xs, a.nsb * 64);
    __syncthreads();
    for (; sb < a.nsb; sb += a.ksplit) {
        const int sbn = min(sb + a.ksplit, a.nsb - 1);     // past the end a super-block is requested again: no branch around the loads
        wave_lds_fence();                      // the previous super-block's operand reads come first
        img_store(slot, img);
        wave_lds_fence();
        img_load(img, wrow + (size_t)sbn * 210, offs);   // the next image into the registers just written out
        x_load(xn, xq_lane, sbn);
        q6k_read(cur, slot, j, c);
        const float *xs_blk = xs + 8 * sb * 8 + tok4;
        float part_sb[4] = { 0.f, 0.f, 0.f, 0.f };           // the super-block's sum before its scale d
        q6k_run<0, 0>(cur, xc, keep0, xs_blk, part_sb);
        q6k_run<0, 1>(cur, xc, keep0, xs_blk, part_sb);
        q6k_run<0, 2>(cur, xc, keep0, xs_blk, part_sb);
        q6k_run<0, 3>(cur, xc, keep0, xs_blk, part_sb);
        q6k_run<1, 0>(cur, xc, keep0, xs_blk, part_sb);
        q6k_run<1, 1>(cur, xc, keep0, xs_blk, part_sb);
        q6k_run<1, 2>(cur, xc, keep0, xs_blk, part_sb);
        q6k_run<1, 3>(cur, xc, keep0, xs_blk, part_sb);
        const float d = h2f(cur.d);
#pragma unroll
        for (int r = 0; r < 4; r++) acc[r] += d * part_sb[r];
        xc = xn;
    }
#pragma unroll
    for (int r = 0; r < 4; r++) acc[r] *= pf;
    mb_finish(a, pl, acc, part);
}

}  // namespace

bool qgemv_mb_serves(int type, size_t N, size_t K, int batch) {
    if (type != RT_GGML_Q4_K && type != RT_GGML_Q6_K) return false;
    return batch >= kGemvMbMinBatch && batch <= 8 && N >= 1 && N < ((size_t)1 << 31) && K >= 256 && K % 256 == 0 &&
           (type == RT_GGML_Q4_K ? 2 : 1) * K <= kMbLdsMax;
}

size_t qgemv_mb_scratch_bytes(size_t K) { return 16 * K + 2 * (K / 32 * 8 * 4); }

hipError_t launch_qgemv_mb_prep(hipStream_t s, const float *x, int batch, size_t K, void *work) {
    if (!x || !work || batch < 1 || batch > 8 || K < 256 || K % 256 != 0) return hipErrorInvalidValue;
    if (((uintptr_t)x & 15) || ((uintptr_t)work & 255)) return hipErrorInvalidValue;
    uint8_t *xq = static_cast<uint8_t *>(work);
    float *xs = reinterpret_cast<float *>(xq + 16 * K);
    float *xb = xs + K / 4;
    dim3 pg((unsigned)((K / 4 + 255) / 256), 8);
    xq8_prep_kernel<<<pg, 256, 0, s>>>(x, batch, (int)K, xq, xs, xb);
    return hipGetLastError();
}

hipError_t launch_qgemv_mb_group(hipStream_t s, int type, const MbProb *probs, int n, size_t K, int batch, const void *work) {
    if (!probs || n < 1 || n > kMbMaxProbs || !work || ((uintptr_t)work & 255)) return hipErrorInvalidValue;
    const size_t block = type == RT_GGML_Q4_K ? 144 : 210, nsb = K / 256;
    size_t groups = 0;
    for (int i = 0; i < n; i++) {
        const MbProb &q = probs[i];
        if (!qgemv_mb_serves(type, q.N, K, batch) || !q.w || !q.y) return hipErrorInvalidValue;
        if (type == RT_GGML_Q4_K && (((uintptr_t)q.w & 15) || q.row_bytes % 16)) return hipErrorInvalidValue;   // 16-byte pieces of 16-byte aligned blocks
        if (q.row_bytes < nsb * block || q.row_bytes * 16 >= ((size_t)1 << 32)) return hipErrorInvalidValue;    // 32-bit offsets within a group of rows
        groups += (q.N + 15) / 16;
    }
    // k is dealt out to S waves per group of 16 rows.  Among the S that give every SIMD two waves, the one whose
    // workgroups divide most evenly over the 256 CUs (344 workgroups would leave a third of the CUs with twice the work
    // of the others); the smaller S on a tie.  Short of 2048 waves: the largest S the row allows.
    int ksplit = 0;
    double best = 0;
    for (int sp = 1; sp <= kMbWaves; sp *= 2) {
        if ((size_t)sp > nsb || groups * sp < 2048) continue;
        const double wgs = (double)((groups * sp + kMbWaves - 1) / kMbWaves), uneven = (double)(((size_t)wgs + 255) / 256) * 256.0 / wgs;
        if (!ksplit || uneven < best - 1e-9) { ksplit = sp; best = uneven; }
    }
    if (!ksplit) {
        ksplit = kMbWaves;
        while ((size_t)ksplit > nsb) ksplit /= 2;
    }
    const size_t per_wg = kMbWaves / ksplit;
    MbArgs a;
    memset(&a, 0, sizeof a);
    const uint8_t *xq = static_cast<const uint8_t *>(work);
    a.n = n; a.nsb = (int)nsb; a.xq = xq; a.xs = reinterpret_cast<const float *>(xq + 16 * K); a.xb = a.xs + K / 4;
    a.batch = batch; a.ksplit = ksplit;
    size_t wgs = 0;
    for (int i = 0; i < n; i++) {
        a.p[i] = MbProbDev{ static_cast<const uint8_t *>(probs[i].w), probs[i].row_bytes, probs[i].y, probs[i].res, (int)probs[i].N, (int)wgs };
        wgs += ((probs[i].N + 15) / 16 + per_wg - 1) / per_wg;
    }
    if (wgs >= ((size_t)1 << 31)) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)wgs;
    if (type == RT_GGML_Q4_K) qgemv_mb_q4k_kernel<<<grid, kMbThreads, 2 * K, s>>>(a);     // x scales and block sums
    else qgemv_mb_q6k_kernel<<<grid, kMbThreads, K, s>>>(a);
    return hipGetLastError();
}

hipError_t launch_qgemv_mb(hipStream_t s, int type, const void *w, size_t row_bytes, size_t N, size_t K, const float *x, int batch,
                           float *y, const float *res, void *work) {
    if (!qgemv_mb_serves(type, N, K, batch)) return hipErrorInvalidValue;
    hipError_t e = launch_qgemv_mb_prep(s, x, batch, K, work);
    if (e != hipSuccess) return e;
    const MbProb p{ w, row_bytes, N, y, res };
    return launch_qgemv_mb_group(s, type, &p, 1, K, batch, work);
}

}  // namespace rt
