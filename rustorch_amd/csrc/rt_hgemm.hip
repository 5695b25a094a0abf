// Prefill contraction for the formats that have no fused dequantizing kernel: Y[M,N] = X[M,K] . W[N,K]^T with W as
// fp16.  Unquantized F16 matrices are read as they are; the other formats (and F32) are first written out as an fp16
// copy in the caller's workspace -- the exact block decode, rounded once to fp16 (relative 2^-11 per weight, three
// orders of magnitude inside the tolerance of 1e-3 * |w_row| * |x| on a dot product).  Y = x . W^T as in
// Linear::forward (src/nn/linear.rs:150-270).
//
// A workgroup of four waves owns 128 weight rows x 128 tokens; 64-wide k stages of both operands go through a
// double-buffered, swizzled LDS tile (fetched with fully used 128-byte lines), and each wave multiplies 64 x 64 of it
// with v_mfma_f32_32x32x16_f16.  k is split over grid.z, the splits leave partial planes that splitk_reduce_kernel sums.
// X goes in as fp16 scaled per row by a power of two (largest magnitude in [2^14, 2^15)); the result is scaled back.
#include "rt_device.h"

#include <algorithm>

namespace rt {

namespace {

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

// fp16 copy of a weight matrix, one thread per 32 consecutive elements of a row (K % 32 == 0): the 32 share their
// block header, which the compiler then decodes once
#pragma clang fp contract(off)
__global__ __launch_bounds__(256) void dequant_f16_kernel(int type, const uint8_t *w, size_t row_bytes, size_t n_rows, size_t n_cols,
                                                          _Float16 *out) {
    const size_t per_row = n_cols / 32, total = n_rows * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / per_row, c = 32 * (i % per_row);
        const uint8_t *row = w + r * row_bytes;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            half8v o;
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = (_Float16)deq_elem(type, row, c + 8 * g + e);
            *reinterpret_cast<half8v *>(out + r * n_cols + c + 8 * g) = o;
        }
    }
}
#pragma clang fp contract(fast)

// X f32 [M,K] -> fp16 [M,K] in place order, scaled per row; inv_scale[m] undoes the scale.  One workgroup per row.
__global__ __launch_bounds__(256) void xscale_f16_kernel(const float *X, size_t K, _Float16 *Xh, float *inv_scale) {
    __shared__ float red[4];
    const size_t m = blockIdx.x;
    const float4 *x4 = reinterpret_cast<const float4 *>(X + m * K);
    float amax = 0.f;
    for (size_t i = threadIdx.x; i < K / 4; i += 256) {
        const float4 v = x4[i];
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    amax = block_max(amax, red);
    int e = 0;
    float scale = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        (void)frexpf(amax, &e);
        int se = 15 - e;
        se = se > 100 ? 100 : (se < -100 ? -100 : se);
        scale = ldexpf(1.f, se);
        inv = ldexpf(1.f, -se);
    }
    if (threadIdx.x == 0) inv_scale[m] = inv;
    for (size_t i = threadIdx.x; i < K / 4; i += 256) {
        const float4 v = x4[i];
        _Float16 *o = Xh + m * K + 4 * i;
        o[0] = (_Float16)(v.x * scale); o[1] = (_Float16)(v.y * scale); o[2] = (_Float16)(v.z * scale); o[3] = (_Float16)(v.w * scale);
    }
}

constexpr int kHT = 128;        // tile: 128 weight rows x 128 tokens per workgroup (4 waves, 64 x 64 each)
constexpr int kHK = 64;         // k per LDS stage: one 128-byte line per row

// byte offset of 16-byte chunk c (0..7) of row r in a 128 x 64 fp16 stage: rows two apart fall on different chunk
// slots, so the 32 rows of a matrix fragment spread over all banks (no conflicts on the b128 reads)
__device__ __forceinline__ uint32_t stage_off(int r, int c) { return (uint32_t)r * 128u + 16u * (uint32_t)(c ^ ((r >> 1) & 7)); }

// grid (ceil(N / 128), ceil(M / 128), ksplit); split z covers k in [z * k_per_split, min(K, (z + 1) * k_per_split)), k_per_split a
// multiple of 64.  planes: ksplit planes of M x N floats.  LDS: two stages of {W tile, X tile}, 64 KB.
// A stage is fetched with fully used lines (8 lanes per row), held in registers while the previous stage is multiplied,
// then written to the other LDS buffer: one barrier per stage.
__global__ __launch_bounds__(256) void hgemm_kernel(const _Float16 *W, const _Float16 *Xh, const float *inv_scale, float *planes, int N, int K,
                                                    int M, int k_per_split) {
    __shared__ __align__(16) uint8_t lds[2][2][kHT * kHK * 2];      // [buffer][W | X][128 rows x 128 bytes]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, hh = lane >> 5;
    const int wn = wave & 1, wm = wave >> 1;
    const int n0 = blockIdx.x * kHT, m0 = blockIdx.y * kHT;
    const int k0 = blockIdx.z * k_per_split, k1 = min(K, k0 + k_per_split), T = (k1 - k0) / kHK;

    // the thread's four chunks of each tile: chunk q = tid + 256 i is row q / 8, 16-byte column q % 8
    const _Float16 *wsrc[4], *xsrc[4];
    uint32_t dst[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int q = tid + 256 * i, row = q >> 3, c = q & 7;
        wsrc[i] = W + (size_t)min(n0 + row, N - 1) * K + k0 + 8 * c;      // rows past the end repeat the last one; never stored
        xsrc[i] = Xh + (size_t)min(m0 + row, M - 1) * K + k0 + 8 * c;
        dst[i] = stage_off(row, c);
    }
    half8v wreg[4], xreg[4];
    auto fetch = [&](int t) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            wreg[i] = *reinterpret_cast<const half8v *>(wsrc[i] + (size_t)t * kHK);
            xreg[i] = *reinterpret_cast<const half8v *>(xsrc[i] + (size_t)t * kHK);
        }
    };
    auto park = [&](int b) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *reinterpret_cast<half8v *>(&lds[b][0][dst[i]]) = wreg[i];
            *reinterpret_cast<half8v *>(&lds[b][1][dst[i]]) = xreg[i];
        }
    };

    float16v acc[2][2];           // [token fragment][row fragment]
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;

    fetch(0);
    park(0);
    __syncthreads();
    for (int t = 0; t < T; t++) {
        const int b = t & 1;
        if (t + 1 < T) fetch(t + 1);                           // uniform over the workgroup
#pragma unroll
        for (int s4 = 0; s4 < 4; s4++) {
            half8v wf[2], xf[2];
#pragma unroll
            for (int c2 = 0; c2 < 2; c2++) {
                wf[c2] = *reinterpret_cast<const half8v *>(&lds[b][0][stage_off(wn * 64 + 32 * c2 + r, 2 * s4 + hh)]);
                xf[c2] = *reinterpret_cast<const half8v *>(&lds[b][1][stage_off(wm * 64 + 32 * c2 + r, 2 * s4 + hh)]);
            }
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int c2 = 0; c2 < 2; c2++) acc[a][c2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[a], wf[c2], acc[a][c2], 0, 0, 0);
        }
        if (t + 1 < T) park(b ^ 1);                            // the other buffer: its readers passed the barrier of the step before
        __syncthreads();
    }

    // X is the first operand: register i of lane (r, hh) holds token 8 (i / 4) + 4 hh + i % 4 of token fragment a and weight
    // row r of row fragment c2, so a store instruction writes two runs of 32 consecutive floats
    float *yp = planes + (size_t)blockIdx.z * (size_t)M * (size_t)N;
#pragma unroll
    for (int c2 = 0; c2 < 2; c2++) {
        const int n = n0 + wn * 64 + 32 * c2 + r;
        if (n < N) {
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int m = m0 + wm * 64 + 32 * a + 8 * (i >> 2) + 4 * hh + (i & 3);
                    if (m < M) yp[(size_t)m * N + n] = acc[a][c2][i] * inv_scale[m];
                }
        }
    }
}

struct HPlan { int ksplit, kps; };

HPlan hgemm_plan(size_t M, size_t N, size_t K) {
    HPlan p;
    const size_t tiles = ((N + kHT - 1) / kHT) * ((M + kHT - 1) / kHT);
    // split k until there are two workgroups per CU (256 CUs), each split at least 256 long
    size_t ks = 1;
    while (tiles * ks * 2 <= 512 && K / (ks * 2) >= 256 && ks < 16) ks *= 2;
    size_t kps = ((K + ks - 1) / ks + kHK - 1) / kHK * kHK;
    p.kps = (int)kps;
    p.ksplit = (int)((K + kps - 1) / kps);
    return p;
}

size_t align256h(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

bool hgemm_serves(int type, size_t M, size_t N, size_t K) {
    // below 32 rows the GEMV kernel run once per row is as fast as making the fp16 copy
    return M >= 32 && K % 64 == 0 && K >= 64 && N % 4 == 0 && type_block_elems(type) != 0 && !qgemm_on_matrix_cores(type, M, N, K);
}

// workspace: fp16 X, its row scales, the fp16 copy of W (not for F16 weights), the partial planes
size_t hgemm_scratch_bytes(int type, size_t M, size_t N, size_t K) {
    const HPlan p = hgemm_plan(M, N, K);
    return align256h(M * K * 2) + align256h(M * 4) + (type == RT_GGML_F16 ? 0 : align256h(N * K * 2)) + (size_t)p.ksplit * M * N * 4;
}

// fp16 copy of a whole weight matrix (N x K halves), for a caller that keeps it beside the blocks
hipError_t launch_weights_f16(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes, _Float16 *out) {
    if (type_block_elems(type) == 0 || K % 32 != 0 || N == 0 || K == 0 || ((uintptr_t)out & 15)) return hipErrorInvalidValue;
    const size_t total = N * (K / 32);
    dequant_f16_kernel<<<dim3((unsigned)std::min<size_t>((total + 255) / 256, 65536)), 256, 0, s>>>(type, w, row_bytes, N, K, out);
    return hipGetLastError();
}

// w_f16 (optional): a ready fp16 copy of the matrix; then no copy is made and the workspace needs no room for one
hipError_t launch_hgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const float *X, size_t M, float *Y,
                        const float *res, void *scratch, size_t scratch_bytes, const _Float16 *w_f16) {
    if (!hgemm_serves(type, M, N, K) || N % 4 != 0 || M > 65535 * 128 || N * K >= ((size_t)1 << 40)) return hipErrorInvalidValue;
    if (w_f16) {
        w = reinterpret_cast<const uint8_t *>(w_f16);
        type = RT_GGML_F16;
    }
    if (scratch_bytes < hgemm_scratch_bytes(type, M, N, K)) return hipErrorInvalidValue;
    if (((uintptr_t)w | (uintptr_t)X | (uintptr_t)scratch) & 15) return hipErrorInvalidValue;
    const HPlan p = hgemm_plan(M, N, K);
    char *base = reinterpret_cast<char *>(scratch);
    _Float16 *Xh = reinterpret_cast<_Float16 *>(base);
    float *inv = reinterpret_cast<float *>(base + align256h(M * K * 2));
    char *after = base + align256h(M * K * 2) + align256h(M * 4);
    const _Float16 *Wh;
    if (type == RT_GGML_F16) {
        Wh = reinterpret_cast<const _Float16 *>(w);
    } else {
        _Float16 *copy = reinterpret_cast<_Float16 *>(after);
        after += align256h(N * K * 2);
        hipError_t e = launch_weights_f16(s, type, w, N, K, row_bytes, copy);
        if (e != hipSuccess) return e;
        Wh = copy;
    }
    float *planes = reinterpret_cast<float *>(after);
    xscale_f16_kernel<<<dim3((unsigned)M), 256, 0, s>>>(X, K, Xh, inv);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const dim3 grid((unsigned)((N + kHT - 1) / kHT), (unsigned)((M + kHT - 1) / kHT), (unsigned)p.ksplit);
    hgemm_kernel<<<grid, 256, 0, s>>>(Wh, Xh, inv, planes, (int)N, (int)K, (int)M, p.kps);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_plane_sum(s, PlaneSum{ planes, M * N, p.ksplit }, res, Y, M * N);
}

}  // namespace rt
