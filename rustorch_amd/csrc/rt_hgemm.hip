// Prefill contraction for the formats that have no fused dequantizing kernel: Y[M,N] = X[M,K] . W[N,K]^T with W as
// fp16.  Unquantized F16 matrices are read as they are; the other formats (and F32) are first written out as an fp16
// copy in the caller's workspace -- the exact block decode, rounded once to fp16 (relative 2^-11 per weight, three
// orders of magnitude inside the tolerance of 1e-3 * |w_row| * |x| on a dot product).  Y = x . W^T as in
// Linear::forward (src/nn/linear.rs:150-270).
//
// The kernel keeps no tile in LDS: both matrix operands of v_mfma_f32_32x32x16_f16 are 16 contiguous bytes of a row
// per lane (row = lane % 32, k = 8 * (lane / 32) .. + 7), so a wave loads its fragments straight from global memory /
// L2, three k steps ahead of the matrix instructions, and never meets another wave.  A wave owns 64 weight rows x
// 32 * MT tokens; k is split over grid.z, the splits leave partial planes for the plane-sum consumers.
// X goes in as fp16 scaled per row by a power of two (largest magnitude in [2^14, 2^15)); the result is scaled back.
#include "rt_device.h"

#include <algorithm>

namespace rt {

namespace {

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

// fp16 copy of a weight matrix, one thread per 8 consecutive elements of a row (K % 8 == 0)
#pragma clang fp contract(off)
__global__ __launch_bounds__(256) void dequant_f16_kernel(int type, const uint8_t *w, size_t row_bytes, size_t n_rows, size_t n_cols,
                                                          _Float16 *out) {
    const size_t per_row = n_cols / 8, total = n_rows * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / per_row, c = 8 * (i % per_row);
        const uint8_t *row = w + r * row_bytes;
        half8v o;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = (_Float16)deq_elem(type, row, c + e);
        *reinterpret_cast<half8v *>(out + r * n_cols + c) = o;
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

constexpr int kHWaves = 4;      // waves per workgroup, side by side along the weight rows
constexpr int kHRing = 4;       // k steps (16 elements each) in the register ring: fragments are requested three steps ahead

// grid (ceil(N / (64 * kHWaves)), ceil(M / (32 MT)), ksplit); the split z covers k in [z * k_per_split, min(K, (z + 1) * k_per_split)),
// k_per_split a multiple of 64.  planes: ksplit planes of M x N floats.  A wave owns 64 weight rows x 32 MT tokens.
template <int MT>
__global__ __launch_bounds__(64 * kHWaves, 2) void hgemm_kernel(const _Float16 *W, const _Float16 *Xh, const float *inv_scale, float *planes,
                                                                int N, int K, int M, int k_per_split) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), r = lane & 31, hh = lane >> 5;
    const int n0 = (blockIdx.x * kHWaves + wave) * 64, m0 = blockIdx.y * 32 * MT;
    if (n0 >= N) return;                                       // whole wave outside the matrix (no barrier in this kernel)
    const int k0 = blockIdx.z * k_per_split, k1 = min(K, k0 + k_per_split);
    // rows / tokens past the end repeat the last one; their results are never stored
    const _Float16 *wp[2] = { W + (size_t)min(n0 + r, N - 1) * K + 8 * hh, W + (size_t)min(n0 + 32 + r, N - 1) * K + 8 * hh };
    const _Float16 *xp[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) xp[t] = Xh + (size_t)min(m0 + 32 * t + r, M - 1) * K + 8 * hh;

    float16v acc[MT][2];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[t][c][i] = 0.f;

    half8v wf[kHRing][2], xf[kHRing][MT];
    auto request = [&](int st, int k) {
        k = min(k, k1 - 16);                                   // past the end a step requests the last one again (no branch around loads)
        wf[st][0] = *reinterpret_cast<const half8v *>(wp[0] + k);
        wf[st][1] = *reinterpret_cast<const half8v *>(wp[1] + k);
#pragma unroll
        for (int t = 0; t < MT; t++) xf[st][t] = *reinterpret_cast<const half8v *>(xp[t] + k);
    };
    auto consume = [&](int st) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
            acc[t][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[st][t], wf[st][0], acc[t][0], 0, 0, 0);
            acc[t][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[st][t], wf[st][1], acc[t][1], 0, 0, 0);
        }
    };
    request(0, k0);
    request(1, k0 + 16);
    request(2, k0 + 32);
    for (int k = k0; k < k1; k += 64) {                        // k1 - k0 is a multiple of 64
        request(3, k + 48); consume(0);
        request(0, k + 64); consume(1);
        request(1, k + 80); consume(2);
        request(2, k + 96); consume(3);
    }

    // X is the first operand: register i of lane (r, hh) holds token 8 (i / 4) + 4 hh + i % 4 of fragment t and weight
    // row r of column block c, so a store instruction writes two runs of 32 consecutive floats
    float *yp = planes + (size_t)blockIdx.z * (size_t)M * (size_t)N;
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const int n = n0 + 32 * c + r;
        if (n < N) {
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int m = m0 + 32 * t + 8 * (i >> 2) + 4 * hh + (i & 3);
                    if (m < M) yp[(size_t)m * N + n] = acc[t][c][i] * inv_scale[m];
                }
        }
    }
}

struct HPlan { int mt, ksplit, kps; };

HPlan hgemm_plan(size_t M, size_t N, size_t K) {
    HPlan p;
    p.mt = M > 64 ? 4 : (M > 32 ? 2 : 1);
    const size_t waves = ((N + 63) / 64) * ((M + 32 * (size_t)p.mt - 1) / (32 * (size_t)p.mt));
    // split k until there are about two waves per SIMD (256 CUs x 4 SIMDs), each split at least 256 long
    size_t ks = 1;
    while (waves * ks * 2 <= 2048 && K / (ks * 2) >= 256 && ks < 16) ks *= 2;
    size_t kps = ((K + ks - 1) / ks + 63) / 64 * 64;
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

hipError_t launch_hgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const float *X, size_t M, float *Y,
                        const float *res, void *scratch, size_t scratch_bytes) {
    if (!hgemm_serves(type, M, N, K) || N % 4 != 0 || M > 65535 * 32 || N * K >= ((size_t)1 << 40)) return hipErrorInvalidValue;
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
        const size_t total = N * (K / 8);
        dequant_f16_kernel<<<dim3((unsigned)std::min<size_t>((total + 255) / 256, 65536)), 256, 0, s>>>(type, w, row_bytes, N, K, copy);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        Wh = copy;
    }
    float *planes = reinterpret_cast<float *>(after);
    xscale_f16_kernel<<<dim3((unsigned)M), 256, 0, s>>>(X, K, Xh, inv);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const dim3 grid((unsigned)((N + 64 * kHWaves - 1) / (64 * kHWaves)), (unsigned)((M + 32 * p.mt - 1) / (32 * p.mt)), (unsigned)p.ksplit);
    if (p.mt == 4) hgemm_kernel<4><<<grid, 64 * kHWaves, 0, s>>>(Wh, Xh, inv, planes, (int)N, (int)K, (int)M, p.kps);
    else if (p.mt == 2) hgemm_kernel<2><<<grid, 64 * kHWaves, 0, s>>>(Wh, Xh, inv, planes, (int)N, (int)K, (int)M, p.kps);
    else hgemm_kernel<1><<<grid, 64 * kHWaves, 0, s>>>(Wh, Xh, inv, planes, (int)N, (int)K, (int)M, p.kps);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_plane_sum(s, PlaneSum{ planes, M * N, p.ksplit }, res, Y, M * N);
}

}  // namespace rt
