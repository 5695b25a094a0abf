// Stand-alone dequant-fused GEMV launch (decode, batch 1..8): y = dequant(W) . x with W in raw GGUF blocks.
// Workgroups of 1024 threads (one per CU) for small launches, of 512 threads (two per CU) for large ones;
// device code in rt_gemv_device.h.
#include "rt_gemv_device.h"

#include <algorithm>

namespace rt {

namespace {

// Launches that stream less than this many weight bytes use 1024-thread workgroups: with few rows per wave
// the start-up (one staging of x per workgroup) dominates and fewer, larger workgroups pay it less often.
// Larger launches run faster with two 512-thread workgroups per CU, which do not stall on each other's barriers.
#ifndef RT_GEMV_BIG_BYTES
#define RT_GEMV_BIG_BYTES (64.0 * 1024 * 1024)
#endif

template <int THREADS>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void qgemv_kernel(GemvArgs a, int r2) {
    RT_DYN_LDS(uint4, lds4);
    __shared__ float red[THREADS / 64];
    uint32_t *lds = reinterpret_cast<uint32_t *>(lds4);
    const int wg = blockIdx.x;
    int pi = 0;
#pragma unroll
    for (int i = 1; i < kMaxGemvProbs; i++)
        if (i < a.n && wg >= a.p[i].tile0) pi = i;
    const GemvProb &P = a.p[pi];
    gemv_dispatch<false, true>(P, wg - P.tile0, P.rows_per_tile, blockIdx.y, r2 != 0, lds, red);
}

}  // namespace

// Gives every problem a share of the workgroups in proportion to its weight bytes (tile0 = first workgroup,
// rows_per_tile = number of workgroups of the problem) and launches one grid over all of them
// (grid.y = batch row).  Workgroups of a problem stage x once and deal its rows out round-robin.
hipError_t launch_qgemv(hipStream_t s, GemvArgs &a, int batch) {
    if (a.n <= 0 || a.n > kMaxGemvProbs || batch <= 0) return hipErrorInvalidValue;
    double total_bytes = 0;
    size_t lds = 0, total_rows = 0;
    for (int i = 0; i < a.n; i++) {
        if ((double)a.p[i].N * (double)a.p[i].row_bytes >= 4294967296.0) return hipErrorInvalidValue;   // row offsets are 32-bit
        if ((a.p[i].type == RT_GGML_Q5_K || a.p[i].type == RT_GGML_Q3_K || a.p[i].type == RT_GGML_Q2_K) && a.p[i].epi == kEpiSwiglu)
            return hipErrorInvalidValue;   // no pair form for these
        total_bytes += (double)a.p[i].N * (double)a.p[i].row_bytes * (a.p[i].epi == kEpiSwiglu ? 2.0 : 1.0);
        total_rows += (size_t)a.p[i].N;
        lds = std::max(lds, gemv_lds_bytes(a.p[i].type, (size_t)a.p[i].K));
    }
    if (total_bytes <= 0) return hipErrorInvalidValue;
    // 16 resident waves per CU over 256 CUs, as one or two workgroups
    const int threads = total_bytes >= RT_GEMV_BIG_BYTES ? 512 : 1024;
    const int kGemvWaves = threads / 64;
    int budget = 256 * (1024 / threads) / batch;
    if (budget < a.n) budget = a.n;
    // two rows per wave step once every wave has at least three steps of work, else one
    const int r2 = total_rows >= (size_t)3 * 2 * (size_t)budget * kGemvWaves ? 1 : 0;
    int wgs = 0;
    for (int i = 0; i < a.n; i++) {
        const GemvProb &p = a.p[i];
        double bytes = (double)p.N * (double)p.row_bytes * (p.epi == kEpiSwiglu ? 2.0 : 1.0);
        int n = (int)(budget * (bytes / total_bytes) + 0.5);
        int rows_per_group = (p.epi == kEpiSwiglu) ? 1 : (r2 ? 2 : 1);
        int max_useful = ((p.N + rows_per_group - 1) / rows_per_group + kGemvWaves - 1) / kGemvWaves;
        if (n > max_useful) n = max_useful;
        if (n < 1) n = 1;
        a.p[i].tile0 = wgs;
        a.p[i].rows_per_tile = n;
        wgs += n;
    }
    if (lds > kGemvLdsMax) return hipErrorInvalidValue;    // x of the longest row must fit the workgroup's LDS
    dim3 grid((unsigned)wgs, (unsigned)batch);
    if (lds > 64 * 1024) {
        // rows longer than 27 000 elements (the 70B-class FFN): more than the default 64 KB of dynamic LDS, granted per
        // kernel and device on request
        static bool attr_set[2][64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorInvalidDevice;
        const int which = threads == 512 ? 0 : 1;
        if (!attr_set[which][dev]) {
            const void *fn = which == 0 ? (const void *)qgemv_kernel<512> : (const void *)qgemv_kernel<1024>;
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGemvLdsMax);
            if (e != hipSuccess) return e;
            attr_set[which][dev] = true;
        }
    }
    if (threads == 512) qgemv_kernel<512><<<grid, 512, lds, s>>>(a, r2);
    else qgemv_kernel<1024><<<grid, 1024, lds, s>>>(a, r2);
    return hipGetLastError();
}

}  // namespace rt
