// Stand-alone dequant-fused GEMV launch (decode, batch 1..8): y = dequant(W) . x with W in raw GGUF blocks.
// Workgroups of 1024 threads (one per CU) for small launches, of 512 threads (two per CU) for large ones;
// device code in rt_gemv_device.h (every format) and rt_gemv_lean.h (the benchmark's four formats), planning in rt_gemv_plan.h.
#include "rt_gemv_lean.h"
#include "rt_gemv_plan.h"

#include <cstdio>

namespace rt {

namespace {

template <int THREADS>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void qgemv_kernel(GemvArgs a, int r2) {
    RT_DYN_LDS(uint4, lds4);
    __shared__ float red[THREADS / 64];
    const int wg = blockIdx.x;
    RT_GEMV_PICK_PROBLEM(a, wg, P);
    gemv_dispatch<false, true>(P, wg - P.tile0, P.rows_per_tile, blockIdx.y, r2 != 0, reinterpret_cast<uint32_t *>(lds4), red);
}

// The same launch for problems that are all in the benchmark's four formats: the lean code path, R rows per step (the
// gate / up pair form always takes a pair).  PAIR: the kernel contains the pair form.  WPE: waves per SIMD the register
// allocation is made for -- 4 (128 registers), or 5 (96 registers; the form without the pair form fits, with 640-thread
// workgroups two of which fill a compute unit's twenty wave slots).
template <int THREADS, int R, bool PAIR, int WPE>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void qgemv_lean_kernel(GemvArgs a) {
    RT_DYN_LDS(uint4, lds4);
    __shared__ float red[THREADS / 64];
    const int wg = blockIdx.x;
    RT_GEMV_PICK_PROBLEM(a, wg, P);
    lean_dispatch<R, PAIR>(P, wg - P.tile0, P.rows_per_tile, blockIdx.y, reinterpret_cast<uint32_t *>(lds4), red);
}

}  // namespace

// The plan of a launch as the launcher makes it: the lean path is opt-in (rt_hip_set_option), the general kernel serves
// every launch otherwise.
static bool plan_launch(GemvArgs &a, int batch, GemvPlan &pl) {
    GemvPlanHints hints;
    const int lean = path_option(RT_HIP_OPT_GEMV_LEAN);
    hints.lean = lean >= 1 ? 1 : 0;
    hints.five_waves = lean == 2 ? 1 : 0;
    return plan_qgemv(a, batch, pl, hints);
}

// Which kernel launch_qgemv would run for these problems and how it would cut the launch, as text (for reports).
bool describe_qgemv(GemvArgs &a, int batch, char *out, size_t out_bytes) {
    GemvPlan pl;
    if (!plan_launch(a, batch, pl)) return false;
    int n = pl.lean ? snprintf(out, out_bytes, "qgemv_lean_kernel<%d,1,%s,%d>", pl.threads, pl.pair ? "true" : "false", pl.threads == 640 ? 5 : 4)
                    : snprintf(out, out_bytes, "qgemv_kernel<%d>", pl.threads);
    if (n < 0 || (size_t)n >= out_bytes) return true;
    n += snprintf(out + n, out_bytes - n, " grid %dx%d lds %zu%s shares", pl.wgs, batch, pl.lds, pl.lean ? "" : (pl.r2 ? " two rows per step" : " one row per step"));
    for (int i = 0; i < a.n && (size_t)n < out_bytes; i++)
        n += snprintf(out + n, out_bytes - n, " %d%s", a.p[i].rows_per_tile, a.p[i].ksplit ? "k" : "");
    return true;
}

// One grid over all problems (grid.y = batch row).  Workgroups of a problem stage x once and deal its rows out round-robin.
hipError_t launch_qgemv(hipStream_t s, GemvArgs &a, int batch) {
    GemvPlan pl;
    if (!plan_launch(a, batch, pl)) return hipErrorInvalidValue;
    dim3 grid((unsigned)pl.wgs, (unsigned)batch);
    const size_t lds = pl.lds;
    if (lds > 64 * 1024) {
        // rows longer than 27 000 elements (the 70B-class FFN): more than the default 64 KB of dynamic LDS, granted per
        // kernel on request (the general path only; setting the attribute again is harmless, so no state is kept)
        const void *fn = pl.threads == 512 ? (const void *)qgemv_kernel<512> : (const void *)qgemv_kernel<1024>;
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGemvLdsMax);
        if (e != hipSuccess) return e;
    }
    if (pl.lean) {      // the planner gives this path one row per step
        if (pl.threads == 640) qgemv_lean_kernel<640, 1, false, 5><<<grid, 640, lds, s>>>(a);      // only planned without a pair problem
        else if (pl.threads == 512 && pl.pair) qgemv_lean_kernel<512, 1, true, 4><<<grid, 512, lds, s>>>(a);
        else if (pl.threads == 512) qgemv_lean_kernel<512, 1, false, 4><<<grid, 512, lds, s>>>(a);
        else if (pl.pair) qgemv_lean_kernel<1024, 1, true, 4><<<grid, 1024, lds, s>>>(a);
        else qgemv_lean_kernel<1024, 1, false, 4><<<grid, 1024, lds, s>>>(a);
    } else if (pl.threads == 512) qgemv_kernel<512><<<grid, 512, lds, s>>>(a, pl.r2);
    else qgemv_kernel<1024><<<grid, 1024, lds, s>>>(a, pl.r2);
    return hipGetLastError();
}

}  // namespace rt
