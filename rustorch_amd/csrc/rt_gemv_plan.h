// Host-side planning of a grouped GEMV launch: workgroup size, rows per wave step, and each problem's share of the
// workgroups.  Kept apart from the launcher so that a CPU build of the device code walks exactly the grids the GPU runs.
#pragma once

#include "rt_internal.h"

#include <algorithm>

namespace rt {

// Launches that stream less than this many weight bytes use 1024-thread workgroups: with few rows per wave
// the start-up (one staging of x per workgroup) dominates and fewer, larger workgroups pay it less often.
// Larger launches run faster with two 512-thread workgroups per CU, which do not stall on each other's barriers.
#ifndef RT_GEMV_BIG_BYTES
#define RT_GEMV_BIG_BYTES (64.0 * 1024 * 1024)
#endif

struct GemvPlan {
    int threads = 0;      // workgroup size: 512 or 1024
    int r2 = 0;           // two rows per wave step (else one)
    int wgs = 0;          // grid.x
    size_t lds = 0;       // launch-sized LDS
    bool lean = false;    // every problem is in one of the benchmark's four formats and takes its residual in place
};

// What a test may fix instead of leaving it to the planner (-1: the planner decides), to walk at a small scale the
// code paths that large launches take.
struct GemvPlanHints {
    int threads = -1, r2 = -1, budget = -1;
};

// Gives every problem a share of the workgroups in proportion to its weight bytes (tile0 = first workgroup,
// rows_per_tile = number of workgroups of the problem).  Returns false for arguments no launch accepts.
inline bool plan_qgemv(GemvArgs &a, int batch, GemvPlan &pl, const GemvPlanHints &hints = GemvPlanHints()) {
    if (a.n <= 0 || a.n > kMaxGemvProbs || batch <= 0) return false;
    double total_bytes = 0;
    size_t lds = 0, total_rows = 0;
    for (int i = 0; i < a.n; i++) {
        if ((double)a.p[i].N * (double)a.p[i].row_bytes >= 4294967296.0) return false;   // row offsets are 32-bit
        if ((a.p[i].type == RT_GGML_Q5_K || a.p[i].type == RT_GGML_Q3_K || a.p[i].type == RT_GGML_Q2_K) && a.p[i].epi == kEpiSwiglu)
            return false;   // no pair form for these
        total_bytes += (double)a.p[i].N * (double)a.p[i].row_bytes * (a.p[i].epi == kEpiSwiglu ? 2.0 : 1.0);
        total_rows += (size_t)a.p[i].N;
        lds = std::max(lds, gemv_lds_bytes(a.p[i].type, (size_t)a.p[i].K));
    }
    if (total_bytes <= 0) return false;
    if (lds > kGemvLdsMax) return false;    // x of the longest row must fit the workgroup's LDS
    bool lean = lds <= 64 * 1024;
    for (int i = 0; i < a.n; i++) {
        const GemvProb &p = a.p[i];
        lean = lean && (p.res == nullptr || p.res == p.y) &&
               (p.type == RT_GGML_Q4_K || p.type == RT_GGML_Q6_K || p.type == RT_GGML_Q8_0 || p.type == RT_GGML_Q4_0);
    }
    // 16 resident waves per CU over 256 CUs, as one or two workgroups
    const int threads = hints.threads > 0 ? hints.threads : (total_bytes >= RT_GEMV_BIG_BYTES ? 512 : 1024);
    const int waves = threads / 64;
    int budget = hints.budget > 0 ? hints.budget : 256 * (1024 / threads) / batch;
    if (budget < a.n) budget = a.n;
    // General path: two rows per wave step once every wave has at least three steps of work, else one (two rows share one
    // read of x from LDS).  Lean path: one row per step at every size -- measured on the layer workload and on single
    // matrices of each format and row length, one row was as fast or faster (28.6 against 31.1 us for the layer): the finer
    // steps even out the end of the launch, and its x reads are cheap next to the rest.
    const int r2 = hints.r2 >= 0 ? hints.r2 : (lean ? 0 : (total_rows >= (size_t)3 * 2 * (size_t)budget * waves ? 1 : 0));
    int wgs = 0;
    for (int i = 0; i < a.n; i++) {
        const GemvProb &p = a.p[i];
        double bytes = (double)p.N * (double)p.row_bytes * (p.epi == kEpiSwiglu ? 2.0 : 1.0);
        int n = (int)(budget * (bytes / total_bytes) + 0.5);
        int rows_per_group = (p.epi == kEpiSwiglu) ? 1 : (r2 ? 2 : 1);
        int max_useful = ((p.N + rows_per_group - 1) / rows_per_group + waves - 1) / waves;
        if (n > max_useful) n = max_useful;
        if (n < 1) n = 1;
        a.p[i].tile0 = wgs;
        a.p[i].rows_per_tile = n;
        wgs += n;
    }
    pl.threads = threads; pl.r2 = r2; pl.wgs = wgs; pl.lds = lds; pl.lean = lean;
    return true;
}

}  // namespace rt
