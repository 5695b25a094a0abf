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
    int threads = 0;      // workgroup size: 512 or 1024 (640: the lean path's five-waves-per-SIMD form)
    bool pair = false;    // some problem has the gate / up pair (SwiGLU) epilogue
    int r2 = 0;           // two rows per wave step (else one)
    int wgs = 0;          // grid.x
    size_t lds = 0;       // launch-sized LDS
    bool lean = false;    // every problem is in one of the benchmark's four formats and takes its residual in place
};

// What a test may fix instead of leaving it to the planner (-1: the planner decides), to walk at a small scale the
// code paths that large launches take.
struct GemvPlanHints {
    int threads = -1, r2 = -1, budget = -1;
    int lean = -1;        // 0: never the lean path; 1 or -1: wherever every problem of the launch qualifies
    int five_waves = 0;   // 1: lean launches without a pair problem use 640-thread workgroups, two per compute unit
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
    bool lean = hints.lean != 0 && lds <= 64 * 1024;
    for (int i = 0; i < a.n; i++) {
        const GemvProb &p = a.p[i];
        lean = lean && (p.res == nullptr || p.res == p.y) &&
               (p.type == RT_GGML_Q4_K || p.type == RT_GGML_Q6_K || p.type == RT_GGML_Q8_0 || p.type == RT_GGML_Q4_0);
    }
    bool pair = false;
    for (int i = 0; i < a.n; i++) pair = pair || a.p[i].epi == kEpiSwiglu;
    // 16 resident waves per CU over 256 CUs, as one or two workgroups; or 20 as two workgroups of ten
    const bool five = lean && !pair && hints.five_waves == 1;
    const int threads = hints.threads > 0 ? hints.threads : (five ? 640 : (total_bytes >= RT_GEMV_BIG_BYTES ? 512 : 1024));
    const int waves = threads / 64;
    int budget = hints.budget > 0 ? hints.budget : 256 * (threads == 1024 ? 1 : 2) / batch;
    if (budget < a.n) budget = a.n;
    // General path: two rows per wave step once every wave has at least three steps of work, else one (two rows share one
    // read of x from LDS).  Lean path: one row per step at every size -- measured on the layer workload and on single
    // matrices of each format and row length, one row was as fast or faster (28.6 against 31.1 us for the layer): the finer
    // steps even out the end of the launch, and its x reads are cheap next to the rest.
    const int r2 = hints.r2 >= 0 ? hints.r2 : (lean ? 0 : (total_rows >= (size_t)3 * 2 * (size_t)budget * waves ? 1 : 0));

    // A launch ends when its slowest wave does, and a wave streams at 1/4096 of the device's rate: a 9 KB row of the 7B
    // down-projection is 6 us of a wave's time, so "3 or 4 rows per wave" is a 14 % longer launch.  Two remedies.
    // (1) Lean path, rows of more than one pass, one row per step, plain store: the unit of work becomes one pass of one row
    //     (ksplit); a workgroup owns whole rows, deals their passes out to its waves and sums them through LDS at its end.
    // (2) The workgroups are shared out by what each problem's busiest wave would stream, rounding included, not by bytes:
    //     start from the shares by bytes, then move workgroups to the problem whose waves stream most for as long as that
    //     lowers the maximum.
    struct Cost {
        int n_iter, rows_per_group, max_wg;
        bool split, dual;
        size_t part_bytes_per_row;
    } cs[kMaxGemvProbs];
    for (int i = 0; i < a.n; i++) {
        GemvProb &p = a.p[i];
        Cost &c = cs[i];
        const bool kq = p.type == RT_GGML_Q2_K || p.type == RT_GGML_Q3_K || p.type == RT_GGML_Q4_K || p.type == RT_GGML_Q5_K || p.type == RT_GGML_Q6_K;
        const int units = gemv_float_weights(p.type) ? p.K / (p.type == RT_GGML_F16 ? 8 : 4) : (kq ? p.K / 64 : p.K / 32);
        c.n_iter = (units + 63) / 64;
        c.dual = p.epi == kEpiSwiglu;
        c.rows_per_group = c.dual ? 1 : (r2 ? 2 : 1);
        c.split = lean && !c.dual && r2 == 0 && c.n_iter > 1;
        c.part_bytes_per_row = (size_t)c.n_iter * sizeof(float);
        const int groups = (p.N + c.rows_per_group - 1) / c.rows_per_group;
        c.max_wg = c.split ? std::max(1, std::min(p.N, (int)((size_t)p.N * c.n_iter / waves))) : std::max(1, (groups + waves - 1) / waves);
        p.ksplit = 0;
    }
    // bytes the busiest wave of problem i streams when the problem has n workgroups
    auto wave_bytes = [&](int i, int n) -> double {
        const GemvProb &p = a.p[i];
        const Cost &c = cs[i];
        if (c.split) {
            const long rows_wg = (p.N + n - 1) / n, items = rows_wg * c.n_iter;
            return (double)((items + waves - 1) / waves) * (double)p.row_bytes / c.n_iter;
        }
        const long groups = (p.N + c.rows_per_group - 1) / c.rows_per_group;
        const long steps = (groups + (long)waves * n - 1) / ((long)waves * n);
        return (double)steps * c.rows_per_group * (double)p.row_bytes * (c.dual ? 2.0 : 1.0);
    };
    int share[kMaxGemvProbs];
    int used = 0;
    for (int i = 0; i < a.n; i++) {
        const GemvProb &p = a.p[i];
        const double bytes = (double)p.N * (double)p.row_bytes * (p.epi == kEpiSwiglu ? 2.0 : 1.0);
        int n = (int)(budget * (bytes / total_bytes) + 0.5);
        if (n > cs[i].max_wg) n = cs[i].max_wg;
        if (n < 1) n = 1;
        share[i] = n;
        used += n;
    }
    for (int round = 0; round < 4 * budget && a.n > 1; round++) {
        int hi = 0;
        double worst = 0;
        for (int i = 0; i < a.n; i++) {
            const double c = wave_bytes(i, share[i]);
            if (c > worst) { worst = c; hi = i; }
        }
        // the fewest extra workgroups that shorten the busiest problem
        int add = 0;
        for (int k = 1; k <= 64 && share[hi] + k <= cs[hi].max_wg; k++)
            if (wave_bytes(hi, share[hi] + k) < worst) { add = k; break; }
        if (add == 0) break;
        int trial[kMaxGemvProbs];
        for (int i = 0; i < a.n; i++) trial[i] = share[i];
        trial[hi] += add;
        int need = add - std::max(0, budget - used);          // workgroups the budget has not handed out yet come first
        if (need < 0) need = 0;
        bool ok = true;
        while (need > 0 && ok) {
            int donor = -1;
            double best = worst;
            for (int j = 0; j < a.n; j++) {
                if (j == hi || trial[j] <= 1) continue;
                const double c = wave_bytes(j, trial[j] - 1);
                if (c < best) { best = c; donor = j; }
            }
            if (donor < 0) ok = false;
            else { trial[donor]--; need--; }
        }
        if (!ok) break;
        double now = 0;
        int sum = 0;
        for (int i = 0; i < a.n; i++) { now = std::max(now, wave_bytes(i, trial[i])); sum += trial[i]; }
        if (!(now < worst)) break;
        for (int i = 0; i < a.n; i++) share[i] = trial[i];
        used = sum;
    }
    int wgs = 0;
    size_t lds_all = lds;
    for (int i = 0; i < a.n; i++) {
        GemvProb &p = a.p[i];
        p.tile0 = wgs;
        p.rows_per_tile = share[i];
        wgs += share[i];
        if (cs[i].split) {
            // partial sums of the workgroup's rows sit behind x in LDS; a problem whose rows per workgroup would not fit keeps whole rows
            const size_t rows_wg = ((size_t)p.N + share[i] - 1) / share[i];
            const size_t need = ((gemv_lds_bytes(p.type, (size_t)p.K) + 15) & ~(size_t)15) + rows_wg * cs[i].part_bytes_per_row;
            if (need <= 64 * 1024) { p.ksplit = 1; lds_all = std::max(lds_all, need); }
        }
    }
    lds = lds_all;
    pl.threads = threads; pl.r2 = r2; pl.wgs = wgs; pl.lds = lds; pl.lean = lean; pl.pair = pair;
    return true;
}

}  // namespace rt
