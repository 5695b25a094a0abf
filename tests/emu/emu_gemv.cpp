// CPU run of the decode GEMV's device code -- the general path (rustorch_amd/csrc/rt_gemv_device.h) and the lean path of the
// benchmark's formats (rt_gemv_lean.h) -- under AddressSanitizer, on the grids the launcher's own planner lays out.
// TEST INFRASTRUCTURE.  Every GPU thread is a fiber; see tests/emu/hip/hip_runtime.h for the execution model.
// What it checks, per case: no access outside the weight blocks (an exact-size heap block plus the 64 bytes of slack an
// upload adds), x, y or the launch's LDS; the lean path's result equals the general path's bit for bit; both sit within the
// held tolerance of the f64 dot products of the CPU oracle.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "rt_gemv_lean.h"
#include "rt_gemv_plan.h"

#include "emu_fibers.h"

extern "C" {
size_t rt_hip_type_block_bytes(int t) { return rt::type_block_bytes(t); }
size_t rt_hip_type_block_elems(int t) { return rt::type_block_elems(t); }
int orc_qgemv_f64(int type, const void *raw, size_t N, size_t K, const float *x, size_t M, double *y, double *wnorm, int nthreads);
}

namespace {

struct Weights {
    int type;
    size_t N, K, row_bytes;
    uint8_t *data;
};
Weights make_weights(int type, uint64_t id, size_t N, size_t K) {
    Weights w{ type, N, K, K / rt::type_block_elems(type) * rt::type_block_bytes(type), nullptr };
    w.data = (uint8_t *)malloc(w.row_bytes * N + 64);      // the slack rt_hip_qweight_upload adds for trailing 16-byte loads
    memset(w.data + w.row_bytes * N, 0, 64);
    const bool q8 = type == RT_GGML_Q8_0 || type == RT_GGML_Q8_1;
    const float lo = q8 ? 1e-4f : 1e-3f, hi = q8 ? 2e-3f : 1e-2f;
    rt_synth_blocks(type, 11, id, N * (K / rt::type_block_elems(type)), lo, hi, w.data);
    return w;
}

// the ready-made activation form, written on the host as the quantizing kernels write it (rt_internal.h)
std::vector<uint8_t> quantize_host(const float *x, size_t K) {
    std::vector<uint8_t> xq(rt::xq_stride(K), 0);
    int8_t *qh = (int8_t *)xq.data();
    uint8_t *ql = xq.data() + K;
    float *s = (float *)(xq.data() + 2 * K), *bs = s + K / 32;
    for (size_t b = 0; b < K / 32; b++) {
        float amax = 0.f;
        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(x[32 * b + i]));
        const float inv = amax > 0.f ? 16383.0f / amax : 0.f;
        s[b] = amax / 16383.0f;
        int sum[2] = { 0, 0 };
        for (int i = 0; i < 32; i++) {
            int q = (int)nearbyintf(x[32 * b + i] * inv);
            q = q > 16383 ? 16383 : (q < -16383 ? -16383 : q);
            qh[32 * b + i] = (int8_t)(q >> 7);
            ql[32 * b + i] = (uint8_t)(q & 127);
            sum[i >> 4] += q;
        }
        bs[2 * b] = s[b] * (float)sum[0];
        bs[2 * b + 1] = s[b] * (float)sum[1];
    }
    return xq;
}

struct Case {
    const char *name;
    int type;
    size_t N, K;
    int stage, epi;      // rt::kStage*, rt::kEpi*
    bool residual;
    int threads, r2, budget, batch;
    bool lean = true;    // the planner sends the case down the lean path too (else: the general path alone, against the oracle)
};

int run_case(const Case &c) {
    using namespace rt;
    Weights w = make_weights(c.type, 1, c.N, c.K), w2 = make_weights(c.type, 2, c.N, c.K);
    std::vector<float> x(c.K * (size_t)c.batch), gamma(c.K), res(c.N * (size_t)c.batch);
    rt_synth_normal_f32(11, 3, x.size(), 0.f, 1.f, x.data());
    rt_synth_normal_f32(11, 4, c.K, 1.f, 0.01f, gamma.data());
    rt_synth_normal_f32(11, 5, res.size(), 0.f, 1.f, res.data());
    // exact-size heap copies of what the kernel is handed
    float *xd = (float *)malloc(x.size() * 4);
    memcpy(xd, x.data(), x.size() * 4);
    std::vector<uint8_t> xqv;
    for (int m = 0; m < c.batch; m++) {
        std::vector<uint8_t> one = quantize_host(x.data() + c.K * (size_t)m, c.K);
        xqv.insert(xqv.end(), one.begin(), one.end());
    }
    uint8_t *xqd = (uint8_t *)malloc(xqv.size());
    memcpy(xqd, xqv.data(), xqv.size());
    float *gd = (float *)malloc(c.K * 4);
    memcpy(gd, gamma.data(), c.K * 4);

    // the vector the weights meet, in f32, for the oracle
    std::vector<float> xeff(x);
    if (c.stage == kStageRms) {
        for (int m = 0; m < c.batch; m++) {
            float *xr = xeff.data() + c.K * (size_t)m;
            float acc = 0.f;
            for (size_t i = 0; i < c.K; i++) acc += xr[i] * xr[i];
            const float rms = sqrtf(acc / (float)c.K + 1e-5f);
            for (size_t i = 0; i < c.K; i++) xr[i] = gamma[i] * (xr[i] / rms);
        }
    }
    std::vector<double> y64(c.N * (size_t)c.batch), y64b(c.N * (size_t)c.batch), wn(c.N), wn2(c.N);
    orc_qgemv_f64(c.type, w.data, c.N, c.K, xeff.data(), (size_t)c.batch, y64.data(), wn.data(), 0);
    if (c.epi == kEpiSwiglu) orc_qgemv_f64(c.type, w2.data, c.N, c.K, xeff.data(), (size_t)c.batch, y64b.data(), wn2.data(), 0);

    bool split_used = false;
    // one launch of the case down one path (0: general, 1: lean) with the planner given `budget` workgroups
    auto run = [&](int path, int budget, float *y, int &rc, bool whole_rows = false) {
        for (size_t i = 0; i < c.N * (size_t)c.batch; i++) y[i] = c.residual ? res[i] : -12345.f;
        GemvArgs a;
        memset(&a, 0, sizeof a);
        a.n = 1;
        GemvProb &p = a.p[0];
        p.w = w.data; p.w2 = c.epi == kEpiSwiglu ? w2.data : nullptr;
        p.x = c.stage == kStageXq ? (const void *)xqd : (const void *)xd;
        p.gamma = gd; p.eps = 1e-5f; p.y = y; p.res = c.residual ? y : nullptr;
        p.row_bytes = w.row_bytes; p.type = c.type; p.N = (int)c.N; p.K = (int)c.K; p.stage = c.stage; p.epi = c.epi;
        GemvPlan pl;
        GemvPlanHints h;
        h.threads = c.threads; h.r2 = c.r2; h.budget = budget;
        if (!plan_qgemv(a, c.batch, pl, h)) { printf("%s: plan refused\n", c.name); rc = 1; return; }
        if (pl.lean != c.lean) { printf("%s: the planner %s this case down the lean path\n", c.name, pl.lean ? "sends" : "does not send"); rc = 1; return; }
        if (path == 0 || whole_rows) p.ksplit = 0;      // the general path knows whole rows only
        split_used = split_used || p.ksplit != 0;
        for (int m = 0; m < c.batch && !rc; m++) {
            static float red[16];
            bool ok = emu::launch((unsigned)pl.wgs, (unsigned)pl.threads, pl.lds, [&] {
                RT_DYN_LDS(uint4, lds4);
                uint32_t *lds = reinterpret_cast<uint32_t *>(lds4);
                const int wg = (int)blockIdx.x;
                RT_GEMV_PICK_PROBLEM(a, wg, P);
                if (path == 0) gemv_dispatch<false, true>(P, wg - P.tile0, P.rows_per_tile, m, pl.r2 != 0, lds, red);
                else if (pl.r2) lean_dispatch<2, true>(P, wg - P.tile0, P.rows_per_tile, m, lds, red);
                else if (pl.pair) lean_dispatch<1, true>(P, wg - P.tile0, P.rows_per_tile, m, lds, red);       // as the launcher: the kernel without
                else lean_dispatch<1, false>(P, wg - P.tile0, P.rows_per_tile, m, lds, red);                   // the pair form when no problem is a pair
            });
            if (!ok) { printf("%s: path %d stalled\n", c.name, path); rc = 1; }
        }
        // against the f64 products
        for (int m = 0; m < c.batch && !rc; m++) {
            double xn = 0;
            for (size_t i = 0; i < c.K; i++) xn += (double)xeff[c.K * m + i] * xeff[c.K * m + i];
            xn = sqrt(xn);
            double worst = 0;
            for (size_t n = 0; n < c.N; n++) {
                const size_t o = c.N * (size_t)m + n;
                double want = y64[o], yard = wn[n] * xn;
                if (c.epi == kEpiSwiglu) {
                    const double g = y64[o], u = y64b[o];
                    want = u * (g / (1.0 + exp(-g)));
                    yard = (wn[n] * fabs(u) + wn2[n] * fabs(g) * 1.1 + wn[n] * wn2[n] * xn * 1e-3) * xn + 1e-30;   // first-order error propagation
                } else if (c.residual) want += (double)res[o];
                worst = fmax(worst, fabs((double)y[o] - want) / yard);
            }
            if (!(worst <= 2e-5)) { printf("%s: path %d row %d: max |delta| / (|w| |x|) = %.3e\n", c.name, path, m, worst); rc = 1; }
        }
    };
    const size_t n_out = c.N * (size_t)c.batch;
    float *out[3] = { (float *)malloc(n_out * 4), (float *)malloc(n_out * 4), (float *)malloc(n_out * 4) };
    int rc = 0;
    run(0, c.budget, out[0], rc);
    if (c.lean && !rc) {
        run(1, c.budget, out[1], rc);
        if (!rc) run(1, c.budget + 2, out[2], rc);      // the same rows cut into another number of workgroups
        if (!rc && memcmp(out[1], out[2], n_out * 4) != 0) { printf("%s: the lean result depends on how the launch is cut\n", c.name); rc = 1; }
        // a launch too tight on LDS to deal passes out keeps whole rows per wave: the same bits all the same
        if (!rc && split_used) {
            run(1, c.budget, out[2], rc, true);
            if (!rc && memcmp(out[1], out[2], n_out * 4) != 0) { printf("%s: whole rows and dealt-out passes give different bits\n", c.name); rc = 1; }
        }
        // rows of one pass: the general path's bits; rows of several: pass sums added in order, same bound
        if (!rc && !split_used && memcmp(out[0], out[1], n_out * 4) != 0) {
            size_t bad = 0;
            for (size_t i = 0; i < n_out; i++) bad += out[0][i] != out[1][i];
            printf("%s: lean and general results differ in %zu of %zu elements\n", c.name, bad, n_out);
            rc = 1;
        }
    }
    printf("%-50s %s%s\n", c.name, rc ? "FAIL" : "ok", split_used ? "  (passes dealt out)" : "");
    fflush(stdout);
    free(out[0]); free(out[1]); free(out[2]); free(xd); free(xqd); free(gd); free(w.data); free(w2.data);
    return rc;
}

// Several problems in one launch, as the decode step and the benchmark's layer issue them: every problem's result is, bit
// for bit, what a launch of that problem alone gives, and within the held tolerance of the oracle's f64 products.
struct GroupSpec { int type; size_t N, K; };
int run_group(const char *name, const std::vector<GroupSpec> &specs, int budget) {
    using namespace rt;
    const size_t n = specs.size();
    std::vector<Weights> ws;
    std::vector<float *> xs, ys, singles;
    for (size_t i = 0; i < n; i++) {
        ws.push_back(make_weights(specs[i].type, 20 + i, specs[i].N, specs[i].K));
        float *x = (float *)malloc(specs[i].K * 4);
        rt_synth_normal_f32(11, 40 + i, specs[i].K, 0.f, 1.f, x);
        xs.push_back(x);
        ys.push_back((float *)malloc(specs[i].N * 4));
        singles.push_back((float *)malloc(specs[i].N * 4));
    }
    int rc = 0;
    auto launch = [&](size_t first, size_t count, std::vector<float *> &out, int wgs_budget) {
        GemvArgs a;
        memset(&a, 0, sizeof a);
        a.n = (int)count;
        for (size_t i = 0; i < count; i++) {
            GemvProb &p = a.p[i];
            const Weights &w = ws[first + i];
            p.w = w.data; p.x = xs[first + i]; p.y = out[first + i]; p.eps = 1e-5f;
            p.row_bytes = w.row_bytes; p.type = w.type; p.N = (int)w.N; p.K = (int)w.K; p.stage = kStageF32; p.epi = kEpiStore;
            for (size_t r = 0; r < w.N; r++) out[first + i][r] = -12345.f;
        }
        GemvPlan pl;
        GemvPlanHints h;
        h.budget = wgs_budget;
        if (!plan_qgemv(a, 1, pl, h) || !pl.lean) { printf("%s: plan refused or not lean\n", name); rc = 1; return; }
        static float red[16];
        bool ok = emu::launch((unsigned)pl.wgs, (unsigned)pl.threads, pl.lds, [&] {
            RT_DYN_LDS(uint4, lds4);
            uint32_t *lds = reinterpret_cast<uint32_t *>(lds4);
            const int wg = (int)blockIdx.x;
            RT_GEMV_PICK_PROBLEM(a, wg, P);
            if (pl.r2) lean_dispatch<2, true>(P, wg - P.tile0, P.rows_per_tile, 0, lds, red);
            else lean_dispatch<1, false>(P, wg - P.tile0, P.rows_per_tile, 0, lds, red);
        });
        if (!ok) { printf("%s: stalled\n", name); rc = 1; }
    };
    launch(0, n, ys, budget);
    for (size_t i = 0; i < n && !rc; i++) {
        launch(i, 1, singles, 3);
        if (rc) break;
        if (memcmp(ys[i], singles[i], specs[i].N * 4) != 0) { printf("%s: problem %zu differs from its own launch\n", name, i); rc = 1; }
        std::vector<double> y64(specs[i].N), wn(specs[i].N);
        orc_qgemv_f64(specs[i].type, ws[i].data, specs[i].N, specs[i].K, xs[i], 1, y64.data(), wn.data(), 0);
        double xn = 0, worst = 0;
        for (size_t k = 0; k < specs[i].K; k++) xn += (double)xs[i][k] * xs[i][k];
        xn = sqrt(xn);
        for (size_t r = 0; r < specs[i].N; r++) worst = fmax(worst, fabs((double)ys[i][r] - y64[r]) / (wn[r] * xn));
        if (!(worst <= 2e-5)) { printf("%s: problem %zu: max |delta| / (|w| |x|) = %.3e\n", name, i, worst); rc = 1; }
    }
    printf("%-50s %s\n", name, rc ? "FAIL" : "ok");
    fflush(stdout);
    for (size_t i = 0; i < n; i++) { free(ws[i].data); free(xs[i]); free(ys[i]); free(singles[i]); }
    return rc;
}

}  // namespace

// The planner on the benchmark's own launches (no device code runs): shares are positive, contiguous and within the
// budget, and the busiest wave of the layer launch streams within 5 % of the mean (31.7 KB), rounding included.
int check_planner() {
    using namespace rt;
    struct M { int type, N, K; size_t rb; };
    const M layer[7] = { { RT_GGML_Q4_K, 4096, 4096, 2304 }, { RT_GGML_Q4_K, 4096, 4096, 2304 }, { RT_GGML_Q6_K, 4096, 4096, 3360 }, { RT_GGML_Q4_K, 4096, 4096, 2304 },
                         { RT_GGML_Q4_K, 11008, 4096, 2304 }, { RT_GGML_Q4_K, 11008, 4096, 2304 }, { RT_GGML_Q6_K, 4096, 11008, 9030 } };
    int rc = 0;
    for (int which = 0; which < 3; which++) {      // the layer in one launch; q, k, v of the decode step; the down-projection with its residual
        GemvArgs a;
        memset(&a, 0, sizeof a);
        static float dummy;
        const int first = which == 0 ? 0 : (which == 1 ? 0 : 6), n = which == 0 ? 7 : (which == 1 ? 3 : 1);
        a.n = n;
        double bytes = 0;
        for (int i = 0; i < n; i++) {
            const M &mm = layer[first + i];
            GemvProb &p = a.p[i];
            p.type = mm.type; p.N = mm.N; p.K = mm.K; p.row_bytes = mm.rb; p.y = &dummy; p.res = which == 2 ? &dummy : nullptr;
            bytes += (double)mm.N * mm.rb;
        }
        GemvPlan pl;
        if (!plan_qgemv(a, 1, pl)) { printf("planner: launch %d refused\n", which); return 1; }
        const int waves = pl.threads / 64, budget = 256 * (1024 / pl.threads);
        int next = 0;
        double busiest = 0;
        printf("planner launch %d: %d threads, lean %d, lds %zu, shares", which, pl.threads, (int)pl.lean, pl.lds);
        for (int i = 0; i < n; i++) {
            const GemvProb &p = a.p[i];
            printf(" %d%s", p.rows_per_tile, p.ksplit ? "*" : "");
            if (p.tile0 != next || p.rows_per_tile < 1) rc = 1;
            next += p.rows_per_tile;
            const int n_iter = (p.K / 64 + 63) / 64;
            double wb;
            if (p.ksplit) {
                const long rows_wg = (p.N + p.rows_per_tile - 1) / p.rows_per_tile;
                wb = (double)((rows_wg * n_iter + waves - 1) / waves) * p.row_bytes / n_iter;
                if (rows_wg * n_iter * 4 + ((gemv_lds_bytes(p.type, (size_t)p.K) + 15) & ~(size_t)15) > pl.lds) rc = 1;
            } else wb = (double)((p.N + (long)waves * p.rows_per_tile - 1) / ((long)waves * p.rows_per_tile)) * p.row_bytes;
            busiest = wb > busiest ? wb : busiest;
        }
        const double mean = bytes / ((double)next * waves);
        printf("  (* passes dealt out); busiest wave %.1f KB, mean %.1f KB\n", busiest / 1024, mean / 1024);
        if (next != pl.wgs || next > budget || !pl.lean) rc = 1;
        if (which == 0 && busiest > 1.05 * mean) rc = 1;
    }
    if (rc) printf("planner: FAIL\n");
    return rc;
}

int main(int argc, char **argv) {
    using namespace rt;
    const int Q4K = RT_GGML_Q4_K, Q6K = RT_GGML_Q6_K, Q80 = RT_GGML_Q8_0, Q40 = RT_GGML_Q4_0, Q81 = RT_GGML_Q8_1;
    // threads / r2 / budget: -1 leaves the choice to the planner (1024 threads, one row per step at these sizes)
    const Case cases[] = {
        { "q4k 37x256 f32", Q4K, 37, 256, kStageF32, kEpiStore, false, 512, 0, 2, 1 },
        { "q4k 20x4096 xq, two rows per step", Q4K, 20, 4096, kStageXq, kEpiStore, false, 512, 1, 1, 1 },
        { "q4k 21x4096 rms, residual, two rows", Q4K, 21, 4096, kStageRms, kEpiStore, true, 512, 1, 1, 1 },
        { "q4k 9x8192 xq (two whole passes)", Q4K, 9, 8192, kStageXq, kEpiStore, false, 512, 1, 1, 1 },
        { "q4k 12x4096 rms, gate/up pair", Q4K, 12, 4096, kStageRms, kEpiSwiglu, false, 512, 0, 1, 1 },
        { "q4k 5x768 f32 (planner's own choice)", Q4K, 5, 768, kStageF32, kEpiStore, false, -1, -1, 3, 2 },
        { "q6k 9x11008 xq (ragged third pass)", Q6K, 9, 11008, kStageXq, kEpiStore, false, 512, 1, 1, 1 },
        { "q6k 7x11008 f32, residual, one row", Q6K, 7, 11008, kStageF32, kEpiStore, true, 512, 0, 1, 1 },
        { "q6k 18x4096 rms, two rows", Q6K, 18, 4096, kStageRms, kEpiStore, false, 512, 1, 2, 1 },
        { "q6k 5x768 xq, gate/up pair", Q6K, 5, 768, kStageXq, kEpiSwiglu, false, 512, 0, 1, 1 },
        { "q8_0 5x96 f32", Q80, 5, 96, kStageF32, kEpiStore, false, -1, -1, 2, 1 },
        { "q8_0 19x4096 xq (two whole passes), two rows", Q80, 19, 4096, kStageXq, kEpiStore, false, 512, 1, 1, 1 },
        { "q4_0 5x96 rms", Q40, 5, 96, kStageRms, kEpiStore, false, -1, -1, 2, 1 },
        { "q4_0 11x11008 xq (ragged sixth pass), two rows", Q40, 11, 11008, kStageXq, kEpiStore, true, 512, 1, 1, 1 },
        { "q4_0 6x2048 f32, gate/up pair", Q40, 6, 2048, kStageF32, kEpiSwiglu, false, 512, 0, 1, 1 },
        // one row per step and rows of several passes: the passes of a row go to different waves and meet in LDS
        { "q6k 21x11008 xq, one row per step", Q6K, 21, 11008, kStageXq, kEpiStore, false, 512, 0, 2, 1 },
        { "q4k 13x8192 rms, one row per step, residual", Q4K, 13, 8192, kStageRms, kEpiStore, true, 512, 0, 3, 1 },
        { "q8_0 9x4096 f32, one row per step, two vectors", Q80, 9, 4096, kStageF32, kEpiStore, false, 512, 0, 1, 2 },
        { "q4_0 5x11008 xq, planner's own choice", Q40, 5, 11008, kStageXq, kEpiStore, false, -1, -1, 2, 1 },
        // 640-thread workgroups (ten waves: the five-waves-per-SIMD form of the lean path)
        { "q4k 23x4096 xq, 640 threads", Q4K, 23, 4096, kStageXq, kEpiStore, false, 640, 0, 2, 1 },
        { "q6k 21x11008 rms, 640 threads, residual (row longer than the staged trips)", Q6K, 21, 11008, kStageRms, kEpiStore, true, 640, 0, 2, 1 },
        { "q4k 11x11008 xq, 640 threads", Q4K, 11, 11008, kStageXq, kEpiStore, false, 640, 0, 1, 1 },
        { "q8_0 5x96 f32, 640 threads", Q80, 5, 96, kStageF32, kEpiStore, false, 640, 0, 1, 2 },
        { "q4_0 9x11008 f32, 640 threads", Q40, 9, 11008, kStageF32, kEpiStore, false, 640, 0, 2, 1 },
        // formats of the general path alone
        { "q8_1 5x96 f32", Q81, 5, 96, kStageF32, kEpiStore, false, -1, -1, 2, 1, false },
        { "q8_1 13x4096 rms, two rows, residual", Q81, 13, 4096, kStageRms, kEpiStore, true, 512, 1, 1, 1, false },
        { "q8_1 7x11008 xq (ragged), gate/up pair", Q81, 7, 11008, kStageXq, kEpiSwiglu, false, 512, 0, 1, 1, false },
    };
    int rc = check_planner();
    const int only = argc > 1 ? atoi(argv[1]) : -1;
    for (size_t i = 0; i < sizeof cases / sizeof cases[0]; i++)
        if (only < 0 || only == (int)i) rc |= run_case(cases[i]);
    if (only < 0) {
        rc |= run_group("five problems of mixed formats and row lengths", { { Q4K, 40, 4096 }, { Q4K, 12, 4096 }, { Q6K, 33, 4096 }, { Q6K, 9, 11008 }, { Q80, 10, 4096 } }, 9);
        rc |= run_group("a layer's seven projections, rows / 128", { { Q4K, 32, 4096 }, { Q4K, 32, 4096 }, { Q6K, 32, 4096 }, { Q4K, 32, 4096 }, { Q4K, 86, 4096 }, { Q4K, 86, 4096 }, { Q6K, 32, 11008 } }, 12);
        rc |= run_group("more problems than the budget has workgroups", { { Q40, 5, 96 }, { Q4K, 3, 256 }, { Q6K, 7, 768 }, { Q80, 4, 11008 } }, 2);
    }
    printf(rc ? "EMU FAIL\n" : "EMU OK\n");
    return rc;
}
