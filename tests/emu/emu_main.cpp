// CPU run of the persistent decode-step kernel (tests/emu/rt_mega_device.h) under AddressSanitizer.
// TEST INFRASTRUCTURE.  Every GPU thread is a fiber; see tests/emu/hip/hip_runtime.h for the execution model.
// What it checks: no out-of-bounds access to any buffer the kernel is handed, every workgroup leaves the
// kernel (no barrier time-out, no dead rendezvous), and the logits agree with the CPU oracle.
//
// usage: emu_main [n_wg [layers hidden heads ffn vocab max_pos [steps]]]
//   n_wg: number of workgroups, a multiple of 8 and >= heads (default 8; the device launches one per compute unit, 256 --
//   that many workgroups of 1024 fibers, all alive at once, need the build flags -DEMU_STACK_ARENA=262144
//   -DEMU_STACK_BYTES=65536); the model's shape defaults to 2 256 2 512 128 8, steps to 3.

#include <cstdio>
#include <cstdlib>
#include <functional>
#include <vector>

#include "rt_mega_device.h"

#include "emu_fibers.h"

// ------------------------------------------------------------------ the test
extern "C" {
size_t rt_hip_type_block_bytes(int t) { return rt::type_block_bytes(t); }
size_t rt_hip_type_block_elems(int t) { return rt::type_block_elems(t); }
// oracle (oracle/rt_oracle.c)
void *orc_llama_create(int, int, int, int, int, int, float, float, int);
int orc_llama_set_tensor(void *, int, int, int, const void *, size_t, size_t);
int orc_llama_forward(void *, const int *, int, int, float *, int);
void orc_llama_destroy(void *);
}

struct Tensor {
    int type;
    size_t rows, cols, row_bytes;
    uint8_t *data;   // exact-size heap block
};

static Tensor make_tensor(int type, uint64_t seed, uint64_t id, size_t rows, size_t cols) {
    Tensor t{ type, rows, cols, cols / rt::type_block_elems(type) * rt::type_block_bytes(type), nullptr };
    size_t nblocks = rows * (cols / rt::type_block_elems(type));
    t.data = (uint8_t *)malloc(t.row_bytes * rows);
    float lo = type == RT_GGML_Q8_0 ? 1e-4f : 1e-3f, hi = type == RT_GGML_Q8_0 ? 2e-3f : 1e-2f;
    rt_synth_blocks(type, seed, id, nblocks, lo, hi, t.data);
    return t;
}

static float *make_norm(uint64_t seed, uint64_t id, size_t n) {
    float *p = (float *)malloc(n * 4);
    rt_synth_normal_f32(seed, id, n, 1.0f, 0.01f, p);
    return p;
}

int main(int argc, char **argv) {
    const int nwg = argc > 1 ? atoi(argv[1]) : 8;
    const bool shaped = argc >= 8;
    const int L = shaped ? atoi(argv[2]) : 2, H = shaped ? atoi(argv[3]) : 256, NH = shaped ? atoi(argv[4]) : 2, HD = H / NH;
    const int F = shaped ? atoi(argv[5]) : 512, V = shaped ? atoi(argv[6]) : 128, P = shaped ? atoi(argv[7]) : 8;
    const int n_steps = argc >= 9 ? atoi(argv[8]) : 3;
    if (HD != 128 || H % 256 || F % 256 || n_steps < 1 || n_steps > P) { fprintf(stderr, "shape not served: head_dim 128, hidden and ffn multiples of 256, steps <= max_pos\n"); return 2; }
    const float eps = 1e-5f, theta = 10000.f;
    const uint64_t seed = 5;
    if (nwg % 8 || nwg < NH) { fprintf(stderr, "n_wg must be a multiple of 8 and >= %d\n", NH); return 2; }

    void *om = orc_llama_create(L, H, NH, F, V, P, eps, theta, 1);
    Tensor embd = make_tensor(RT_GGML_Q8_0, seed, 1, V, H), wout = make_tensor(RT_GGML_Q6_K, seed, 2, V, H);
    float *out_norm = make_norm(seed, 3, H);
    orc_llama_set_tensor(om, 0, -1, embd.type, embd.data, V, H);
    orc_llama_set_tensor(om, 1, -1, wout.type, wout.data, V, H);
    orc_llama_set_tensor(om, 2, -1, 0, out_norm, 1, H);

    std::vector<rt::MegaLayer> layers((size_t)L);
    uint16_t *kcache = (uint16_t *)calloc((size_t)L * P * H, 2), *vcache = (uint16_t *)calloc((size_t)L * P * H, 2);
    for (int l = 0; l < L; l++) {
        uint64_t base = 100 * (uint64_t)(l + 1);
        Tensor q = make_tensor(RT_GGML_Q4_K, seed, base + 0, H, H), k = make_tensor(RT_GGML_Q4_K, seed, base + 1, H, H);
        Tensor v = make_tensor(RT_GGML_Q6_K, seed, base + 2, H, H), o = make_tensor(RT_GGML_Q4_K, seed, base + 3, H, H);
        Tensor g = make_tensor(RT_GGML_Q4_K, seed, base + 4, F, H), u = make_tensor(RT_GGML_Q4_K, seed, base + 5, F, H);
        Tensor d = make_tensor(RT_GGML_Q6_K, seed, base + 6, H, F);
        float *an = make_norm(seed, base + 7, H), *fn = make_norm(seed, base + 8, H);
        const Tensor *ts[7] = { &q, &k, &v, &o, &g, &u, &d };
        for (int i = 0; i < 7; i++) orc_llama_set_tensor(om, 10 + i, l, ts[i]->type, ts[i]->data, ts[i]->rows, ts[i]->cols);
        orc_llama_set_tensor(om, 17, l, 0, an, 1, H);
        orc_llama_set_tensor(om, 18, l, 0, fn, 1, H);
        rt::MegaLayer &m = layers[(size_t)l];
        m.wq = q.data; m.wk = k.data; m.wv = v.data; m.wo = o.data; m.wgate = g.data; m.wup = u.data; m.wdown = d.data;
        m.rb_q = q.row_bytes; m.rb_k = k.row_bytes; m.rb_v = v.row_bytes; m.rb_o = o.row_bytes; m.rb_g = g.row_bytes; m.rb_d = d.row_bytes;
        m.t_q = q.type; m.t_k = k.type; m.t_v = v.type; m.t_o = o.type; m.t_g = g.type; m.t_d = d.type;
        m.attn_norm = an; m.ffn_norm = fn;
        m.kc = kcache + (size_t)l * P * H;
        m.vc = vcache + (size_t)l * P * H;
    }

    rt::MegaArgs A;
    memset(&A, 0, sizeof A);
    A.layers = layers.data(); A.n_layers = L; A.hidden = H; A.n_heads = NH; A.head_dim = HD; A.ffn = F; A.vocab = V; A.max_pos = P;
    A.eps = eps;
    A.embd = embd.data; A.rb_embd = embd.row_bytes; A.t_embd = embd.type;
    A.wout = wout.data; A.rb_out = wout.row_bytes; A.t_out = wout.type; A.out_norm = out_norm;
    A.x = (float *)malloc(H * 4); A.q = (float *)malloc(H * 4); A.k = (float *)malloc(H * 4); A.v = (float *)malloc(H * 4);
    A.a = (float *)malloc(H * 4); A.f = (float *)malloc(F * 4); A.logits = (float *)malloc(V * 4);
    float *inv = (float *)malloc(HD / 2 * 4);
    for (int i = 0; i < HD / 2; i++) inv[i] = (float)pow((double)theta, -2.0 * i / HD);
    A.inv_freq = inv;
    int *state = (int *)calloc(4, 4), *out_tokens = (int *)calloc((size_t)P + 1, 4);
    A.state = state; A.out_tokens = out_tokens; A.forced = nullptr;
    A.bar = (unsigned *)malloc(rt::kMegaBarBytes);
    // q / k / v share the workgroups in proportion to their bytes, as the host side of the kernel did
    {
        const double bq = (double)layers[0].rb_q * H, bk = (double)layers[0].rb_k * H, bv = (double)layers[0].rb_v * H, tot = bq + bk + bv;
        A.wg_q = (int)(nwg * bq / tot + 0.5);
        A.wg_k = (int)(nwg * bk / tot + 0.5);
        if (A.wg_q < 1) A.wg_q = 1;
        if (A.wg_k < 1) A.wg_k = 1;
        if (A.wg_q + A.wg_k > nwg - 1) { A.wg_q = nwg / 3; A.wg_k = nwg / 3; }
    }
    A.want_logits = 1; A.do_advance = 1;
    const size_t lds = rt::mega_lds_bytes(H, F, HD, P);
    // What the kernel assumes and no launch checked: every GEMV problem's staged x fits the launch's LDS, and every matrix is
    // below 4 GB (its row offsets are 32-bit).
    {
        struct { const char *name; int type; size_t K, N, rb; } probs[] = {
            { "q", layers[0].t_q, (size_t)H, (size_t)H, layers[0].rb_q }, { "k", layers[0].t_k, (size_t)H, (size_t)H, layers[0].rb_k },
            { "v", layers[0].t_v, (size_t)H, (size_t)H, layers[0].rb_v }, { "o", layers[0].t_o, (size_t)H, (size_t)H, layers[0].rb_o },
            { "gate/up", layers[0].t_g, (size_t)H, (size_t)F, layers[0].rb_g }, { "down", layers[0].t_d, (size_t)F, (size_t)H, layers[0].rb_d },
            { "output", wout.type, (size_t)H, (size_t)V, wout.row_bytes } };
        for (const auto &p : probs) {
            if (rt::gemv_lds_bytes(p.type, p.K) > lds) { fprintf(stderr, "%s: x of %zu elements needs %zu bytes of LDS, the launch has %zu\n", p.name, p.K, rt::gemv_lds_bytes(p.type, p.K), lds); return 1; }
            if ((double)p.N * (double)p.rb >= 4294967296.0) { fprintf(stderr, "%s: %zu rows of %zu bytes exceed 32-bit row offsets\n", p.name, p.N, p.rb); return 1; }
        }
        printf("%d workgroups (q %d, k %d, v %d), launch LDS %zu bytes\n", nwg, A.wg_q, A.wg_k, nwg - A.wg_q - A.wg_k, lds);
    }

    std::vector<int> toks((size_t)n_steps);
    for (int i = 0; i < n_steps; i++) toks[(size_t)i] = (i == 0 ? 3 : i == 1 ? 77 : 100 + 37 * i) % V;
    std::vector<float> want((size_t)n_steps * V);
    orc_llama_forward(om, toks.data(), n_steps, 0, want.data(), 0);
    state[0] = 0; state[1] = toks[0]; state[3] = 0;
    int rc = 0;
    for (int p = 0; p < n_steps; p++) {
        state[1] = toks[(size_t)p];   // teacher forcing
        memset(A.bar, 0, rt::kMegaBarBytes);
        bool ok = emu::launch((unsigned)nwg, rt::kMegaThreads, lds, [&] { rt::llama_step_kernel(A); });
        unsigned flag = A.bar[rt::kMegaErrWord];
        float err = 0.f, scale = 0.f;
        int amax = 0;
        for (int i = 0; i < V; i++) {
            err = fmaxf(err, fabsf(A.logits[i] - want[(size_t)p * V + i]));
            scale = fmaxf(scale, fabsf(want[(size_t)p * V + i]));
            if (want[(size_t)p * V + i] > want[(size_t)p * V + amax]) amax = i;
        }
        printf("step %d: launch %s, barrier flag %u, pos -> %d, pick %d (oracle %d), max |delta logit| %.3e (scale %.3e), %ld fiber switches\n",
               p, ok ? "completed" : "STALLED", flag, state[0], state[2], amax, err, scale, emu::g_switches);
        // a long run hunts for faults and stalls: a position where the tiny model is ill conditioned is reported, not fatal
        const bool numbers_ok = err <= (n_steps > 3 ? 2e-2f : 1e-3f) * scale + 1e-3f;
        if (!numbers_ok) printf("step %d: logits outside the bound\n", p);
        if (!ok || flag || (!numbers_ok && n_steps <= 3) || !(err <= 0.2f * scale) || state[0] != p + 1) rc = 1;
        if (rc) break;
    }
    printf(rc ? "EMU FAIL\n" : "EMU OK\n");
    return rc;
}
