// CPU run of the persistent decode-step kernel (tests/emu/rt_mega_device.h) under AddressSanitizer.
// TEST INFRASTRUCTURE.  Every GPU thread is a fiber; see tests/emu/hip/hip_runtime.h for the execution model.
// What it checks: no out-of-bounds access to any buffer the kernel is handed, every workgroup leaves the
// kernel (no barrier time-out, no dead rendezvous), and the logits agree with the CPU oracle.
//
// usage: emu_main [n_wg]        (n_wg: number of workgroups, a multiple of 8 and >= n_heads; default 8)

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
    const int L = 2, H = 256, NH = 2, HD = 128, F = 512, V = 128, P = 8;
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
    A.wg_q = nwg / 3 > 0 ? nwg / 3 : 1; A.wg_k = A.wg_q;
    A.want_logits = 1; A.do_advance = 1;
    const size_t lds = rt::mega_lds_bytes(H, F, HD, P);

    const int toks[3] = { 3, 77, 100 };
    std::vector<float> want((size_t)3 * V);
    orc_llama_forward(om, toks, 3, 0, want.data(), 0);
    state[0] = 0; state[1] = toks[0]; state[3] = 0;
    int rc = 0;
    for (int p = 0; p < 3; p++) {
        state[1] = toks[p];   // teacher forcing
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
        if (!ok || flag || !(err <= 1e-3f * scale + 1e-3f) || state[0] != p + 1) rc = 1;
        if (rc) break;
    }
    printf(rc ? "EMU FAIL\n" : "EMU OK\n");
    return rc;
}
