// CPU run of the persistent decode-step kernel (rustorch_amd/csrc/rt_mega_device.h) under AddressSanitizer.
// TEST INFRASTRUCTURE.  Every GPU thread is a fiber; see tests/emu/hip/hip_runtime.h for the execution model.
// What it checks: no out-of-bounds access to any buffer the kernel is handed, every workgroup leaves the
// kernel (no barrier time-out, no dead rendezvous), and the logits agree with the CPU oracle.
//
// usage: emu_main [n_wg]        (n_wg: number of workgroups, a multiple of 8 and >= n_heads; default 8)
#include <sys/mman.h>
#include <ucontext.h>

#include <cstdio>
#include <cstdlib>
#include <functional>
#include <vector>

#include "rt_mega_device.h"

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define EMU_ASAN 1
#include <sanitizer/common_interface_defs.h>
#endif
#endif

// ------------------------------------------------------------------ fiber runtime
namespace emu {

enum State { RUNNABLE, AT_SYNC, AT_WAVE, SPIN, DONE };
constexpr size_t kStack = 512 * 1024;

struct Fiber {
    ucontext_t ctx;
    char *stack = nullptr;
    State state = RUNNABLE;
    Idx3 tid{ 0, 0, 0 };
    int block = 0;
    uint32_t xval = 0, xres = 0;
    int xsrc = 0;
    bool started = false;
};

struct Block {
    std::vector<Fiber> fibers;
    Idx3 bid{ 0, 0, 0 };
    bool done = false;
};

Fiber *g_cur = nullptr;
static ucontext_t g_main;
static const void *g_main_bottom = nullptr;
static size_t g_main_size = 0;
static std::vector<Block> g_blocks;
static Idx3 g_bdim{ 1, 1, 1 }, g_gdim{ 1, 1, 1 };
static std::vector<char> g_lds;
static std::function<void()> g_kernel;
static long g_switches = 0;

Idx3 &tid() { return g_cur->tid; }
Idx3 &bid() { return g_blocks[(size_t)g_cur->block].bid; }
Idx3 &bdim() { return g_bdim; }
Idx3 &gdim() { return g_gdim; }
void *dyn_lds() { return g_lds.data(); }
int lane_id() { return (int)(g_cur->tid.x & 63); }

static void to_main() {
    Fiber *f = g_cur;
#ifdef EMU_ASAN
    void *fake = nullptr;
    __sanitizer_start_switch_fiber(f->state == DONE ? nullptr : &fake, g_main_bottom, g_main_size);
#endif
    swapcontext(&f->ctx, &g_main);
#ifdef EMU_ASAN
    __sanitizer_finish_switch_fiber(fake, &g_main_bottom, &g_main_size);
#endif
}

void sync_threads() { g_cur->state = AT_SYNC; to_main(); }
void spin_yield() { g_cur->state = SPIN; to_main(); }
uint32_t wave_exchange(uint32_t v, int src) {
    g_cur->xval = v;
    g_cur->xsrc = src;
    g_cur->state = AT_WAVE;
    to_main();
    return g_cur->xres;
}

static void fiber_entry() {
#ifdef EMU_ASAN
    __sanitizer_finish_switch_fiber(nullptr, &g_main_bottom, &g_main_size);
#endif
    g_kernel();
    g_cur->state = DONE;
    to_main();
}

static void resume(Fiber &f) {
    g_cur = &f;
    g_switches++;
#ifdef EMU_ASAN
    void *fake = nullptr;
    __sanitizer_start_switch_fiber(&fake, f.stack, kStack);
#endif
    swapcontext(&g_main, &f.ctx);
#ifdef EMU_ASAN
    __sanitizer_finish_switch_fiber(fake, nullptr, nullptr);
#endif
    g_cur = nullptr;
}

// Runs the workgroup until it is finished or stuck in a spin wait. Returns false on a dead rendezvous.
static bool run_block(Block &b) {
    for (;;) {
        for (Fiber &f : b.fibers)
            if (f.state == RUNNABLE) resume(f);
        bool progressed = false;
        size_t n = b.fibers.size();
        // wave rendezvous: exchange among the lanes that are waiting at a wave operation
        for (size_t w0 = 0; w0 < n; w0 += 64) {
            size_t w1 = std::min(n, w0 + 64);
            bool any = false;
            for (size_t i = w0; i < w1; i++) any = any || b.fibers[i].state == AT_WAVE;
            if (!any) continue;
            for (size_t i = w0; i < w1; i++) {
                Fiber &f = b.fibers[i];
                if (f.state != AT_WAVE) continue;
                size_t s = w0 + (size_t)(f.xsrc & 63);
                f.xres = (f.xsrc >= 0 && s < w1 && b.fibers[s].state == AT_WAVE) ? b.fibers[s].xval : f.xval;
            }
            for (size_t i = w0; i < w1; i++)
                if (b.fibers[i].state == AT_WAVE) b.fibers[i].state = RUNNABLE;
            progressed = true;
        }
        if (progressed) continue;
        size_t at_sync = 0, done = 0, spin = 0;
        for (Fiber &f : b.fibers) {
            at_sync += f.state == AT_SYNC;
            done += f.state == DONE;
            spin += f.state == SPIN;
        }
        if (done == n) { b.done = true; return true; }
        if (at_sync + done == n) {
            for (Fiber &f : b.fibers)
                if (f.state == AT_SYNC) f.state = RUNNABLE;
            continue;
        }
        if (spin > 0) {   // waiting on other workgroups: let them run
            for (Fiber &f : b.fibers)
                if (f.state == SPIN) f.state = RUNNABLE;
            return true;
        }
        fprintf(stderr, "emu: dead rendezvous in workgroup %u (at_sync=%zu done=%zu)\n", b.bid.x, at_sync, done);
        return false;
    }
}

// Launch `kernel` on grid x block threads (1-D) with lds_bytes of launch-sized LDS. Returns false on a stall.
bool launch(unsigned grid, unsigned block, size_t lds_bytes, std::function<void()> kernel) {
    g_kernel = std::move(kernel);
    g_bdim = Idx3{ block, 1, 1 };
    g_gdim = Idx3{ grid, 1, 1 };
    g_lds.assign(lds_bytes, 0);   // a heap buffer of exactly the launch's size: overruns are caught
    g_blocks.assign(grid, Block());
    for (unsigned bi = 0; bi < grid; bi++) {
        Block &b = g_blocks[bi];
        b.bid = Idx3{ bi, 0, 0 };
        b.fibers.resize(block);
        for (unsigned t = 0; t < block; t++) {
            Fiber &f = b.fibers[t];
            f.tid = Idx3{ t, 0, 0 };
            f.block = (int)bi;
            f.stack = (char *)mmap(nullptr, kStack, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
            if (f.stack == (char *)MAP_FAILED) { perror("mmap"); exit(2); }
            getcontext(&f.ctx);
            f.ctx.uc_stack.ss_sp = f.stack;
            f.ctx.uc_stack.ss_size = kStack;
            f.ctx.uc_link = nullptr;
            makecontext(&f.ctx, fiber_entry, 0);
        }
    }
    bool ok = true;
    for (long rounds = 0; ok; rounds++) {
        bool all = true;
        for (Block &b : g_blocks) {
            if (b.done) continue;
            all = false;
            if (!run_block(b)) { ok = false; break; }
        }
        if (all) break;
        if (rounds > 100000) { fprintf(stderr, "emu: no progress after %ld rounds\n", rounds); ok = false; }
    }
    for (Block &b : g_blocks)
        for (Fiber &f : b.fibers) munmap(f.stack, kStack);
    g_blocks.clear();
    return ok;
}

}  // namespace emu

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
