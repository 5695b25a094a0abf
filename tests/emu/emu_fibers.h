// Fiber runtime of the CPU emulation: every GPU thread of a launch is a fiber (see tests/emu/hip/hip_runtime.h for the
// execution model).  TEST INFRASTRUCTURE: included by exactly one translation unit per emulation program.
#pragma once

#include <sys/mman.h>
#include <ucontext.h>

#include <cstdio>
#include <cstdlib>
#include <functional>
#include <vector>

#include <hip/hip_runtime.h>

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

