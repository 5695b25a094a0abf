// Fiber runtime of the CPU emulation: every GPU thread of a launch is a fiber (see tests/emu/hip/hip_runtime.h for the
// execution model).  TEST INFRASTRUCTURE: included by exactly one translation unit per emulation program.
#pragma once

#include <sys/mman.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <vector>

#include <hip/hip_runtime.h>

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define EMU_ASAN 1
#include <sanitizer/asan_interface.h>
#include <sanitizer/common_interface_defs.h>
#endif
#endif
// EMU_TSAN is given on the command line of the race-detecting build: this file itself is compiled without the
// instrumentation there (the scheduler's own bookkeeping is touched from every context by design).
#ifdef EMU_TSAN
#include <sanitizer/tsan_interface.h>
#endif

// ------------------------------------------------------------------ fiber runtime
// The switch between two stacks, written out (x86-64, System V): callee-saved registers on the old stack, stack pointers
// exchanged, the same registers off the new stack.  swapcontext would do, but AddressSanitizer intercepts it and clears
// the shadow of the whole stack it switches to, every time, which makes a launch of a few hundred thousand fibers take
// minutes.  The sanitizer is told about every switch through its fiber interface instead.
extern "C" void emu_switch_stack(void **save_sp, void *new_sp);
asm(R"(
    .text
    .p2align 4
    .globl emu_switch_stack
    .hidden emu_switch_stack
    .type emu_switch_stack,@function
emu_switch_stack:
    pushq %rbp
    pushq %rbx
    pushq %r12
    pushq %r13
    pushq %r14
    pushq %r15
    movq %rsp, (%rdi)
    movq %rsi, %rsp
    popq %r15
    popq %r14
    popq %r13
    popq %r12
    popq %rbx
    popq %rbp
    ret
    .size emu_switch_stack, .-emu_switch_stack
)");

// the scheduler's own bookkeeping is touched from every context by design: never watched by the race detector, whether
// this file is compiled into a translation unit with the instrumentation (a self-contained test program) or without
#ifdef EMU_TSAN
#pragma clang attribute push(__attribute__((no_sanitize("thread"))), apply_to = function)
#endif
namespace emu {

enum State { RUNNABLE, AT_SYNC, AT_WAVE, AT_GATHER, AT_UNIFORM, SPIN, DONE };
// EMU_STACK_BYTES: stack of a fiber (default 256 KB above one guard page).  EMU_STACK_ARENA = n: the stacks of up to n
// fibers come out of one mapping without guard pages -- for grids of hundreds of thousands of fibers that are all alive at
// once (a kernel whose workgroups wait for one another), where one mapping per fiber would exceed the kernel's limit on
// mappings per process.
#ifndef EMU_STACK_BYTES
#define EMU_STACK_BYTES (256 * 1024)
#endif
constexpr size_t kStack = EMU_STACK_BYTES;

struct Fiber {
    void *sp = nullptr;       // where the fiber's registers lie while it is not running
    char *stack = nullptr;
    State state = RUNNABLE;
    Idx3 tid{ 0, 0, 0 };
    unsigned linear = 0;      // thread number within the workgroup (x fastest): lanes of a wave are 64 consecutive numbers
    int block = 0;
    uint32_t xval = 0, xres = 0;
    int xsrc = 0;
    const void *gmine = nullptr;   // wave gather: this lane's contribution ...
    size_t gbytes = 0;             // ... of this many bytes
    const void *gall = nullptr;    // ... and, afterwards, the wave's 64 contributions in lane order
};

struct Block {
    std::vector<Fiber> fibers;
    std::vector<std::vector<char>> gather;   // one buffer per wave
    Idx3 bid{ 0, 0, 0 };
    bool started = false, done = false;
};

Fiber *g_cur = nullptr;
static void *g_main_sp = nullptr;
static const void *g_main_bottom = nullptr;
static size_t g_main_size = 0;
static std::vector<Block> g_blocks;
static Idx3 g_bdim{ 1, 1, 1 }, g_gdim{ 1, 1, 1 };
static std::vector<char> g_lds;
static std::function<void()> g_kernel;
static long g_switches = 0;
static std::vector<char *> g_stack_pool;

// Under ThreadSanitizer a wave is a thread of the race detector: its 64 lanes share one context (they run in lockstep
// on the device, so what one lane writes another may read), different waves of a workgroup are different contexts
// with no order between them except at a workgroup barrier, and workgroups and launches follow one another.  A
// write by one wave and an access by another with no barrier between is then reported as a data race.
#ifdef EMU_TSAN
static void *g_tsan_main = nullptr;
static std::vector<void *> g_tsan_wave;
static char g_tsan_barrier, g_tsan_order;      // addresses the happens-before edges hang on
static void *tsan_wave(unsigned wave) {
    while (g_tsan_wave.size() <= wave) g_tsan_wave.push_back(__tsan_create_fiber(0));
    return g_tsan_wave[wave];
}
#endif

Idx3 &tid() { return g_cur->tid; }
Idx3 &bid() { return g_blocks[(size_t)g_cur->block].bid; }
Idx3 &bdim() { return g_bdim; }
Idx3 &gdim() { return g_gdim; }
void *dyn_lds() { return g_lds.data(); }
size_t dyn_lds_bytes() { return g_lds.size(); }
int lane_id() { return (int)(g_cur->linear & 63); }

static void to_main() {
    Fiber *f = g_cur;
#ifdef EMU_TSAN
    __tsan_switch_to_fiber(g_tsan_main, __tsan_switch_to_fiber_no_sync);
#endif
#ifdef EMU_ASAN
    void *fake = nullptr;
    __sanitizer_start_switch_fiber(f->state == DONE ? nullptr : &fake, g_main_bottom, g_main_size);
#endif
    emu_switch_stack(&f->sp, g_main_sp);
#ifdef EMU_ASAN
    __sanitizer_finish_switch_fiber(fake, &g_main_bottom, &g_main_size);
#endif
}

void sync_threads() {
#ifdef EMU_TSAN
    __tsan_release(&g_tsan_barrier);       // every lane arrives before any leaves
#endif
    g_cur->state = AT_SYNC;
    to_main();
#ifdef EMU_TSAN
    __tsan_acquire(&g_tsan_barrier);
#endif
}
void spin_yield() { g_cur->state = SPIN; to_main(); }
uint32_t wave_exchange(uint32_t v, int src) {
    g_cur->xval = v;
    g_cur->xsrc = src;
    g_cur->state = AT_WAVE;
    to_main();
    return g_cur->xres;
}
void uniform_point() { g_cur->state = AT_UNIFORM; to_main(); }
const void *wave_gather(const void *mine, size_t bytes) {
    g_cur->gmine = mine;
    g_cur->gbytes = bytes;
    g_cur->state = AT_GATHER;
    to_main();
    return g_cur->gall;
}

static void fiber_entry() {
#ifdef EMU_ASAN
    __sanitizer_finish_switch_fiber(nullptr, &g_main_bottom, &g_main_size);
#endif
#ifdef EMU_TSAN
    __tsan_acquire(&g_tsan_order);         // after the host's writes and the workgroups that ran before this one
#endif
    g_kernel();
#ifdef EMU_TSAN
    __tsan_release(&g_tsan_order);
#endif
    g_cur->state = DONE;
    to_main();
}

static void resume(Fiber &f) {
    g_cur = &f;
    g_switches++;
#ifdef EMU_TSAN
    __tsan_switch_to_fiber(tsan_wave(f.linear >> 6), __tsan_switch_to_fiber_no_sync);
#endif
#ifdef EMU_ASAN
    void *fake = nullptr;
    __sanitizer_start_switch_fiber(&fake, f.stack, kStack);
#endif
    emu_switch_stack(&g_main_sp, f.sp);
#ifdef EMU_ASAN
    __sanitizer_finish_switch_fiber(fake, nullptr, nullptr);
#endif
    g_cur = nullptr;
}

static char *take_stack() {
    if (!g_stack_pool.empty()) {
        char *s = g_stack_pool.back();
        g_stack_pool.pop_back();
#ifdef EMU_ASAN
        __asan_unpoison_memory_region(s, kStack);      // the frames of the fiber that ran here last never returned
#endif
        return s;
    }
#ifdef EMU_STACK_ARENA
    static char *arena = nullptr;
    static size_t taken = 0;
    if (!arena) {
        arena = (char *)mmap(nullptr, (size_t)EMU_STACK_ARENA * kStack, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
        if (arena == (char *)MAP_FAILED) { perror("mmap"); exit(2); }
    }
    if (taken == (size_t)EMU_STACK_ARENA) { fprintf(stderr, "emu: more than EMU_STACK_ARENA fibers alive\n"); exit(2); }
    return arena + kStack * taken++;
#else
    char *s = (char *)mmap(nullptr, kStack + 4096, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (s == (char *)MAP_FAILED) { perror("mmap"); exit(2); }
    mprotect(s, 4096, PROT_NONE);      // a fiber that outgrows its stack stops here instead of writing into another's
    return s + 4096;
#endif
}

static void start_block(Block &b, int index) {
    const unsigned n = g_bdim.x * g_bdim.y * g_bdim.z;
    b.fibers.resize(n);
    b.gather.assign((n + 63) / 64, std::vector<char>(64 * 64));      // room for 64 bytes per lane, sized here once
    for (unsigned t = 0; t < n; t++) {
        Fiber &f = b.fibers[t];
        f.linear = t;
        f.tid = Idx3{ t % g_bdim.x, t / g_bdim.x % g_bdim.y, t / (g_bdim.x * g_bdim.y) };
        f.block = index;
        f.stack = take_stack();
        // the first switch to the fiber pops six registers and returns into fiber_entry, the stack then as after a call
        void **top = reinterpret_cast<void **>(f.stack + kStack);
        *--top = nullptr;                                   // the return address fiber_entry never uses
        *--top = reinterpret_cast<void *>(&fiber_entry);
        for (int r = 0; r < 6; r++) *--top = nullptr;
        f.sp = top;
    }
    b.started = true;
#ifdef EMU_TSAN
    __tsan_release(&g_tsan_order);         // the lanes read what was set up here (their indices)
#endif
}

static void finish_block(Block &b) {
#ifdef EMU_TSAN
    __tsan_acquire(&g_tsan_order);         // the host continues after the workgroup's last access (and frees what its lanes read)
#endif
    for (Fiber &f : b.fibers) g_stack_pool.push_back(f.stack);
    b.fibers.clear();
    b.fibers.shrink_to_fit();
    b.gather.clear();
    b.done = true;
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
            bool any = false, any_gather = false, any_uniform = false;
            for (size_t i = w0; i < w1; i++) {
                any = any || b.fibers[i].state == AT_WAVE;
                any_gather = any_gather || b.fibers[i].state == AT_GATHER;
                any_uniform = any_uniform || b.fibers[i].state == AT_UNIFORM;
            }
            // lanes at an instruction every lane executes (a wait, which lanes cannot skip) stay there until the lanes
            // that are still at wave operations before it have caught up: lanes that skipped a predicated operation
            // run ahead of the others by that much and no further
            if (any_uniform && !any && !any_gather) {
                for (size_t i = w0; i < w1; i++)
                    if (b.fibers[i].state == AT_UNIFORM) b.fibers[i].state = RUNNABLE;
                progressed = true;
            }
            if (any) {
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
            if (any_gather) {
                size_t bytes = 0;
                for (size_t i = w0; i < w1; i++)
                    if (b.fibers[i].state == AT_GATHER) bytes = std::max(bytes, b.fibers[i].gbytes);
                // (byte loops, not memset / memcpy: the race-detecting build intercepts those and would book them as
                // accesses of the host, while this is the wave handing its own registers round)
                std::vector<char> &buf = b.gather[w0 / 64];
                if (buf.size() < 64 * bytes) buf.resize(64 * bytes);
                volatile char *dst = buf.data();
                for (size_t k = 0; k < 64 * bytes; k++) dst[k] = 0;      // lanes that are not at the operation contribute zeros
                for (size_t i = w0; i < w1; i++) {
                    Fiber &f = b.fibers[i];
                    if (f.state != AT_GATHER) continue;
                    const volatile char *src = static_cast<const char *>(f.gmine);
                    for (size_t k = 0; k < f.gbytes; k++) dst[(i - w0) * bytes + k] = src[k];
                }
                for (size_t i = w0; i < w1; i++) {
                    Fiber &f = b.fibers[i];
                    if (f.state != AT_GATHER) continue;
                    f.gall = buf.data();
                    f.state = RUNNABLE;
                }
                progressed = true;
            }
        }
        if (progressed) continue;
        size_t at_sync = 0, done = 0, spin = 0;
        for (Fiber &f : b.fibers) {
            at_sync += f.state == AT_SYNC;
            done += f.state == DONE;
            spin += f.state == SPIN;
        }
        if (done == n) { finish_block(b); return true; }
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
        fprintf(stderr, "emu: dead rendezvous in workgroup (%u,%u,%u) (at_sync=%zu done=%zu)\n", b.bid.x, b.bid.y, b.bid.z, at_sync, done);
        return false;
    }
}

// Launch `kernel` on grid x block threads with lds_bytes of launch-sized LDS.  Returns false on a stall.  A workgroup's
// fibers exist from its first turn to its end; workgroups that never wait for one another run one after the other.
bool launch3(Idx3 grid, Idx3 block, size_t lds_bytes, std::function<void()> kernel) {
    g_kernel = std::move(kernel);
    g_bdim = block;
    g_gdim = grid;
    // a heap buffer of exactly the launch's size: overruns are caught; LDS comes up undefined on the device, so it is
    // filled with NaN patterns here and a kernel that reads what it never wrote does not pass its test by luck
    g_lds.assign(lds_bytes, (char)0xFF);
#ifdef EMU_TSAN
    g_tsan_main = __tsan_get_current_fiber();
    __tsan_release(&g_tsan_order);
#endif
    const size_t n_blocks = (size_t)grid.x * grid.y * grid.z;
    g_blocks.assign(n_blocks, Block());
    for (size_t bi = 0; bi < n_blocks; bi++)
        g_blocks[bi].bid = Idx3{ (unsigned)(bi % grid.x), (unsigned)(bi / grid.x % grid.y), (unsigned)(bi / ((size_t)grid.x * grid.y)) };
    bool ok = true;
    for (long rounds = 0; ok; rounds++) {
        bool all = true;
        for (size_t bi = 0; bi < n_blocks; bi++) {
            Block &b = g_blocks[bi];
            if (b.done) continue;
            all = false;
            if (!b.started) start_block(b, (int)bi);
            if (!run_block(b)) { ok = false; break; }
        }
        if (all) break;
        if (rounds > 100000) { fprintf(stderr, "emu: no progress after %ld rounds\n", rounds); ok = false; }
    }
    for (Block &b : g_blocks)
        if (b.started && !b.done) finish_block(b);
    g_blocks.clear();
    g_kernel = nullptr;
    return ok;
}

bool launch(unsigned grid, unsigned block, size_t lds_bytes, std::function<void()> kernel) {
    return launch3(Idx3{ grid, 1, 1 }, Idx3{ block, 1, 1 }, lds_bytes, std::move(kernel));
}

}  // namespace emu
#ifdef EMU_TSAN
#pragma clang attribute pop
#endif
