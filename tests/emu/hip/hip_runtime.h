// CPU stand-in for <hip/hip_runtime.h>: the HIP device vocabulary the sources of rustorch_amd/csrc use (thread indices,
// LDS, wave operations, matrix-core and LDS-DMA builtins, buffer loads, atomics, the few hand-written instructions) and the
// part of the host API they call (memory, streams, events, captured graphs), so that the same sources compile as host C++
// and run under AddressSanitizer or ThreadSanitizer.  TEST INFRASTRUCTURE: used only by the programs and the emulated
// library under tests/emu.
//
// Execution model (tests/emu/emu_fibers.h): a GPU thread is a fiber; a workgroup's fibers run one after the other, each
// until it reaches __syncthreads(), a wave operation (shuffle / DPP / readlane / a matrix instruction / a wave barrier /
// a hand-written LDS instruction / a wait), a sleep inside a spin loop, or its end.  Workgroups run one after the other; a
// workgroup is left before its end only while it spins on another one (a grid barrier), at which point its LDS contents
// are dead, so one launch-sized LDS buffer serves all workgroups.  Wave operations are a rendezvous of the wave's lanes.
#pragma once

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))

struct uint2 { uint32_t x, y; };
struct alignas(16) uint4 { uint32_t x, y, z, w; };
struct float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
inline uint2 make_uint2(uint32_t x, uint32_t y) { return uint2{ x, y }; }
inline uint4 make_uint4(uint32_t x, uint32_t y, uint32_t z, uint32_t w) { return uint4{ x, y, z, w }; }
inline float2 make_float2(float x, float y) { return float2{ x, y }; }
inline float4 make_float4(float x, float y, float z, float w) { return float4{ x, y, z, w }; }
struct dim3 { unsigned x = 1, y = 1, z = 1; dim3() {} dim3(unsigned a, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {} };

typedef int hipError_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2, hipErrorInvalidDevice = 101, hipErrorInvalidSymbol = 13, hipErrorNotSupported = 801, hipErrorLaunchFailure = 719 };
inline const char *hipGetErrorString(hipError_t e) {
    return e == hipSuccess ? "no error" : (e == hipErrorNotSupported ? "not supported by the emulation" : (e == hipErrorLaunchFailure ? "emulated launch stalled" : "emulated HIP error"));
}

namespace emu {

struct Idx3 { unsigned x, y, z; };
struct Fiber;
extern Fiber *g_cur;          // the fiber that is running
Idx3 &tid();
Idx3 &bid();
Idx3 &bdim();
Idx3 &gdim();
void *dyn_lds();
size_t dyn_lds_bytes();
void sync_threads();
void spin_yield();
// 64-lane rendezvous: every live lane of the wave deposits v; returns the value deposited by lane `src`
uint32_t wave_exchange(uint32_t v, int src);
// 64-lane rendezvous: every live lane deposits `bytes` bytes; returns the wave's 64 deposits in lane order (valid until
// the wave's next operation; lanes that are not at the operation count as zeros)
const void *wave_gather(const void *mine, size_t bytes);
// An instruction that every lane of a wave executes whatever its predicates (the sources' hand-placed waits): the lanes
// that arrive first wait here for the rest of their wave.  Lanes that skipped a predicated wave operation would otherwise
// pair up, from then on, with the others' previous operation.
void uniform_point();
int lane_id();
bool launch3(Idx3 grid, Idx3 block, size_t lds_bytes, std::function<void()> kernel);
bool trace_launches();      // EMU_TRACE_LAUNCHES=1 in the environment: every launch is named on stderr (a report then has its context)
hipError_t &last_error();

}  // namespace emu

// ---- the host API the library uses: one device, synchronous "streams", device memory = exact-size heap blocks
typedef struct emu_stream *hipStream_t;
struct emu_event { std::chrono::steady_clock::time_point at; };
typedef emu_event *hipEvent_t;
typedef struct emu_graph *hipGraph_t;
typedef struct emu_graph_exec *hipGraphExec_t;
enum hipMemcpyKind { hipMemcpyHostToHost, hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice, hipMemcpyDefault };
enum { hipStreamNonBlocking = 1, hipStreamCaptureModeThreadLocal = 1, hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
constexpr size_t kEmuDeviceBytes = (size_t)8 << 30;      // what the emulated device reports and hands out
struct hipDeviceProp_t {
    char name[256];
    char gcnArchName[256];
    int multiProcessorCount, warpSize, cooperativeLaunch;
    size_t totalGlobalMem, sharedMemPerBlock;
};
inline hipError_t hipGetLastError() { hipError_t e = emu::last_error(); emu::last_error() = hipSuccess; return e; }
inline hipError_t hipGetDeviceCount(int *n) { *n = 1; return hipSuccess; }
inline hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidDevice; }
inline hipError_t hipGetDevice(int *d) { *d = 0; return hipSuccess; }
inline hipError_t hipGetDeviceProperties(hipDeviceProp_t *p, int d) {
    if (d != 0) return hipErrorInvalidDevice;
    memset(p, 0, sizeof *p);
    snprintf(p->name, sizeof p->name, "CPU emulation of an MI355X");
    snprintf(p->gcnArchName, sizeof p->gcnArchName, "gfx950 (emulated)");
    p->multiProcessorCount = 256; p->warpSize = 64; p->cooperativeLaunch = 0;
    p->totalGlobalMem = kEmuDeviceBytes; p->sharedMemPerBlock = 64 * 1024;
    return hipSuccess;
}
// device memory: exact-size heap blocks (the sanitizer guards their ends), counted against the size the device reports
hipError_t hipMalloc(void **p, size_t n);
hipError_t hipFree(void *p);
inline hipError_t hipMemcpy(void *d, const void *s, size_t n, hipMemcpyKind) { memcpy(d, s, n); return hipSuccess; }
// Work given to a stream runs at once -- or, while the stream is being captured, is recorded for the graph's replays.
namespace emu { bool submit(hipStream_t s, std::function<void()> work); }
inline hipError_t hipMemcpyAsync(void *d, const void *s, size_t n, hipMemcpyKind, hipStream_t st) {
    emu::submit(st, [=] { memmove(d, s, n); });
    return hipSuccess;
}
inline hipError_t hipMemsetAsync(void *d, int v, size_t n, hipStream_t st) {
    emu::submit(st, [=] { memset(d, v, n); });
    return hipSuccess;
}
inline hipError_t hipStreamCreate(hipStream_t *s) { *s = (hipStream_t)malloc(1); return hipSuccess; }
inline hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) { return hipStreamCreate(s); }
inline hipError_t hipStreamDestroy(hipStream_t s) { free(s); return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
inline hipError_t hipEventCreate(hipEvent_t *e) { *e = new emu_event(); return hipSuccess; }
inline hipError_t hipEventDestroy(hipEvent_t e) { delete e; return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t e, hipStream_t) { e->at = std::chrono::steady_clock::now(); return hipSuccess; }
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventElapsedTime(float *ms, hipEvent_t a, hipEvent_t b) {
    *ms = std::chrono::duration<float, std::milli>(b->at - a->at).count();
    return hipSuccess;
}
template <class F> inline hipError_t hipFuncSetAttribute(F, int, int) { return hipSuccess; }
// a __device__ variable is a host global here: its address is its own
#define HIP_SYMBOL(x) (x)
template <class T> inline hipError_t hipGetSymbolAddress(void **p, T &symbol) { *p = (void *)&symbol; return hipSuccess; }
// captured graphs: the list of work recorded between begin and end; a launch of the graph runs the list again
hipError_t hipStreamBeginCapture(hipStream_t s, int mode);
hipError_t hipStreamEndCapture(hipStream_t s, hipGraph_t *g);
hipError_t hipGraphInstantiate(hipGraphExec_t *e, hipGraph_t g, void *, void *, size_t);
hipError_t hipGraphLaunch(hipGraphExec_t e, hipStream_t s);
hipError_t hipGraphDestroy(hipGraph_t g);
hipError_t hipGraphExecDestroy(hipGraphExec_t e);

// kernel<<<grid, block, lds, stream>>>(args) of the sources, rewritten by tests/emu/build_emulated.py: runs the grid to its
// end before it returns (arguments are taken by value, as a launch takes them); a stall -- a barrier that not every
// thread reaches -- is reported as a failed launch
inline emu::Idx3 emu_idx3(dim3 d) { return emu::Idx3{ d.x, d.y, d.z }; }
#define EMU_LAUNCH(kernel, grid, block, lds, stream, ...)                                                                   \
    do {                                                                                                                    \
        const emu::Idx3 emu_g = emu_idx3(dim3(grid)), emu_b = emu_idx3(dim3(block));                                        \
        const size_t emu_l = (size_t)(lds);                                                                                 \
        if (emu::trace_launches()) fprintf(stderr, "emu: launch %s at %s:%d\n", #kernel, __FILE__, __LINE__);                \
        emu::submit(stream, [=] {                                                                                           \
            if (!emu::launch3(emu_g, emu_b, emu_l, [=] { kernel(__VA_ARGS__); })) emu::last_error() = hipErrorLaunchFailure; \
        });                                                                                                                 \
    } while (0)


#define threadIdx (emu::tid())
#define blockIdx (emu::bid())
#define blockDim (emu::bdim())
#define gridDim (emu::gdim())
#define RT_DYN_LDS(T, name) T *name = reinterpret_cast<T *>(emu::dyn_lds())

inline void __syncthreads() { emu::sync_threads(); }

// ---- scalar helpers of the HIP device library
inline int __float_as_int(float f) { int i; std::memcpy(&i, &f, 4); return i; }
inline float __int_as_float(int i) { float f; std::memcpy(&f, &i, 4); return f; }
inline float __uint_as_float(unsigned i) { float f; std::memcpy(&f, &i, 4); return f; }
// v_cvt_i32_f32: NaN gives 0, values beyond the range saturate (a plain C++ conversion of those is undefined)
inline int __float2int_rn(float f) {
    if (f != f) return 0;
    const float r = std::nearbyintf(f);
    return r >= 2147483648.0f ? 2147483647 : (r <= -2147483648.0f ? (-2147483647 - 1) : (int)r);
}
inline int __mul24(int a, int b) { return (int)((unsigned)((a << 8) >> 8) * (unsigned)((b << 8) >> 8)); }     // v_mul_i32_i24
using std::max;
using std::min;
inline void sincosf_emu(float a, float *s, float *c) { *s = std::sin(a); *c = std::cos(a); }
#define sincosf sincosf_emu

// ---- wave operations
inline float __shfl_xor(float v, int mask, int = 64) {
    return __int_as_float((int)emu::wave_exchange((uint32_t)__float_as_int(v), emu::lane_id() ^ mask));
}
inline int __shfl_xor(int v, int mask, int = 64) { return (int)emu::wave_exchange((uint32_t)v, emu::lane_id() ^ mask); }

inline int emu_update_dpp(int old, int src, int ctrl, int row_mask, int /*bank_mask*/, bool /*bound_ctrl*/) {
    int l = emu::lane_id(), from = l;
    bool write = ((row_mask >> (l >> 4)) & 1) != 0;
    if (ctrl < 0x100) from = (l & ~3) + ((ctrl >> (2 * (l & 3))) & 3);   // quad_perm
    else if (ctrl == 0x141) from = (l & ~7) + (7 - (l & 7));               // row_half_mirror
    else if (ctrl == 0x140) from = (l & ~15) + (15 - (l & 15));            // row_mirror
    else if (ctrl == 0x142) { from = (l & ~15) - 1; if (l < 16) { from = l; write = false; } }   // row_bcast:15
    else if (ctrl == 0x143) { from = 31; if (l < 32) { from = l; write = false; } }              // row_bcast:31
    int got = (int)emu::wave_exchange((uint32_t)src, from);
    return write ? got : old;
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) emu_update_dpp(old, src, ctrl, rm, bm, bc)
#define __builtin_amdgcn_readlane(v, l) ((int)emu::wave_exchange((uint32_t)(v), (l)))
#define __builtin_amdgcn_readfirstlane(v) (v)
inline int emu_sdot4(int a, int b, int c) {
    for (int i = 0; i < 4; i++) c += (int)(int8_t)(a >> (8 * i)) * (int)(int8_t)(b >> (8 * i));
    return c;
}
#define __builtin_amdgcn_sdot4(a, b, c, clamp) emu_sdot4(a, b, c)
// v_perm_b32: byte i of the result is byte sel_i of the eight bytes { s1 (0..3), s0 (4..7) }; selectors from 12 up give constants
inline unsigned emu_perm(unsigned s0, unsigned s1, unsigned sel) {
    const unsigned long long src = ((unsigned long long)s0 << 32) | s1;
    unsigned r = 0;
    for (int i = 0; i < 4; i++) {
        const unsigned k = (sel >> (8 * i)) & 0xFF;
        const unsigned byte = k < 8 ? (unsigned)(src >> (8 * k)) & 0xFF : (k >= 13 ? 0xFFu : 0u);
        r |= byte << (8 * i);
    }
    return r;
}
#define __builtin_amdgcn_perm(a, b, sel) emu_perm(a, b, sel)
inline void unsafeAtomicAdd(float *p, float v) {
    uint32_t seen, want;
    __atomic_load(reinterpret_cast<uint32_t *>(p), &seen, __ATOMIC_RELAXED);
    do {
        float f;
        memcpy(&f, &seen, 4);
        f += v;
        memcpy(&want, &f, 4);
    } while (!__atomic_compare_exchange(reinterpret_cast<uint32_t *>(p), &seen, &want, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED));
}
// buffer resources (raw, stride 0): base pointer and num_records.  A load must lie inside the resource -- the sources never
// rely on the zeros the hardware returns for an out-of-range lane, so here such a lane ends the run, which is stricter than
// the device and than the address sanitizer (a wild offset can land inside another live block).  The check is made both
// ways the range check may be defined (with and without the scalar offset), and the bytes must belong to one allocation of
// the emulated device where the runtime that tracks them is linked in.
struct emu_buffer_rsrc { const unsigned char *base; unsigned num; };
typedef emu_buffer_rsrc __amdgpu_buffer_rsrc_t;
typedef unsigned int emu_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int emu_u32x2 __attribute__((ext_vector_type(2)));
extern "C" int emu_device_owns(const void *p, size_t n) __attribute__((weak));      // emu_library.cpp; absent in stand-alone drivers
inline emu_buffer_rsrc emu_make_rsrc(const void *p, int num) { return emu_buffer_rsrc{ (const unsigned char *)p, (unsigned)num }; }
inline void emu_bload(void *dst, emu_buffer_rsrc r, unsigned voff, unsigned soff, unsigned size) {
    if ((unsigned long long)voff + soff + size > r.num) {
        fprintf(stderr, "emu: buffer load out of range: voffset %u + soffset %u + %u bytes > num_records %u\n", voff, soff, size, r.num);
        abort();
    }
    if (emu_device_owns && !emu_device_owns(r.base + voff + soff, size)) {
        fprintf(stderr, "emu: buffer load of %u bytes at %p (voffset %u, soffset %u) is not inside one device allocation\n", size,
                (const void *)(r.base + voff + soff), voff, soff);
        abort();
    }
    __builtin_memcpy(dst, r.base + voff + soff, size);
}
inline emu_u32x4 emu_bload128(emu_buffer_rsrc r, unsigned voff, unsigned soff) { emu_u32x4 v; emu_bload(&v, r, voff, soff, 16); return v; }
inline emu_u32x2 emu_bload64(emu_buffer_rsrc r, unsigned voff, unsigned soff) { emu_u32x2 v; emu_bload(&v, r, voff, soff, 8); return v; }
inline unsigned int emu_bload32(emu_buffer_rsrc r, unsigned voff, unsigned soff) { unsigned int v; emu_bload(&v, r, voff, soff, 4); return v; }
inline short emu_bload16(emu_buffer_rsrc r, unsigned voff, unsigned soff) { short v; emu_bload(&v, r, voff, soff, 2); return v; }
#define __builtin_amdgcn_make_buffer_rsrc(p, stride, num, flags) emu_make_rsrc(p, num)
#define __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, aux) emu_bload128(r, voff, soff)
#define __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, aux) emu_bload64(r, voff, soff)
#define __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, aux) emu_bload32(r, voff, soff)
#define __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, aux) emu_bload16(r, voff, soff)
#define __builtin_amdgcn_s_sleep(n) emu::spin_yield()
#define __builtin_amdgcn_s_waitcnt(n) emu::uniform_point()     // nothing to wait for; see uniform_point

// ---- device-scope atomics: fibers never run concurrently, so any access would be exact; they go through the
// compiler's atomics so that the race detector of the ThreadSanitizer build knows them for what they are
#define __HIP_MEMORY_SCOPE_AGENT 0
template <class T> inline T emu_atomic_load(const T *p) { T v; __atomic_load(p, &v, __ATOMIC_RELAXED); return v; }
template <class T> inline void emu_atomic_store(T *p, T v) { __atomic_store(p, &v, __ATOMIC_RELAXED); }
template <class T> inline T emu_fetch_add(T *p, T v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }
#define __hip_atomic_load(p, order, scope) emu_atomic_load(p)
#define __hip_atomic_store(p, v, order, scope) emu_atomic_store(p, v)
#define __hip_atomic_fetch_add(p, v, order, scope) emu_fetch_add(p, v)

// ---- workgroup / wave barriers and fences.  The lanes of a wave run one after the other here, in lockstep on the
// device: where a wave's lanes hand data to one another through LDS without a workgroup barrier, the sources mark the
// point with a wave barrier, and the emulation makes it a rendezvous of the wave's lanes.
inline void emu_wave_sync() { (void)emu::wave_exchange(0u, emu::lane_id()); }
#define __builtin_amdgcn_s_barrier() emu::sync_threads()
#define __builtin_amdgcn_wave_barrier() emu_wave_sync()
#define __builtin_amdgcn_fence(order, scope) ((void)0)
#define __builtin_amdgcn_sched_barrier(mask) ((void)0)
inline void __threadfence() {}

// ---- matrix-core operations: the 64 lanes deposit their A and B registers, each lane then works out its own part of D.
// v_mfma_i32_16x16x32_i8: lane l holds A[l % 16][8 (l / 16) .. +7] and B[8 (l / 16) .. +7][l % 16] as eight int8;
// D register r of lane l is D[4 (l / 16) + r][l % 16].
typedef int emu_i32x4 __attribute__((ext_vector_type(4)));
typedef float emu_f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 emu_f16x8 __attribute__((ext_vector_type(8)));
inline emu_i32x4 emu_mfma_i32_16x16x32_i8(long a, long b, emu_i32x4 c) {
    struct { long a, b; } mine{ a, b };
    const auto *all = static_cast<const decltype(mine) *>(emu::wave_gather(&mine, sizeof mine));
    const int l = emu::lane_id(), col = l % 16;
    for (int r = 0; r < 4; r++) {
        const int row = 4 * (l / 16) + r;
        int acc = c[r];
        for (int kb = 0; kb < 4; kb++) {
            const long av = all[16 * kb + row].a, bv = all[16 * kb + col].b;
            for (int j = 0; j < 8; j++) acc += (int)(int8_t)(av >> (8 * j)) * (int)(int8_t)(bv >> (8 * j));
        }
        c[r] = acc;
    }
    return c;
}
#define __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, c, cbsz, abid, blgp) emu_mfma_i32_16x16x32_i8(a, b, c)
// v_mfma_f32_32x32x16_f16: lane l holds A[l % 32][8 (l / 32) .. +7] and B[8 (l / 32) .. +7][l % 32] as eight halves;
// D register r of lane l is D[8 (r / 4) + 4 (l / 32) + r % 4][l % 32].  Products are exact in f32; the sum is taken in
// double and rounded once (the hardware's own order of additions is not specified).
inline emu_f32x16 emu_mfma_f32_32x32x16_f16(emu_f16x8 a, emu_f16x8 b, emu_f32x16 c) {
    struct { emu_f16x8 a, b; } mine{ a, b };
    const auto *all = static_cast<const decltype(mine) *>(emu::wave_gather(&mine, sizeof mine));
    const int l = emu::lane_id(), col = l % 32;
    for (int r = 0; r < 16; r++) {
        const int row = 8 * (r / 4) + 4 * (l / 32) + r % 4;
        double acc = c[r];
        for (int kb = 0; kb < 2; kb++)
            for (int j = 0; j < 8; j++) acc += (double)((float)all[32 * kb + row].a[j] * (float)all[32 * kb + col].b[j]);
        c[r] = (float)acc;
    }
    return c;
}
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, cbsz, abid, blgp) emu_mfma_f32_32x32x16_f16(a, b, c)

// v_mfma_f32_32x32x2f32: lane l holds A[l % 32][l / 32] and B[l / 32][l % 32]; D as for the other 32 x 32 shapes
inline emu_f32x16 emu_mfma_f32_32x32x2f32(float a, float b, emu_f32x16 c) {
    struct { float a, b; } mine{ a, b };
    const auto *all = static_cast<const decltype(mine) *>(emu::wave_gather(&mine, sizeof mine));
    const int l = emu::lane_id(), col = l % 32;
    for (int r = 0; r < 16; r++) {
        const int row = 8 * (r / 4) + 4 * (l / 32) + r % 4;
        float acc = c[r];
        for (int kb = 0; kb < 2; kb++) acc = fmaf(all[32 * kb + row].a, all[32 * kb + col].b, acc);
        c[r] = acc;
    }
    return c;
}
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, cbsz, abid, blgp) emu_mfma_f32_32x32x2f32(a, b, c)

// ---- LDS by 32-bit address (hand-written LDS traffic) and loads that land in LDS: addresses are the low half of the
// host address of the launch-sized LDS buffer, and every access is checked against that buffer
inline char *emu_lds_at(uint32_t addr, size_t bytes) {
    char *base = static_cast<char *>(emu::dyn_lds());
    const uintptr_t host = ((uintptr_t)base & ~(uintptr_t)0xFFFFFFFFu) | addr;
    if (host < (uintptr_t)base || host + bytes > (uintptr_t)base + emu::dyn_lds_bytes()) {
        fprintf(stderr, "emu: LDS access of %zu bytes at offset %ld outside the launch's %zu bytes\n", bytes, (long)(host - (uintptr_t)base), emu::dyn_lds_bytes());
        abort();
    }
    return reinterpret_cast<char *>(host);
}
inline void emu_global_load_lds(const void *g, void *lds_wave_base, unsigned size, unsigned offset) {
    char *dst = static_cast<char *>(lds_wave_base) + offset + (size_t)emu::lane_id() * size;     // lanes land side by side
    char *base = static_cast<char *>(emu::dyn_lds());
    if (dst < base || dst + size > base + emu::dyn_lds_bytes()) { fprintf(stderr, "emu: load-to-LDS outside the launch's LDS\n"); abort(); }
    memcpy(dst, g, size);
}
#define __builtin_amdgcn_global_load_lds(g, l, size, offset, aux) emu_global_load_lds((const void *)(g), (void *)(l), size, offset)

// ---- inline assembly of the sources, rewritten by tests/emu/build_emulated.py into emu_asm(template, operands...):
// outputs first, then inputs, as the template numbers them
struct emu_operand {
    void *out;                     // where an output goes (null for an input)
    alignas(16) char value[16];    // an input's value
    size_t size;
};
template <class T> inline emu_operand emu_out(T &v) { emu_operand o{ &v, {}, sizeof(T) }; memcpy(o.value, &v, sizeof(T) < 16 ? sizeof(T) : 16); return o; }
template <class T> inline emu_operand emu_in(const T &v) { static_assert(sizeof(T) <= 16, ""); emu_operand o{ nullptr, {}, sizeof(T) }; memcpy(o.value, &v, sizeof(T)); return o; }
inline uint64_t emu_u64(const emu_operand &o) { uint64_t v = 0; memcpy(&v, o.value, o.size < 8 ? o.size : 8); return v; }
inline void emu_asm_run(const char *t, emu_operand *op, int n) {
    auto is = [&](const char *m) { return strncmp(t, m, strlen(m)) == 0; };
    if (t[0] == 0) return;                                                                        // a register pin
    if (is("global_load_dwordx4")) { memcpy(op[0].out, (const void *)emu_u64(op[1]), 16); return; }
    if (is("global_load_ushort")) { uint16_t h; memcpy(&h, (const void *)emu_u64(op[1]), 2); uint32_t w = h; memcpy(op[0].out, &w, 4); return; }
    // hand-written LDS traffic: a wave's LDS instructions execute in order for all its lanes at once, and the sources rely
    // on that (a wave writes a tile and reads it back transposed with no barrier between), so each one is a rendezvous
    if (is("ds_")) emu_wave_sync();
    if (is("ds_read_b128")) { memcpy(op[0].out, emu_lds_at((uint32_t)emu_u64(op[1]) + (uint32_t)emu_u64(op[2]), 16), 16); return; }
    if (is("ds_read_b32")) { memcpy(op[0].out, emu_lds_at((uint32_t)emu_u64(op[1]) + (uint32_t)emu_u64(op[2]), 4), 4); return; }
    if (is("ds_write_b128")) { memcpy(emu_lds_at((uint32_t)emu_u64(op[0]) + (uint32_t)emu_u64(op[2]), 16), op[1].value, 16); return; }
    if (is("ds_write_b32")) { memcpy(emu_lds_at((uint32_t)emu_u64(op[0]) + (uint32_t)emu_u64(op[2]), 4), op[1].value, 4); return; }
    if (is("v_and_or_b32")) { uint32_t r = ((uint32_t)emu_u64(op[1]) & (uint32_t)emu_u64(op[2])) | (uint32_t)emu_u64(op[3]); memcpy(op[0].out, &r, 4); return; }
    if (is("v_mov_b32")) { const char *c = strrchr(t, ','); uint32_t r = (uint32_t)strtoul(c + 1, nullptr, 0); memcpy(op[0].out, &r, 4); return; }
    fprintf(stderr, "emu: no emulation of the instruction \"%s\" (%d operands)\n", t, n);
    abort();
}
template <class... Ops> inline void emu_asm(const char *t, Ops... ops) {
    emu_operand op[sizeof...(Ops) + 1] = { ops... };
    emu_asm_run(t, op, (int)sizeof...(Ops));
}
