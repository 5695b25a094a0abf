// CPU stand-in for <hip/hip_runtime.h>: enough of the HIP device vocabulary to compile the kernels of
// rustorch_amd/csrc as host C++ and run them as fibers (one per GPU thread) under AddressSanitizer.
// TEST INFRASTRUCTURE: used only by tests/emu/emu_main.cpp.
//
// Execution model: a workgroup's threads are fibers that run one after the other; a fiber runs until it
// reaches __syncthreads(), a wave operation (shuffle / DPP / readlane), a sleep inside a spin loop, or its
// end.  Workgroups take turns; a workgroup is left only when it is spinning in the grid barrier, at which
// point its LDS contents are dead, so one LDS buffer serves all workgroups.  Wave operations are executed by
// whole waves in the kernels here, so they are modelled as a 64-lane rendezvous with value exchange.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)
#define __align__(n) alignas(n)

struct uint2 { uint32_t x, y; };
struct alignas(16) uint4 { uint32_t x, y, z, w; };
struct float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
inline float2 make_float2(float x, float y) { return float2{ x, y }; }
inline float4 make_float4(float x, float y, float z, float w) { return float4{ x, y, z, w }; }
struct dim3 { unsigned x = 1, y = 1, z = 1; dim3() {} dim3(unsigned a, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {} };

typedef int hipError_t;
typedef void *hipStream_t;
typedef void *hipEvent_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2 };
inline const char *hipGetErrorString(hipError_t) { return "emu"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipSetDevice(int) { return hipSuccess; }

namespace emu {

struct Idx3 { unsigned x, y, z; };
struct Fiber;
extern Fiber *g_cur;          // the fiber that is running
Idx3 &tid();
Idx3 &bid();
Idx3 &bdim();
Idx3 &gdim();
void *dyn_lds();
void sync_threads();
void spin_yield();
// 64-lane rendezvous: every live lane of the wave deposits v; returns the value deposited by lane `src`
uint32_t wave_exchange(uint32_t v, int src);
int lane_id();

}  // namespace emu

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
inline int __float2int_rn(float f) { return (int)std::nearbyintf(f); }
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
inline void unsafeAtomicAdd(float *p, float v) { *p += v; }
// buffer resources: base pointer only (the emulation neither checks ranges nor strides), loads at base + voffset + soffset
struct emu_buffer_rsrc { const unsigned char *base; };
typedef emu_buffer_rsrc __amdgpu_buffer_rsrc_t;
typedef unsigned int emu_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int emu_u32x2 __attribute__((ext_vector_type(2)));
inline emu_buffer_rsrc emu_make_rsrc(const void *p) { return emu_buffer_rsrc{ (const unsigned char *)p }; }
inline emu_u32x4 emu_bload128(emu_buffer_rsrc r, unsigned voff, unsigned soff) { emu_u32x4 v; __builtin_memcpy(&v, r.base + voff + soff, 16); return v; }
inline emu_u32x2 emu_bload64(emu_buffer_rsrc r, unsigned voff, unsigned soff) { emu_u32x2 v; __builtin_memcpy(&v, r.base + voff + soff, 8); return v; }
inline unsigned int emu_bload32(emu_buffer_rsrc r, unsigned voff, unsigned soff) { unsigned int v; __builtin_memcpy(&v, r.base + voff + soff, 4); return v; }
inline short emu_bload16(emu_buffer_rsrc r, unsigned voff, unsigned soff) { short v; __builtin_memcpy(&v, r.base + voff + soff, 2); return v; }
#define __builtin_amdgcn_make_buffer_rsrc(p, stride, num, flags) emu_make_rsrc(p)
#define __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, aux) emu_bload128(r, voff, soff)
#define __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, aux) emu_bload64(r, voff, soff)
#define __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, aux) emu_bload32(r, voff, soff)
#define __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, aux) emu_bload16(r, voff, soff)
#define __builtin_amdgcn_s_sleep(n) emu::spin_yield()
#define __builtin_amdgcn_s_waitcnt(n) ((void)0)

// ---- device-scope atomics: fibers never run concurrently, plain accesses are exact
#define __HIP_MEMORY_SCOPE_AGENT 0
template <class T> inline T emu_atomic_load(const T *p) { return *p; }
template <class T> inline void emu_atomic_store(T *p, T v) { *p = v; }
template <class T> inline T emu_fetch_add(T *p, T v) { T o = *p; *p = o + v; return o; }
#define __hip_atomic_load(p, order, scope) emu_atomic_load(p)
#define __hip_atomic_store(p, v, order, scope) emu_atomic_store(p, v)
#define __hip_atomic_fetch_add(p, v, order, scope) emu_fetch_add(p, v)
