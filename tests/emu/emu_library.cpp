// The one translation unit of the emulated library that holds the fiber runtime and the state of the stand-in host API
// (tests/emu/build_emulated.py compiles it beside the library's own sources).  TEST INFRASTRUCTURE.
#include "emu_fibers.h"

#include <map>
#include <mutex>

namespace emu {
hipError_t &last_error() {
    static hipError_t e = hipSuccess;
    return e;
}
bool trace_launches() {
    static const bool on = getenv("EMU_TRACE_LAUNCHES") != nullptr;
    return on;
}
}  // namespace emu

// ---- device memory
static std::mutex g_mem_mu;
static std::map<void *, size_t> g_mem;
static size_t g_mem_bytes = 0;
hipError_t hipMalloc(void **p, size_t n) {
    std::lock_guard<std::mutex> lock(g_mem_mu);
    *p = nullptr;
    if (n > kEmuDeviceBytes - g_mem_bytes) return hipErrorOutOfMemory;
    // 256-byte aligned like the device allocator's blocks (the launchers check the alignment of workspaces), exact size
    if (posix_memalign(p, 256, n ? n : 1) != 0) { *p = nullptr; return hipErrorOutOfMemory; }
    memset(*p, 0xFF, n ? n : 1);      // undefined on the device; NaN patterns here, so that a read of it does not pass by luck
    g_mem[*p] = n;
    g_mem_bytes += n;
    return hipSuccess;
}
hipError_t hipFree(void *p) {
    if (!p) return hipSuccess;
    std::lock_guard<std::mutex> lock(g_mem_mu);
    auto it = g_mem.find(p);
    if (it == g_mem.end()) return hipErrorInvalidValue;      // not a device allocation (or freed twice)
    g_mem_bytes -= it->second;
    g_mem.erase(it);
    free(p);
    return hipSuccess;
}

// Whether [p, p + n) lies inside one live device allocation (the buffer loads of the stand-in header ask).
extern "C" int emu_device_owns(const void *p, size_t n) {
    std::lock_guard<std::mutex> lock(g_mem_mu);
    auto it = g_mem.upper_bound(const_cast<void *>(p));
    if (it == g_mem.begin()) return 0;
    --it;
    const char *b = static_cast<const char *>(it->first);
    return static_cast<const char *>(p) + n <= b + it->second;
}

// ---- streams and captured graphs
struct emu_graph { std::vector<std::function<void()>> work; };
struct emu_graph_exec { std::vector<std::function<void()>> work; };
static std::map<hipStream_t, emu_graph *> g_capturing;
namespace emu {
bool submit(hipStream_t s, std::function<void()> work) {
    auto it = g_capturing.find(s);
    if (it != g_capturing.end()) { it->second->work.push_back(std::move(work)); return true; }
    work();
    return false;
}
}  // namespace emu
hipError_t hipStreamBeginCapture(hipStream_t s, int) {
    if (g_capturing.count(s)) return hipErrorInvalidValue;
    g_capturing[s] = new emu_graph();
    return hipSuccess;
}
hipError_t hipStreamEndCapture(hipStream_t s, hipGraph_t *g) {
    auto it = g_capturing.find(s);
    if (it == g_capturing.end()) return hipErrorInvalidValue;
    *g = it->second;
    g_capturing.erase(it);
    return hipSuccess;
}
hipError_t hipGraphInstantiate(hipGraphExec_t *e, hipGraph_t g, void *, void *, size_t) {
    if (!g) return hipErrorInvalidValue;
    *e = new emu_graph_exec{ g->work };
    return hipSuccess;
}
hipError_t hipGraphLaunch(hipGraphExec_t e, hipStream_t) {
    if (!e) return hipErrorInvalidValue;
    for (auto &w : e->work) w();
    return hipSuccess;
}
hipError_t hipGraphDestroy(hipGraph_t g) { delete g; return hipSuccess; }
hipError_t hipGraphExecDestroy(hipGraphExec_t e) { delete e; return hipSuccess; }
