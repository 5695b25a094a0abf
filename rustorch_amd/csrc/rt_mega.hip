// Host side of the persistent decode-step kernel (device code and rationale in rt_mega_device.h).
#include "rt_mega_device.h"

namespace rt {

// Number of workgroups a cooperative launch of the step kernel may use (0 when it cannot run here).
int mega_grid(int device, size_t lds_bytes) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, device) != hipSuccess) return 0;
    if (!p.cooperativeLaunch) return 0;
    if (lds_bytes > 64 * 1024 &&
        hipFuncSetAttribute((const void *)llama_step_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, llama_step_kernel, kMegaThreads, lds_bytes) != hipSuccess || per_cu < 1) {
        (void)hipGetLastError();
        return 0;
    }
    int n = p.multiProcessorCount;
    n -= n % (int)kBarGroups;
    return n;
}

hipError_t launch_llama_step(hipStream_t s, MegaArgs &a, int grid, size_t lds_bytes) {
    hipError_t e = hipMemsetAsync(a.bar, 0, kMegaBarBytes, s);
    if (e != hipSuccess) return e;
    void *args[] = { &a };
    return hipLaunchCooperativeKernel((const void *)llama_step_kernel, dim3((unsigned)grid), dim3(kMegaThreads), args, lds_bytes, s);
}

}  // namespace rt
