// Self-test of the race-detecting emulation (tests/emu/emu_fibers.h under ThreadSanitizer; a wave is a thread of the
// detector).  TEST INFRASTRUCTURE.  Built twice by tests/test_emu_races.py: with RACY, wave 1 reads the LDS words wave 0
// wrote with no workgroup barrier in between, and the detector has to say so; without it the barrier is there and the
// run has to be clean.  Lanes of one wave hand words to each other without a barrier in both builds: that is lockstep
// on the device and must not be reported.
#include <cstdio>

#include <hip/hip_runtime.h>

#include "emu_fibers.h"

namespace emu {
hipError_t &last_error() {
    static hipError_t e = hipSuccess;
    return e;
}
bool trace_launches() { return false; }
}  // namespace emu

static void kernel(float *out) {
    RT_DYN_LDS(float, lds);
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (wave == 0) lds[lane] = (float)lane;
    // within the wave: lane l reads what lane 63 - l wrote (lockstep: no barrier needed, the emulation's lanes meet here)
    emu_wave_sync();
    float mine = wave == 0 ? lds[63 - lane] : 0.f;
#ifndef RACY
    __syncthreads();
#endif
    if (wave == 1) mine = lds[lane];
#ifdef RACY
    __syncthreads();
#endif
    out[tid] = mine;
}

int main() {
    static float out[128];
    const bool ok = emu::launch(1, 128, 64 * sizeof(float), [&] { kernel(out); });
    float sum = 0.f;
    for (float v : out) sum += v;
    printf("%s sum %.0f\n", ok ? "ran" : "stalled", sum);
    return ok ? 0 : 1;
}
