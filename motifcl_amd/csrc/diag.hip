// Measurement and test aids declared in include/motifcl_amd_diag.h: the shader-clock probe
// and the spin limit of the strip step's bounded waits.  Not part of the drop-in boundary.
//
// The probe measures the shader clock while other kernels run.  One wave sleeps for a given
// stretch of the constant-rate wall clock and reads the shader cycle counter at both ends;
// launched on a side stream beside the kernels under test it shares their clock domain, so
// cycles / wall time is the frequency those kernels actually ran at.  Matrix-core peaks are
// quoted at the maximum engine clock; under a heavy matrix load the power limit holds the clock
// below it.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/motifcl_amd.h"
#include "../../include/motifcl_amd_diag.h"
#include "launch.hpp"

namespace {

__global__ __launch_bounds__(64) void clock_probe_kernel(unsigned long long* out, unsigned long long wall_ticks) {
    const unsigned long long w0 = wall_clock64();
    const unsigned long long c0 = clock64();
    unsigned long long w = w0;
    // ends when the wall clock has advanced by wall_ticks (bounded by the host)
    while (w - w0 < wall_ticks) {
        __builtin_amdgcn_s_sleep(100);
        w = wall_clock64();
    }
    const unsigned long long c1 = clock64();
    if (threadIdx.x == 0) {
        out[0] = w - w0;
        out[1] = c1 - c0;
    }
}

}  // namespace

extern "C" {

void mcc_compact_counter_fused_strip_set_spin_limit(unsigned spins) { mcc::set_fused_strip_spin_limit(spins); }

int mcc_wall_clock_khz(int* khz) {
    if (!khz) return mcc::report_failure(MCC_E_INVALID, "wall_clock_khz received a null pointer");
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(khz, hipDeviceAttributeWallClockRate, dev);
    if (e != hipSuccess) return mcc::report_hip_failure(e, "wall_clock_khz query failed");
    return MCC_OK;
}

int mcc_clock_probe(void* stream, uint64_t* out, size_t out_nbytes, double seconds) {
    if (!out || out_nbytes < 2 * sizeof(uint64_t))
        return mcc::report_failure(MCC_E_INVALID, "clock_probe needs a 16-byte device buffer");
    if (!(seconds > 0.0) || seconds > 2.0)
        return mcc::report_failure(MCC_E_INVALID, "clock_probe duration must be in (0, 2] seconds");
    int khz = 0;
    const int rc = mcc_wall_clock_khz(&khz);
    if (rc != MCC_OK) return rc;
    const unsigned long long ticks = (unsigned long long)(seconds * 1e3 * (double)khz);
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<unsigned long long*>(out), ticks);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mcc::report_hip_failure(e, "clock_probe launch failed");
    return MCC_OK;
}

}  // extern "C"
