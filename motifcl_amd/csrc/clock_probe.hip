// Measures the shader clock while other kernels run.  One wave sleeps for a given stretch of the
// constant-rate wall clock and reads the shader cycle counter at both ends; launched on a side
// stream beside the kernels under test it shares their clock domain, so cycles / wall time is
// the frequency those kernels actually ran at.  Matrix-core peaks are quoted at the maximum
// engine clock; under a heavy matrix load the power limit holds the clock below it.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "launch.hpp"

namespace mcc {
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

hipError_t launch_clock_probe(hipStream_t stream, unsigned long long* out, unsigned long long wall_ticks) {
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, stream, out, wall_ticks);
    return hipGetLastError();
}

}  // namespace mcc
