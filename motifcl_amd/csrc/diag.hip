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

// Synthetic inputs of the benchmark, generated where they are used.  Element i of stream s:
// two 24-bit uniforms from lowbias32(2i ^ lowbias32(s)) and lowbias32((2i+1) ^ lowbias32(s)),
// shifted into (0, 1), Box-Muller (cosine branch), times sigma.
__device__ __forceinline__ uint32_t lowbias32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

__global__ __launch_bounds__(256) void fill_normal_kernel(float* dst, size_t n, uint32_t stream_hash, float sigma) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint32_t lo = (uint32_t)i, hi = (uint32_t)(i >> 32);
        const uint32_t salt = stream_hash ^ lowbias32(hi + 0x9e3779b9u * hi);
        const float u1 = ((float)(lowbias32((2u * lo) ^ salt) >> 8) + 0.5f) * (1.0f / 16777216.0f);
        const float u2 = ((float)(lowbias32((2u * lo + 1u) ^ salt) >> 8) + 0.5f) * (1.0f / 16777216.0f);
        dst[i] = sigma * (sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2));
    }
}

// Packed counter state with every code uniform on [0, n_codes): group g holds codes 4g .. 4g+3.
__global__ __launch_bounds__(256) void fill_state_kernel(uint8_t* dst, size_t n_groups, uint32_t stream_hash, uint32_t n_codes) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x; g < n_groups; g += stride) {
        uint32_t word = 0;
        for (uint32_t k = 0; k < 4; ++k) {
            const uint64_t e = 4 * g + k;
            const uint32_t h = lowbias32((uint32_t)e ^ stream_hash ^ lowbias32((uint32_t)(e >> 32) * 0x85ebca6bu));
            word |= (uint32_t)(((uint64_t)h * n_codes) >> 32) << (6 * k);
        }
        dst[3 * g] = (uint8_t)word;
        dst[3 * g + 1] = (uint8_t)(word >> 8);
        dst[3 * g + 2] = (uint8_t)(word >> 16);
    }
}

}  // namespace

extern "C" {

int mcc_fill_normal_f32(void* stream, float* dst, size_t n, uint32_t stream_id, float sigma) {
    if (n == 0) return MCC_OK;
    if (!dst) return mcc::report_failure(MCC_E_INVALID, "fill_normal received a null pointer");
    uint32_t h = stream_id;
    h ^= h >> 16; h *= 0x7feb352du; h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
    const size_t want = (n + 255) / 256;
    hipLaunchKernelGGL(fill_normal_kernel, dim3((unsigned)(want < 65536 ? want : 65536)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), dst, n, h, sigma);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mcc::report_hip_failure(e, "fill_normal launch failed");
    return MCC_OK;
}

int mcc_fill_counter_state_u8(void* stream, uint8_t* dst, size_t n_groups, uint32_t stream_id, uint32_t n_codes) {
    if (n_groups == 0) return MCC_OK;
    if (!dst) return mcc::report_failure(MCC_E_INVALID, "fill_counter_state received a null pointer");
    if (n_codes == 0 || n_codes > 64) return mcc::report_failure(MCC_E_INVALID, "fill_counter_state needs 1..64 codes");
    uint32_t h = stream_id ^ 0x5bd1e995u;
    h ^= h >> 16; h *= 0x7feb352du; h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
    const size_t want = (n_groups + 255) / 256;
    hipLaunchKernelGGL(fill_state_kernel, dim3((unsigned)(want < 65536 ? want : 65536)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), dst, n_groups, h, n_codes);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mcc::report_hip_failure(e, "fill_counter_state launch failed");
    return MCC_OK;
}

void mcc_compact_counter_fused_strip_set_spin_limit(unsigned spins) { mcc::set_fused_strip_spin_limit(spins); }

void mcc_compact_counter_fused_strip_set_tile_mode(int mode, int grid_cap) {
    mcc::set_fused_strip_wide_mode(mode, grid_cap);
}

size_t mcc_compact_counter_fused_strip_workspace_nbytes_for_grid(size_t in_features, size_t out_features,
                                                                 size_t batch, int grid_cap) {
    return mcc::fused_strip_workspace_nbytes_for_grid(in_features, out_features, batch, grid_cap);
}

void mcc_contraction_spans_set_test_mode(unsigned polls, int start_first) {
    mcc::set_gemm_tn_wide_spans_test_mode(polls, start_first);
}

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
