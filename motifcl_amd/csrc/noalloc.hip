// The fused step for callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc): the workspace the fused step needs is a
// file-scope device array of this library instead of a buffer lent by the caller.
//
// Every GPU the library runs on holds its own copy of the array at its own address, from the
// first use of the library on that GPU until the process ends.  In host code the array's name is
// only a handle for hipGetSymbolAddress: the device address is looked up once per device, with
// that device current, and everything that touches the array's memory (kernel arguments) uses
// that address.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>
#include <string>

#include "../../include/motifcl_amd.h"
#include "launch.hpp"

namespace {

constexpr size_t kScratchBytes = MCC_NOALLOC_WORKSPACE_NBYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_mu;
void* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each device, once resolved

// Device address of the scratch array on the current device (nullptr on failure, message stored).
void* scratch_on_current_device() {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        mcc::report_hip_failure(e, "compact-counter fused update (static workspace): hipGetDevice failed");
        return nullptr;
    }
    if (device < 0 || device >= kMaxDevices) {
        mcc::report_failure(MCC_E_RUNTIME, "compact-counter fused update (static workspace): device index out of range");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_scratch_ptr[device]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            mcc::report_hip_failure(e, "compact-counter fused update (static workspace): hipGetSymbolAddress failed");
            return nullptr;
        }
        g_scratch_ptr[device] = ptr;
    }
    return g_scratch_ptr[device];
}

}  // namespace

extern "C" {

int mcc_compact_counter_apply_update_fused_static(void* stream, uint8_t* state, size_t state_nbytes, float* scale,
                                                  size_t scale_nbytes, float* v, size_t v_nbytes,
                                                  const float* grad_out, size_t grad_out_nbytes, const float* x,
                                                  size_t x_nbytes, size_t C, size_t in_features, size_t out_features,
                                                  size_t batch, float lr, float lr_scale, float rms_beta,
                                                  float rms_eps, uint32_t seed) {
    // which workspace the shape gets: the full one (contraction into f32[out,in] slices, then the
    // update kernel) when it fits the array, else the strip workspace when the shape and the
    // hyper-parameters allow the strip path and that fits
    const size_t full = mcc_compact_counter_fused_workspace_nbytes(in_features, out_features, batch);
    const size_t strip = mcc_compact_counter_fused_strip_workspace_nbytes(in_features, out_features, batch);
    size_t use = 0;
    if (full != 0 && full <= kScratchBytes)
        use = full;
    else if (strip != 0 && strip <= kScratchBytes && strip < full)
        use = strip;
    if (full != 0 && use == 0)
        return mcc::report_failure(
            MCC_E_INVALID, "compact-counter fused update (static workspace): the step needs " + std::to_string(full) +
                               " bytes of workspace (" + (strip ? std::to_string(strip) + " on the strip path" : "no strip path for this shape") +
                               "), more than the library's static " + std::to_string(kScratchBytes) +
                               " bytes; use mcc_compact_counter_apply_update_fused with a workspace of your own");
    // full == 0: invalid dimensions, reported by the shared validation below with its usual message
    void* ws = scratch_on_current_device();
    if (!ws) return MCC_E_RUNTIME;
    return mcc::fused_update(stream, state, state_nbytes, scale, scale_nbytes, v, v_nbytes, grad_out, grad_out_nbytes, x,
                             x_nbytes, ws, use != 0 ? use : kScratchBytes, C, in_features, out_features, batch, lr,
                             lr_scale, rms_beta, rms_eps, seed);
}

}  // extern "C"
