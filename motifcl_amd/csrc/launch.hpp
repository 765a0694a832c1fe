// Internal launch functions behind the C ABI.  Arguments arrive validated.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace mcc {

hipError_t launch_update_dense(hipStream_t stream, uint8_t* state, float* scale, float* v,
                               const float* grad_w, int C, int in_features, int out_features,
                               float lr, float lr_scale, float rms_beta, float rms_eps,
                               uint32_t seed);

// c[m,n] = a[k,m]^T . b[k,n]
hipError_t launch_gemm_tn_f32(hipStream_t stream, const float* a, const float* b, float* c,
                              int k, int m, int n);

hipError_t launch_decode_weight(hipStream_t stream, const uint8_t* state, const float* scale,
                                float* weight, int C, int in_features, int out_features);

// y[batch,out] = x[batch,in] . W(state)^T
hipError_t launch_forward(hipStream_t stream, const float* x, const uint8_t* state,
                          const float* scale, float* y, int C, int batch, int in_features,
                          int out_features);

// grad_x[batch,in] = grad_out[batch,out] . W(state)
hipError_t launch_backward_input(hipStream_t stream, const float* grad_out, const uint8_t* state,
                                 const float* scale, float* grad_x, int C, int batch,
                                 int in_features, int out_features);

}  // namespace mcc
