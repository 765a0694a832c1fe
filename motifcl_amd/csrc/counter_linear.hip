// Dense decode of the packed counter state (kernels/compact_counter.cl:39-55).  The forward
// and input-gradient products decode inside their contraction and never call this.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "counter_math.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

__device__ __forceinline__ uint32_t load_group(const uint8_t* p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
}

// One thread per packed group (kernels/compact_counter.cl:39-55).
__global__ void decode_weight_kernel(const uint8_t* __restrict__ state,
                                     const float* __restrict__ scale, float* __restrict__ w,
                                     Codec cd, int in_features, long n_groups) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= n_groups) return;
    const int gpr = in_features / 4;
    const long row = gid / gpr;
    const uint32_t word = load_group(state + gid * 3);
    const float s = scale[row];
    float4 o;
    o.x = s * (float)(code_q(code_of(word, 0), cd) - 1);
    o.y = s * (float)(code_q(code_of(word, 1), cd) - 1);
    o.z = s * (float)(code_q(code_of(word, 2), cd) - 1);
    o.w = s * (float)(code_q(code_of(word, 3), cd) - 1);
    float* dst = w + gid * 4;
    dst[0] = o.x; dst[1] = o.y; dst[2] = o.z; dst[3] = o.w;
}

}  // namespace

hipError_t launch_decode_weight(hipStream_t stream, const uint8_t* state, const float* scale,
                                float* weight, int C, int in_features, int out_features) {
    const long n_groups = (long)out_features * (in_features / 4);
    const int block = 256;
    const long grid = (n_groups + block - 1) / block;
    hipLaunchKernelGGL(decode_weight_kernel, dim3((unsigned)grid), dim3(block), 0, stream, state,
                       scale, weight, make_codec(C), in_features, n_groups);
    return hipGetLastError();
}

}  // namespace mcc
