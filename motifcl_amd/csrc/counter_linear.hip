// Consumers of the packed counter state other than the update: dense decode,
// forward (y = x . W^T) and input gradient (grad_x = grad_out . W), with the
// ternary weight decoded from the packed state inside the kernel so that no
// dense [out,in] weight is materialised (kernels/compact_counter.cl:39-55,
// 248-269; kernels/vulkan/counter_forward_f32_rb4.comp).
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

constexpr int kTile = 16;

// y[r,o] = sum_i x[r,i] * (scale[o] * t[o,i]); a 16x16 block shares a tile of
// x and a tile of decoded weights through LDS.
__global__ __launch_bounds__(kTile* kTile) void forward_kernel(
    const float* __restrict__ x, const uint8_t* __restrict__ state, const float* __restrict__ scale,
    float* __restrict__ y, Codec cd, int batch, int in_features, int out_features) {
    __shared__ float xs[kTile][kTile * 4 + 1];
    __shared__ float ws[kTile][kTile * 4 + 1];
    const int tx = threadIdx.x, ty = threadIdx.y;
    const int r = blockIdx.y * kTile + ty;   // batch row of this thread's output
    const int o = blockIdx.x * kTile + tx;   // output feature
    const int gpr = in_features / 4;
    float acc = 0.0f;
    for (int g0 = 0; g0 < gpr; g0 += kTile) {
        // thread (ty,tx) loads group g0+tx of batch row (block r0 + ty) and of weight row (block o0 + ty)
        const int g = g0 + tx;
        const int wr = blockIdx.x * kTile + ty;
        float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r < batch && g < gpr) {
            const float* p = x + (size_t)r * in_features + 4 * g;
            xv = make_float4(p[0], p[1], p[2], p[3]);
        }
        float wv[4] = {0.f, 0.f, 0.f, 0.f};
        if (wr < out_features && g < gpr) {
            const uint32_t word = load_group(state + ((size_t)wr * gpr + g) * 3);
            const float s = scale[wr];
#pragma unroll
            for (int k = 0; k < 4; ++k) wv[k] = s * (float)(code_q(code_of(word, k), cd) - 1);
        }
        xs[ty][4 * tx + 0] = xv.x; xs[ty][4 * tx + 1] = xv.y;
        xs[ty][4 * tx + 2] = xv.z; xs[ty][4 * tx + 3] = xv.w;
#pragma unroll
        for (int k = 0; k < 4; ++k) ws[ty][4 * tx + k] = wv[k];
        __syncthreads();
#pragma unroll 8
        for (int i = 0; i < kTile * 4; ++i) {
            const float p = xs[ty][i] * ws[tx][i];
            acc = acc + p;
        }
        __syncthreads();
    }
    if (r < batch && o < out_features) y[(size_t)r * out_features + o] = acc;
}

// grad_x[r, 4g..4g+3] = sum_o (grad_out[r,o] * scale[o]) * t[o, 4g..4g+3], sequential in o
// exactly as kernels/compact_counter.cl:262-267.  One thread per (r, group).
__global__ void backward_input_kernel(const float* __restrict__ grad_out,
                                      const uint8_t* __restrict__ state,
                                      const float* __restrict__ scale, float* __restrict__ grad_x,
                                      Codec cd, int batch, int in_features, int out_features) {
    const int gpr = in_features / 4;
    const int g = blockIdx.x * blockDim.x + threadIdx.x;
    const int r = blockIdx.y;
    if (g >= gpr || r >= batch) return;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int o = 0; o < out_features; ++o) {
        const uint32_t word = load_group(state + ((size_t)o * gpr + g) * 3);
        const float gs = grad_out[(size_t)r * out_features + o] * scale[o];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float p = gs * (float)(code_q(code_of(word, k), cd) - 1);
            acc[k] = acc[k] + p;
        }
    }
    float* dst = grad_x + (size_t)r * in_features + 4 * g;
    dst[0] = acc[0]; dst[1] = acc[1]; dst[2] = acc[2]; dst[3] = acc[3];
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

hipError_t launch_forward(hipStream_t stream, const float* x, const uint8_t* state,
                          const float* scale, float* y, int C, int batch, int in_features,
                          int out_features) {
    const dim3 grid((out_features + kTile - 1) / kTile, (batch + kTile - 1) / kTile);
    hipLaunchKernelGGL(forward_kernel, grid, dim3(kTile, kTile), 0, stream, x, state, scale, y,
                       make_codec(C), batch, in_features, out_features);
    return hipGetLastError();
}

hipError_t launch_backward_input(hipStream_t stream, const float* grad_out, const uint8_t* state,
                                 const float* scale, float* grad_x, int C, int batch,
                                 int in_features, int out_features) {
    const int gpr = in_features / 4;
    const int block = 64;
    const dim3 grid((gpr + block - 1) / block, batch);
    hipLaunchKernelGGL(backward_input_kernel, grid, dim3(block), 0, stream, grad_out, state, scale,
                       grad_x, make_codec(C), batch, in_features, out_features);
    return hipGetLastError();
}

}  // namespace mcc
