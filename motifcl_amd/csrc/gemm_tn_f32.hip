// Weight-gradient contraction on the gfx950 fp32 matrix cores:
//     c[m,n] = sum_k a[k,m] * b[k,n]        (a = grad_out [tokens,out], b = x [tokens,in])
// The main loop lives in gemm_tile.hpp; this file adds the store epilogue and the launch.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "gemm_tile.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

template <int BM, int BN, bool VEC_A, bool VEC_B>
__global__ __launch_bounds__(kGemmThreads) void gemm_tn_kernel(const float* __restrict__ a,
                                                                const float* __restrict__ b,
                                                                float* __restrict__ c, int K, int M, int N) {
    using Cfg = TileCfg<BM, BN>;
    __shared__ float lds[Cfg::kLdsFloats];
    const TilePos tp = tile_pos<BM, BN>();
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * BN;
    floatx16 acc[Cfg::kTilesM][Cfg::kTilesN];
    gemm_tile_mainloop<BM, BN, VEC_A, VEC_B>(a, b, K, M, N, m0, n0, tp, lds, acc);
#pragma unroll
    for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::kTilesN; ++j) {
            const int col = n0 + tp.wn0 + 32 * j + tp.l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + tp.wm0 + 32 * i + 8 * (r / 4) + 4 * tp.half + (r % 4);
                if (row < M && col < N) c[(size_t)row * N + col] = acc[i][j][r];
            }
        }
}

template <int BM, int BN>
hipError_t launch_tile(hipStream_t stream, const float* a, const float* b, float* c, int k, int m, int n) {
    const dim3 grid((n + BN - 1) / BN, (m + BM - 1) / BM);
    const bool vec_a = (m % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15u) == 0);
    const bool vec_b = (n % 4 == 0) && ((reinterpret_cast<uintptr_t>(b) & 15u) == 0);
    if (vec_a && vec_b)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, true, true>), grid, dim3(kGemmThreads), 0, stream, a, b, c, k, m, n);
    else if (vec_b)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, false, true>), grid, dim3(kGemmThreads), 0, stream, a, b, c, k, m, n);
    else
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, false, false>), grid, dim3(kGemmThreads), 0, stream, a, b, c, k, m, n);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_tn_f32(hipStream_t stream, const float* a, const float* b, float* c, int k, int m, int n) {
    const long tiles128 = (long)((m + 127) / 128) * ((n + 127) / 128);
    if (tiles128 >= 128) return launch_tile<128, 128>(stream, a, b, c, k, m, n);
    return launch_tile<64, 64>(stream, a, b, c, k, m, n);
}

}  // namespace mcc
