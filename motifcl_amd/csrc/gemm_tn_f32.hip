// Weight-gradient contraction on the gfx950 fp32 matrix cores:
//     c[m,n] = sum_k a[k,m] * b[k,n]        (a = grad_out [tokens,out], b = x [tokens,in])
// The main loop lives in gemm_tile.hpp; this file adds the store epilogue and the launch.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "gemm_tile.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

// Token chunk blockIdx.z of `chunk` tokens goes to slice blockIdx.z of `c` (slices are m*n floats
// apart); with one chunk this is the whole contraction.
template <int BM, int BN, bool VEC_A, bool VEC_B, bool DIRECT>
__global__ __launch_bounds__(kGemmThreads) void gemm_tn_kernel(const float* __restrict__ a,
                                                                const float* __restrict__ b,
                                                                float* __restrict__ c, int K, int M, int N,
                                                                int chunk) {
    using Cfg = TileCfg<BM, BN>;
    __shared__ float lds[DIRECT ? DirectCfg<BM, BN>::kLdsFloats : Cfg::kLdsFloats];
    const TilePos tp = tile_pos<BM, BN>();
    const TileXY tile = xcd_tile(gridDim.x, gridDim.y, 8);
    const int m0 = tile.y * BM;
    const int n0 = tile.x * BN;
    const int k_begin = blockIdx.z * chunk;
    const int k_len = K - k_begin < chunk ? K - k_begin : chunk;
    a += (size_t)k_begin * M;
    b += (size_t)k_begin * N;
    c += (size_t)blockIdx.z * M * N;
    floatx16 acc[Cfg::kTilesM][Cfg::kTilesN];
    if (DIRECT)
        gemm_tile_mainloop_direct<BM, BN>(a, b, k_len, M, N, m0, n0, tp, lds, acc);
    else
        gemm_tile_mainloop<BM, BN, VEC_A, VEC_B>(a, b, k_len, M, N, m0, n0, tp, lds, acc);
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

// c[e] = ((p0[e] + p1[e]) + p2[e]) + ...: the chunk sums are added in chunk order, so the result
// does not depend on scheduling.  c may be slice 0 itself.
__global__ __launch_bounds__(256) void reduce_slices_kernel(const float* __restrict__ slices, float* c, size_t mn,
                                                           int n_slices) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < mn; e += (size_t)gridDim.x * blockDim.x) {
        float acc = slices[e];
        for (int s = 1; s < n_slices; ++s) acc = acc + slices[(size_t)s * mn + e];
        c[e] = acc;
    }
}

template <int BM, int BN>
hipError_t launch_tile(hipStream_t stream, const float* a, const float* b, float* c, int k, int m, int n,
                       const GemmTnPlan& plan) {
    const dim3 grid((n + BN - 1) / BN, (m + BM - 1) / BM, plan.splits);
    // every chunk starts at a multiple of 16 tokens, so it is as aligned as the matrix itself
    const bool vec_a = (m % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15u) == 0);
    const bool vec_b = (n % 4 == 0) && ((reinterpret_cast<uintptr_t>(b) & 15u) == 0);
    // whole tiles and whole slabs (every chunk is a multiple of 16 tokens when k is): direct-to-LDS
    const bool direct = vec_a && vec_b && m % BM == 0 && n % BN == 0 && k % kBK == 0;
    if (direct)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, true, true, true>), grid, dim3(kGemmThreads), 0, stream, a, b, c, k,
                           m, n, plan.chunk);
    else if (vec_a && vec_b)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, true, true, false>), grid, dim3(kGemmThreads), 0, stream, a, b, c,
                           k, m, n, plan.chunk);
    else if (vec_b)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, false, true, false>), grid, dim3(kGemmThreads), 0, stream, a, b, c,
                           k, m, n, plan.chunk);
    else
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, false, false, false>), grid, dim3(kGemmThreads), 0, stream, a, b,
                           c, k, m, n, plan.chunk);
    return hipGetLastError();
}

}  // namespace

// How a contraction is cut up is a function of its shape alone, so that every entry point that
// contracts the same operands produces the same bits.  Output tiles are 128 x 128 when that
// gives at least 64 tiles (measured: 2048 x 768 at 16384 tokens runs 15 % faster as 96 large tiles
// in 10 chunks than as 384 small ones in 2; 768 x 768 is faster with small tiles), else 64 x 64;
// the token dimension is split into equal chunks (multiples
// of 16, at least 256 tokens) until about 1024 workgroups -- four per CU -- exist.  A layer of a
// 15M-parameter model is 25 tiles: without the split 231 of 256 CUs idle.
GemmTnPlan plan_gemm_tn(int k, int m, int n) {
    GemmTnPlan p;
    const long tiles128 = (long)((m + 127) / 128) * ((n + 127) / 128);
    p.tile = tiles128 >= 64 ? 128 : 64;
    const long tiles = (long)((m + p.tile - 1) / p.tile) * ((n + p.tile - 1) / p.tile);
    long splits = 1024 / tiles;
    const long max_splits = k / 256;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    int chunk = (int)((k + splits - 1) / splits);
    chunk = (chunk + kBK - 1) / kBK * kBK;
    p.chunk = chunk;
    p.splits = (k + chunk - 1) / chunk;
    return p;
}

size_t gemm_tn_slices(int k, int m, int n) { return (size_t)plan_gemm_tn(k, m, n).splits; }

// `slices` holds plan.splits * m * n floats when the plan splits the tokens (it may start at c);
// it is not touched otherwise.
hipError_t launch_gemm_tn_f32(hipStream_t stream, const float* a, const float* b, float* c, int k, int m, int n,
                              float* slices, int mode) {
    const GemmTnPlan plan = plan_gemm_tn(k, m, n);
    float* out = plan.splits > 1 ? slices : c;
    if (plan.splits > 1 && !slices) return hipErrorInvalidValue;
    hipError_t e;
    if (mode == 1 && gemm_tn_bf16x6_supports(a, b, k, m, n, plan))
        e = launch_gemm_tn_bf16x6(stream, a, b, out, k, m, n, plan);
    else
        e = plan.tile == 128 ? launch_tile<128, 128>(stream, a, b, out, k, m, n, plan)
                                    : launch_tile<64, 64>(stream, a, b, out, k, m, n, plan);
    if (e != hipSuccess || plan.splits == 1) return e;
    const size_t mn = (size_t)m * n;
    const size_t want = (mn + 255) / 256;
    hipLaunchKernelGGL(reduce_slices_kernel, dim3((unsigned)(want < 4096 ? want : 4096)), dim3(256), 0, stream, slices,
                       c, mn, plan.splits);
    return hipGetLastError();
}

}  // namespace mcc
