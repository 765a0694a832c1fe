// Weight-gradient contraction on the gfx950 fp32 matrix cores:
//     c[m,n] = sum_k a[k,m] * b[k,n]        (a = grad_out [tokens,out], b = x [tokens,in])
//
// Both operands are stored token-major, which is exactly the operand shape of
// v_mfma_f32_32x32x2_f32: lane l supplies a[k0 + l/32][m0 + l%32] and
// b[k0 + l/32][n0 + l%32], i.e. 32 consecutive floats of one token row per
// half-wave.  Tiles are therefore staged into LDS in their HBM orientation
// ([k][m] and [k][n]) with 16-byte loads, and read back with conflict-free
// 4-byte reads; no transpose is ever needed.
//
// A workgroup of 4 waves (2x2) owns a BM x BN tile of c; each wave owns
// (BM/2) x (BN/2) as 32x32 MFMA tiles whose accumulators live in registers
// for the whole K loop.  The next K-slab is fetched from HBM into registers
// while the current one is being multiplied (software pipelining), so one
// LDS buffer suffices.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "launch.hpp"

namespace mcc {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kBK = 16;  // tokens per LDS slab

template <int BM, int BN>
struct TileCfg {
    static constexpr int kWaveM = BM / 2;       // rows of c per wave
    static constexpr int kWaveN = BN / 2;       // cols of c per wave
    static constexpr int kTilesM = kWaveM / 32;  // 32x32 MFMA tiles per wave along m
    static constexpr int kTilesN = kWaveN / 32;
    static constexpr int kLdA = BM + 4;  // padded LDS row strides (floats)
    static constexpr int kLdB = BN + 4;
    static constexpr int kA4 = kBK * BM / 4 / kThreads;  // float4 loads per thread per slab
    static constexpr int kB4 = kBK * BN / 4 / kThreads;
};

// One slab row segment of 4 floats, zero-filled outside the matrix.
template <bool VEC>
__device__ __forceinline__ float4 load4(const float* __restrict__ base, int row, int col, int rows,
                                        int cols) {
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row >= rows) return r;
    const float* p = base + (size_t)row * cols + col;
    if (VEC) {
        if (col + 3 < cols) return *reinterpret_cast<const float4*>(p);
    }
    if (col + 0 < cols) r.x = p[0];
    if (col + 1 < cols) r.y = p[1];
    if (col + 2 < cols) r.z = p[2];
    if (col + 3 < cols) r.w = p[3];
    return r;
}

template <int BM, int BN, bool VEC_A, bool VEC_B>
__global__ __launch_bounds__(kThreads) void gemm_tn_kernel(const float* __restrict__ a,
                                                            const float* __restrict__ b,
                                                            float* __restrict__ c, int K, int M,
                                                            int N) {
    using Cfg = TileCfg<BM, BN>;
    __shared__ float lds_a[kBK * Cfg::kLdA];
    __shared__ float lds_b[kBK * Cfg::kLdB];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int half = lane >> 5;
    const int wm0 = (wave >> 1) * Cfg::kWaveM;
    const int wn0 = (wave & 1) * Cfg::kWaveN;
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * BN;

    floatx16 acc[Cfg::kTilesM][Cfg::kTilesN];
#pragma unroll
    for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::kTilesN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    float4 ra[Cfg::kA4], rb[Cfg::kB4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int p = 0; p < Cfg::kA4; ++p) {
            const int idx = tid + kThreads * p;
            const int row = idx / (BM / 4), c4 = idx % (BM / 4);
            ra[p] = load4<VEC_A>(a, k0 + row, m0 + 4 * c4, K, M);
        }
#pragma unroll
        for (int p = 0; p < Cfg::kB4; ++p) {
            const int idx = tid + kThreads * p;
            const int row = idx / (BN / 4), c4 = idx % (BN / 4);
            rb[p] = load4<VEC_B>(b, k0 + row, n0 + 4 * c4, K, N);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int p = 0; p < Cfg::kA4; ++p) {
            const int idx = tid + kThreads * p;
            const int row = idx / (BM / 4), c4 = idx % (BM / 4);
            *reinterpret_cast<float4*>(&lds_a[row * Cfg::kLdA + 4 * c4]) = ra[p];
        }
#pragma unroll
        for (int p = 0; p < Cfg::kB4; ++p) {
            const int idx = tid + kThreads * p;
            const int row = idx / (BN / 4), c4 = idx % (BN / 4);
            *reinterpret_cast<float4*>(&lds_b[row * Cfg::kLdB + 4 * c4]) = rb[p];
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += kBK) {
        stage();
        __syncthreads();
        if (k0 + kBK < K) fetch(k0 + kBK);
#pragma unroll
        for (int kk = 0; kk < kBK / 2; ++kk) {
            float fa[Cfg::kTilesM], fb[Cfg::kTilesN];
            const int krow = 2 * kk + half;
#pragma unroll
            for (int i = 0; i < Cfg::kTilesM; ++i) fa[i] = lds_a[krow * Cfg::kLdA + wm0 + 32 * i + l32];
#pragma unroll
            for (int j = 0; j < Cfg::kTilesN; ++j) fb[j] = lds_b[krow * Cfg::kLdB + wn0 + 32 * j + l32];
#pragma unroll
            for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
                for (int j = 0; j < Cfg::kTilesN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // D layout of the 32x32 tile: lane -> column l32, register r -> row 8*(r/4) + 4*half + r%4.
#pragma unroll
    for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::kTilesN; ++j) {
            const int col = n0 + wn0 + 32 * j + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + 32 * i + 8 * (r / 4) + 4 * half + (r % 4);
                if (row < M && col < N) c[(size_t)row * N + col] = acc[i][j][r];
            }
        }
}

template <int BM, int BN>
hipError_t launch_tile(hipStream_t stream, const float* a, const float* b, float* c, int k, int m,
                       int n) {
    const dim3 grid((n + BN - 1) / BN, (m + BM - 1) / BM);
    const bool vec_a = (m % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15u) == 0);
    const bool vec_b = (n % 4 == 0) && ((reinterpret_cast<uintptr_t>(b) & 15u) == 0);
    if (vec_a && vec_b)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, true, true>), grid, dim3(kThreads), 0, stream, a, b, c, k, m, n);
    else if (vec_b)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, false, true>), grid, dim3(kThreads), 0, stream, a, b, c, k, m, n);
    else
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, false, false>), grid, dim3(kThreads), 0, stream, a, b, c, k, m, n);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_tn_f32(hipStream_t stream, const float* a, const float* b, float* c, int k,
                              int m, int n) {
    const long tiles128 = (long)((m + 127) / 128) * ((n + 127) / 128);
    if (tiles128 >= 128) return launch_tile<128, 128>(stream, a, b, c, k, m, n);
    return launch_tile<64, 64>(stream, a, b, c, k, m, n);
}

}  // namespace mcc
