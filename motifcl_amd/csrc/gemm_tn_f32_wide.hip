// The weight-gradient contraction c[m,n] = sum_k a[k,m] * b[k,n] on the fp32 matrix cores with
// 256 x 256 tiles: 8 waves (2 down x 4 across, 128 x 64 each), slabs of 16 tokens copied straight
// into one of two LDS buffers (global_load_lds_dwordx4).  Against the 128 x 128 tiles of
// gemm_tn_f32.hip a workgroup copies half as many operand bytes per flop and reads 6 instead of
// 8 LDS operands per 8 MFMAs.  Every output element still accumulates its tokens in the same
// order, two at a time, so the result is the same bits.  Whole tiles and whole slabs only.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "gemm_tile.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

constexpr int kWide = 256;
constexpr int kWideThreads = 512;
constexpr int kWideSlabFloats = kBK * 2 * kWide;  // 16 tokens of both operands: 32 KiB

__global__ __launch_bounds__(kWideThreads, 2) void gemm_tn_wide_kernel(const float* __restrict__ a,
                                                                       const float* __restrict__ b,
                                                                       float* __restrict__ c, int K, int M, int N,
                                                                       int chunk) {
    __shared__ __attribute__((aligned(1024))) float lds[2 * kWideSlabFloats];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int wm0 = (wave >> 2) * 128, wn0 = (wave & 3) * 64;
    const TileXY tile = xcd_tile(gridDim.x, gridDim.y, 4);
    const int m0 = tile.y * kWide, n0 = tile.x * kWide;
    const int k_begin = blockIdx.z * chunk;
    const int k_len = K - k_begin < chunk ? K - k_begin : chunk;
    a += (size_t)k_begin * M + m0;
    b += (size_t)k_begin * N + n0;
    c += (size_t)blockIdx.z * M * N;

    floatx16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    typedef __attribute__((address_space(3))) void* lds_ptr;
    typedef const __attribute__((address_space(1))) void* global_ptr;
    // a slab is 32 rows of 1 KiB (16 token rows of a, then 16 of b); wave w copies rows w, w + 8,
    // w + 16, w + 24, lane l the floats 4 l .. 4 l + 3 of the row
    auto issue = [&](int k0, int buf) {
        float* dst = lds + buf * kWideSlabFloats;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int row = wave + 8 * p;
            __builtin_amdgcn_global_load_lds((global_ptr)(a + (size_t)(k0 + row) * M + 4 * lane),
                                             (lds_ptr)(dst + row * kWide), 16, 0, 0);
        }
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int row = wave + 8 * p;
            __builtin_amdgcn_global_load_lds((global_ptr)(b + (size_t)(k0 + row) * N + 4 * lane),
                                             (lds_ptr)(dst + (kBK + row) * kWide), 16, 0, 0);
        }
    };
    issue(0, 0);
    int buf = 0;
    for (int k0 = 0; k0 < k_len; k0 += kBK) {
        __builtin_amdgcn_s_waitcnt(0);  // this wave's part of the slab has landed
        __syncthreads();                // ... and everybody else's; the other buffer is free
        if (k0 + kBK < k_len) issue(k0 + kBK, buf ^ 1);
        const float* lds_a = lds + buf * kWideSlabFloats;
        const float* lds_b = lds_a + kBK * kWide;
        // Operand reads run four steps ahead of the MFMAs that use them: while the next slab is
        // being copied into LDS a read can take several times its usual latency, and with reads
        // issued just in time the matrix pipe waits for them (one step ahead: 89.0 % of the peak on
        // 4096 x 4096, two: 89.8 %, four: 90.3 %, six: 89.9 %).
        constexpr int D = 4;
        float fa[D + 1][4], fb[D + 1][2];
        auto load = [&](int kk, int set) {
            const int krow = 2 * kk + half;
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[set][i] = lds_a[krow * kWide + wm0 + 32 * i + l32];
#pragma unroll
            for (int j = 0; j < 2; ++j) fb[set][j] = lds_b[krow * kWide + wn0 + 32 * j + l32];
        };
#pragma unroll
        for (int q = 0; q < D; ++q) load(q, q);
#pragma unroll
        for (int kk = 0; kk < kBK / 2; ++kk) {
            if (kk + D < kBK / 2) load(kk + D, (kk + D) % (D + 1));
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[kk % (D + 1)][i], fb[kk % (D + 1)][j], acc[i][j], 0, 0, 0);
            if (kk + D < kBK / 2) __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
        }
        buf ^= 1;
    }

#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn0 + 32 * j + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + 32 * i + 8 * (r / 4) + 4 * half + (r % 4);
                c[(size_t)row * N + col] = acc[i][j][r];
            }
        }
}

}  // namespace

bool gemm_tn_wide_supports(const float* a, const float* b, int k, int m, int n, int chunk) {
    return m % kWide == 0 && n % kWide == 0 && k % kBK == 0 && chunk % kBK == 0 &&
           (reinterpret_cast<uintptr_t>(a) & 15u) == 0 && (reinterpret_cast<uintptr_t>(b) & 15u) == 0;
}

// tiles_x x tiles_y tiles starting at a, b, out; m and n are the row lengths of a / b and out
hipError_t launch_gemm_tn_wide(hipStream_t stream, const float* a, const float* b, float* out, int k, int m, int n,
                               int tiles_x, int tiles_y, int chunk, int splits) {
    const dim3 grid(tiles_x, tiles_y, splits);
    hipLaunchKernelGGL(gemm_tn_wide_kernel, grid, dim3(kWideThreads), 0, stream, a, b, out, k, m, n, chunk);
    return hipGetLastError();
}

}  // namespace mcc
