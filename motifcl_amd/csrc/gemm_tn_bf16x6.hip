// Optional form of the weight-gradient contraction c[m,n] = sum_k a[k,m] * b[k,n] on the bf16
// matrix cores, with binary32 accuracy.  Both operands are split into three bf16 terms
// (bf16_split.hpp); a product a*b is then the exact sum of nine bf16 x bf16 products, each exact
// in binary32.  The three smallest (mid*lo, lo*mid, lo*lo <= 2^-24 |a b|) are dropped, which
// leaves an error per product of the size of one binary32 rounding -- what the fp32 matrix
// instruction commits anyway -- and six v_mfma_f32_32x32x16_bf16 passes:
//     hi*hi + hi*mid + mid*hi + hi*lo + lo*hi + mid*mid
// Six passes at 16 x the fp32 matrix rate per pass.  The operands are token-major ([k][m]), the
// bf16 instruction wants 8 consecutive k per lane, so a thread stages a 4-token x 4-column block
// and writes, per column and plane, the 4 tokens as one 8-byte piece of the [column][k] tile.
// Whole tiles only (m, n multiples of 128, token chunks multiples of 32, 16-byte aligned
// operands below 4 GiB); launch_gemm_tn_f32 falls back to the fp32 kernel otherwise.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "bf16_split.hpp"
#include "gemm_tile.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

__global__ __launch_bounds__(kGemmThreads, 3) void gemm_tn_bf16x6_kernel(const float* __restrict__ a,
                                                                         const float* __restrict__ b,
                                                                         float* __restrict__ c, int K, int M, int N,
                                                                         int chunk_tokens) {
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[3 * kPlaneBytes];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[3 * kPlaneBytes];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, kh = lane >> 5;
    const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
    const TileXY tile = xcd_tile(gridDim.x, gridDim.y, 8);
    const int m0 = tile.y * kT, n0 = tile.x * kT;
    const int k_begin = blockIdx.z * chunk_tokens;
    const int k_len = K - k_begin < chunk_tokens ? K - k_begin : chunk_tokens;
    c += (size_t)blockIdx.z * M * N;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // thread (kq, cq): tokens 4 kq .. 4 kq + 3 of the slab, columns 4 cq .. 4 cq + 3.  Eight
    // neighbouring lanes take neighbouring cq, so that a wave's load is eight whole 128-byte lines
    // (lanes that alternate between rows are fetched one 16-byte request at a time).
    const int kq = lane >> 3, cq = 8 * wave + (lane & 7);
    const uint32_t off_a = ((uint32_t)(k_begin + 4 * kq) * (uint32_t)M + (uint32_t)(m0 + 4 * cq)) * 4u;
    const uint32_t off_b = ((uint32_t)(k_begin + 4 * kq) * (uint32_t)N + (uint32_t)(n0 + 4 * cq)) * 4u;
    int lds_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) lds_off[j] = dealt_tile_offset(4 * cq + j, kq >> 1, kq & 1);

    float4 ra[4], rb[4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            ra[r] = *reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(a) + off_a +
                                                     4u * (uint32_t)(k0 + r) * (uint32_t)M);
            rb[r] = *reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(b) + off_b +
                                                     4u * (uint32_t)(k0 + r) * (uint32_t)N);
        }
    };
    auto stage = [&]() {
        // column j of the block: its 4 tokens are consecutive k of row 4 cq + j of the tile
        store_split(lds_a, lds_off[0], ra[0].x, ra[1].x, ra[2].x, ra[3].x);
        store_split(lds_a, lds_off[1], ra[0].y, ra[1].y, ra[2].y, ra[3].y);
        store_split(lds_a, lds_off[2], ra[0].z, ra[1].z, ra[2].z, ra[3].z);
        store_split(lds_a, lds_off[3], ra[0].w, ra[1].w, ra[2].w, ra[3].w);
        store_split(lds_b, lds_off[0], rb[0].x, rb[1].x, rb[2].x, rb[3].x);
        store_split(lds_b, lds_off[1], rb[0].y, rb[1].y, rb[2].y, rb[3].y);
        store_split(lds_b, lds_off[2], rb[0].z, rb[1].z, rb[2].z, rb[3].z);
        store_split(lds_b, lds_off[3], rb[0].w, rb[1].w, rb[2].w, rb[3].w);
    };

    fetch(0);
    for (int k0 = 0; k0 < k_len; k0 += kK) {
        stage();
        __syncthreads();
        if (k0 + kK < k_len) fetch(k0 + kK);
#pragma unroll
        for (int s = 0; s < kK / 16; ++s) {
            const int chunk = 2 * s + kh;
            bf16x8 fa[3][2], fb[3][2];
#pragma unroll
            for (int p = 0; p < 3; ++p)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    fa[p][i] = read_dealt_operand(lds_a + p * kPlaneBytes, wm0 + 32 * i + l32, chunk);
                    fb[p][i] = read_dealt_operand(lds_b + p * kPlaneBytes, wn0 + 32 * i + l32, chunk);
                }
            // smallest terms first
            constexpr int pa[6] = {1, 0, 2, 0, 1, 0};
            constexpr int pb[6] = {1, 2, 0, 1, 0, 0};
#pragma unroll
            for (int t = 0; t < 6; ++t)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[pa[t]][i], fb[pb[t]][j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn0 + 32 * j + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + 32 * i + 8 * (r / 4) + 4 * kh + (r % 4);
                c[(size_t)row * N + col] = acc[i][j][r];
            }
        }
}

}  // namespace

bool gemm_tn_bf16x6_supports(const float* a, const float* b, int k, int m, int n, const GemmTnPlan& plan) {
    return m % kT == 0 && n % kT == 0 && k % kK == 0 && (plan.splits == 1 || plan.chunk % kK == 0) &&
           (reinterpret_cast<uintptr_t>(a) & 15u) == 0 && (reinterpret_cast<uintptr_t>(b) & 15u) == 0 &&
           (uint64_t)k * (uint64_t)m * 4u < (1ull << 32) && (uint64_t)k * (uint64_t)n * 4u < (1ull << 32);
}

hipError_t launch_gemm_tn_bf16x6(hipStream_t stream, const float* a, const float* b, float* out, int k, int m, int n,
                                 const GemmTnPlan& plan) {
    const dim3 grid(n / kT, m / kT, plan.splits);
    hipLaunchKernelGGL(gemm_tn_bf16x6_kernel, grid, dim3(kGemmThreads), 0, stream, a, b, out, k, m, n, plan.chunk);
    return hipGetLastError();
}

}  // namespace mcc
