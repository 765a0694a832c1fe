// The two activation-side products of the counter layer on the gfx950 fp32 matrix cores, with
// the ternary weight decoded from the packed state on its way into LDS, so that no dense
// [out,in] weight exists (kernels/vulkan/counter_forward_f32_rb4.comp and
// counter_backward_input_f32_rb4.comp do the same with a 32x32 register-blocked tile):
//
//   forward         y[r,o]      = sum_i x[r,i]        * (scale[o] * t[o,i])
//   backward_input  grad_x[r,i] = sum_o grad_out[r,o] * (scale[o] * t[o,i])
//
// Both are c[m,n] = sum_k a[m,k] * w(n,k) with the activation a stored k-contiguous.  The
// operand shape of v_mfma_f32_32x32x2_f32 is "lane l holds element (row l%32, k = l/32)", so the
// activation tile is staged in LDS as [m][k] with a row stride of 33 floats: the 32 lanes of a
// half-wave then read 32 different banks, and the 4-byte writes of the staging pass spread two
// per bank, which is the minimum for 64 lanes.  The weight tile is decoded by the thread that
// fetched its packed group (one unaligned 4-byte load per group of 4 weights):
//   forward         w(n = o, k = i): [n][k] rows of 33 floats, like the activation
//   backward_input  w(n = i, k = o): the 4 weights of a group are consecutive in n, so the tile is
//                   [k][n] and takes one 16-byte LDS write per group
// A workgroup of 4 waves (2 x 2) owns a BM x BN tile of c; the next slab's activations and
// packed groups are fetched into registers while the current slab is multiplied.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "counter_math.hpp"
#include "gemm_tile.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

constexpr int kSlab = 32;           // k per LDS slab
constexpr int kLdK = kSlab + 1;     // row stride of a [rows][k] tile

template <int BM, int BN, bool FORWARD>
struct LinCfg {
    static constexpr int kWaveM = BM / 2, kWaveN = BN / 2;
    static constexpr int kTilesM = kWaveM / 32, kTilesN = kWaveN / 32;
    static constexpr int kA4 = BM * kSlab / 4 / kGemmThreads;      // float4 of activation per thread and slab
    static constexpr int kGroups = BN * kSlab / 4 / kGemmThreads;  // packed groups per thread and slab
    static constexpr int kLdN = BN + 4;                            // row stride of the [k][n] weight tile
    static constexpr int kLdsA = BM * kLdK;
    static constexpr int kLdsB = FORWARD ? BN * kLdK : kSlab * kLdN;
};

struct LinArgs {
    const float* act;      // [rows, K]
    const uint8_t* state;  // packed [out, in/4 * 3]
    const float* scale;    // [out]
    float* c;              // [rows, N]
    Codec cd;
    int rows, in_features, out_features;
};

// Packed group `group` of the state, or 0 (which decodes to t = -1 and is multiplied by a zero
// scale) when `valid` is false.  The tensor's last group has no byte after it and is read
// bytewise.
__device__ __forceinline__ uint32_t fetch_group(const uint8_t* state, size_t group, size_t last_group, bool valid) {
    if (!valid) return 0u;
    const uint8_t* p = state + 3 * group;
    if (group == last_group) return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
    uint32_t w;
    __builtin_memcpy(&w, p, 4);
    return w;
}

template <int BM, int BN, bool FORWARD, bool VEC_A>
__global__ __launch_bounds__(kGemmThreads) void counter_linear_kernel(LinArgs a) {
    using Cfg = LinCfg<BM, BN, FORWARD>;
    __shared__ float lds_a[Cfg::kLdsA];
    __shared__ float lds_b[Cfg::kLdsB];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int wm0 = (wave >> 1) * Cfg::kWaveM, wn0 = (wave & 1) * Cfg::kWaveN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int K = FORWARD ? a.in_features : a.out_features;
    const int N = FORWARD ? a.out_features : a.in_features;
    const int gpr = a.in_features >> 2;
    const size_t last_group = (size_t)a.out_features * gpr - 1;

    floatx16 acc[Cfg::kTilesM][Cfg::kTilesN];
#pragma unroll
    for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::kTilesN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    float4 ra[Cfg::kA4];
    uint32_t rw[Cfg::kGroups];
    float rs[Cfg::kGroups];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int p = 0; p < Cfg::kA4; ++p) {
            const int idx = tid + kGemmThreads * p;
            const int row = idx / (kSlab / 4), c4 = idx % (kSlab / 4);
            // load4 takes (row, col, rows, cols) of a row-major matrix
            ra[p] = load4<VEC_A>(a.act, m0 + row, k0 + 4 * c4, a.rows, K);
        }
#pragma unroll
        for (int p = 0; p < Cfg::kGroups; ++p) {
            const int idx = tid + kGemmThreads * p;
            int o, g;  // output row and group-in-row of this thread's packed group
            if (FORWARD) {
                o = n0 + idx / (kSlab / 4);
                g = (k0 >> 2) + idx % (kSlab / 4);
            } else {
                o = k0 + idx / (BN / 4);
                g = (n0 >> 2) + idx % (BN / 4);
            }
            const bool valid = o < a.out_features && g < gpr;
            rw[p] = fetch_group(a.state, (size_t)o * gpr + g, last_group, valid);
            rs[p] = valid ? a.scale[o] : 0.0f;
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int p = 0; p < Cfg::kA4; ++p) {
            const int idx = tid + kGemmThreads * p;
            const int row = idx / (kSlab / 4), c4 = idx % (kSlab / 4);
            float* dst = &lds_a[row * kLdK + 4 * c4];
            dst[0] = ra[p].x;
            dst[1] = ra[p].y;
            dst[2] = ra[p].z;
            dst[3] = ra[p].w;
        }
#pragma unroll
        for (int p = 0; p < Cfg::kGroups; ++p) {
            const int idx = tid + kGemmThreads * p;
            float w[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) w[k] = rs[p] * (float)(code_q(code_of(rw[p], k), a.cd) - 1);
            if (FORWARD) {
                float* dst = &lds_b[(idx / (kSlab / 4)) * kLdK + 4 * (idx % (kSlab / 4))];
                dst[0] = w[0];
                dst[1] = w[1];
                dst[2] = w[2];
                dst[3] = w[3];
            } else {
                float* dst = &lds_b[(idx / (BN / 4)) * Cfg::kLdN + 4 * (idx % (BN / 4))];
                *reinterpret_cast<float4*>(dst) = make_float4(w[0], w[1], w[2], w[3]);
            }
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += kSlab) {
        stage();
        __syncthreads();
        if (k0 + kSlab < K) fetch(k0 + kSlab);
#pragma unroll
        for (int kk = 0; kk < kSlab / 2; ++kk) {
            const int kcol = 2 * kk + half;
            float fa[Cfg::kTilesM], fb[Cfg::kTilesN];
#pragma unroll
            for (int i = 0; i < Cfg::kTilesM; ++i) fa[i] = lds_a[(wm0 + 32 * i + l32) * kLdK + kcol];
#pragma unroll
            for (int j = 0; j < Cfg::kTilesN; ++j)
                fb[j] = FORWARD ? lds_b[(wn0 + 32 * j + l32) * kLdK + kcol]
                                : lds_b[kcol * Cfg::kLdN + wn0 + 32 * j + l32];
#pragma unroll
            for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
                for (int j = 0; j < Cfg::kTilesN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::kTilesN; ++j) {
            const int col = n0 + wn0 + 32 * j + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + 32 * i + 8 * (r / 4) + 4 * half + (r % 4);
                if (row < a.rows && col < N) a.c[(size_t)row * N + col] = acc[i][j][r];
            }
        }
}

template <int BM, int BN, bool FORWARD>
hipError_t launch_tile(hipStream_t stream, const LinArgs& a, int N, int K) {
    const dim3 grid((N + BN - 1) / BN, (a.rows + BM - 1) / BM);
    const bool vec_a = (K % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.act) & 15u) == 0);
    if (vec_a)
        hipLaunchKernelGGL((counter_linear_kernel<BM, BN, FORWARD, true>), grid, dim3(kGemmThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((counter_linear_kernel<BM, BN, FORWARD, false>), grid, dim3(kGemmThreads), 0, stream, a);
    return hipGetLastError();
}

template <bool FORWARD>
hipError_t launch_linear(hipStream_t stream, const float* act, const uint8_t* state, const float* scale, float* c,
                         int C, int rows, int in_features, int out_features) {
    LinArgs a;
    a.act = act;
    a.state = state;
    a.scale = scale;
    a.c = c;
    a.cd = make_codec(C);
    a.rows = rows;
    a.in_features = in_features;
    a.out_features = out_features;
    const int N = FORWARD ? out_features : in_features;
    const int K = FORWARD ? in_features : out_features;
    const long tiles128 = (long)((rows + 127) / 128) * ((N + 127) / 128);
    if (tiles128 >= 128) return launch_tile<128, 128, FORWARD>(stream, a, N, K);
    return launch_tile<64, 64, FORWARD>(stream, a, N, K);
}

}  // namespace

hipError_t launch_forward(hipStream_t stream, const float* x, const uint8_t* state, const float* scale, float* y,
                          int C, int batch, int in_features, int out_features) {
    return launch_linear<true>(stream, x, state, scale, y, C, batch, in_features, out_features);
}

hipError_t launch_backward_input(hipStream_t stream, const float* grad_out, const uint8_t* state,
                                 const float* scale, float* grad_x, int C, int batch, int in_features,
                                 int out_features) {
    return launch_linear<false>(stream, grad_out, state, scale, grad_x, C, batch, in_features, out_features);
}

}  // namespace mcc
