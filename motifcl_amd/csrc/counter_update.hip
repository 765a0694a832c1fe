// Update-only step of the compact-counter layer on gfx950: row statistics,
// stochastic-rounding tick and scale commit in ONE kernel, one wave64 per
// output row.
//
// Why one wave per row: the reference's row reduction
// (kernels/compact_counter.cl:75-91) is 64 strided partial sums (lane l walks
// groups l, l+64, ...) followed by a binary tree.  A wave64 whose lane l owns
// exactly those groups reproduces that order with register accumulation and a
// shuffle tree, so the per-row RMS is bit-identical and no cross-wave
// synchronisation exists.  Lane l's 16-byte gradient loads are perfectly
// coalesced (64 lanes x 16 B = 1 KiB contiguous per instruction).
//
// Why the row stays in registers: every tick needs its row's denominator,
// which needs the whole row's sum of squares first.  Holding the row (up to
// 43 groups per lane for in = 11008) in VGPRs lets HBM see the gradient once:
// 4 B (G) + 0.75 B (state read) + 0.75 B (state write) per weight.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "counter_math.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;

struct UpdateArgs {
    uint8_t* state;
    float* scale;
    float* v;
    const float* grad_w;
    Codec cd;
    int in_features, out_features, gpr;
    float lr, lr_scale, rms_beta, rms_eps;
    uint32_t seed;
};

__device__ __forceinline__ uint32_t load_group(const uint8_t* p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
}

__device__ __forceinline__ void store_group(uint8_t* p, uint32_t w) {
    p[0] = (uint8_t)(w & 0xffu);
    p[1] = (uint8_t)((w >> 8) & 0xffu);
    p[2] = (uint8_t)((w >> 16) & 0xffu);
}

__device__ __forceinline__ void accumulate(float& g_sq, float& grad_s, const float g[4], uint32_t w,
                                           const Codec& cd, bool with_gs) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float sq = g[k] * g[k];
        g_sq = g_sq + sq;
        if (with_gs) {
            const int t = code_q(code_of(w, k), cd) - 1;
            const float gt = g[k] * (float)t;
            grad_s = grad_s + gt;
        }
    }
}

__device__ __forceinline__ float tree_sum(float a) {
    // lg[lid] += lg[lid + s] for s = 32..1 (kernels/compact_counter.cl:88-91)
#pragma unroll
    for (int s = kWave / 2; s > 0; s >>= 1) a = a + __shfl_down(a, s, kWave);
    return a;
}

__device__ __forceinline__ uint32_t tick_group(uint32_t w, const float g[4], const RowConsts& rc,
                                               const UpdateArgs& a, uint32_t elem0) {
    uint32_t nw = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t nc = tick_code(code_of(w, k), g[k], rc, a.seed, elem0 + (uint32_t)k, a.cd);
        nw |= (nc & 0x3fu) << (6 * k);
    }
    return nw;
}

__device__ __forceinline__ RowConsts finish_row(const UpdateArgs& a, int row, int lane, float g_sq,
                                                float grad_s, bool with_gs) {
    g_sq = tree_sum(g_sq);
    g_sq = __shfl(g_sq, 0, kWave);
    if (with_gs) {
        grad_s = tree_sum(grad_s);
        grad_s = __shfl(grad_s, 0, kWave);
    } else {
        grad_s = 0.0f;
    }
    const float s_old = a.scale[row];
    const float v_old = a.v[row];
    const RowStats rs = finish_row_stats(g_sq, grad_s, v_old, s_old, a.in_features, a.lr_scale,
                                         a.rms_beta, a.rms_eps);
    if (lane == 0) {
        a.v[row] = rs.v_new;
        a.scale[row] = rs.scale_new;  // commit (kernels/basic.cl:6-9); s_old stays in a register
    }
    RowConsts rc;
    rc.dn = rs.denom;
    rc.k = a.cd.Cf / rs.scale_new;
    rc.ratio = s_old / rs.scale_new;
    rc.neg_lr = -a.lr;
    return rc;
}

// Register-resident rows: gpr <= 64 * ITERS.  grad_w must be 16-byte aligned.
template <int ITERS, bool WITH_GS>
__global__ __launch_bounds__(kWave* kWavesPerBlock) void update_rows_kernel(UpdateArgs a) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (row >= a.out_features) return;
    const float4* g_row = reinterpret_cast<const float4*>(a.grad_w + (size_t)row * a.in_features);
    uint8_t* s_row = a.state + (size_t)row * a.gpr * 3;

    float g[ITERS][4];
    uint32_t w[ITERS];
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
        const int gi = lane + kWave * j;
        if (gi < a.gpr) {
            const float4 q = g_row[gi];
            g[j][0] = q.x; g[j][1] = q.y; g[j][2] = q.z; g[j][3] = q.w;
            w[j] = load_group(s_row + 3 * gi);
        } else {
            g[j][0] = g[j][1] = g[j][2] = g[j][3] = 0.0f;
            w[j] = 0u;
        }
    }
    float g_sq = 0.0f, grad_s = 0.0f;
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
        // a padded group adds +0.0 (squares) and -0.0 (0 * t, t = -1): both leave the sums unchanged
        accumulate(g_sq, grad_s, g[j], w[j], a.cd, WITH_GS);
    }
    const RowConsts rc = finish_row(a, row, lane, g_sq, grad_s, WITH_GS);
    const uint32_t row_elem = (uint32_t)row * (uint32_t)a.in_features;
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
        const int gi = lane + kWave * j;
        if (gi < a.gpr) {
            const uint32_t nw = tick_group(w[j], g[j], rc, a, row_elem + 4u * (uint32_t)gi);
            store_group(s_row + 3 * gi, nw);
        }
    }
}

// Any row length, any alignment: the row is read twice (the second read hits L2).
template <bool WITH_GS>
__global__ __launch_bounds__(kWave* kWavesPerBlock) void update_rows_generic_kernel(UpdateArgs a) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (row >= a.out_features) return;
    const float* g_row = a.grad_w + (size_t)row * a.in_features;
    uint8_t* s_row = a.state + (size_t)row * a.gpr * 3;

    float g_sq = 0.0f, grad_s = 0.0f;
    for (int gi = lane; gi < a.gpr; gi += kWave) {
        float g[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) g[k] = g_row[4 * gi + k];
        accumulate(g_sq, grad_s, g, load_group(s_row + 3 * gi), a.cd, WITH_GS);
    }
    const RowConsts rc = finish_row(a, row, lane, g_sq, grad_s, WITH_GS);
    const uint32_t row_elem = (uint32_t)row * (uint32_t)a.in_features;
    for (int gi = lane; gi < a.gpr; gi += kWave) {
        float g[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) g[k] = g_row[4 * gi + k];
        const uint32_t nw = tick_group(load_group(s_row + 3 * gi), g, rc, a, row_elem + 4u * (uint32_t)gi);
        store_group(s_row + 3 * gi, nw);
    }
}

template <int ITERS>
void launch_rows(const UpdateArgs& a, hipStream_t stream) {
    const dim3 grid((a.out_features + kWavesPerBlock - 1) / kWavesPerBlock);
    const dim3 block(kWave * kWavesPerBlock);
    if (a.lr_scale != 0.0f)
        hipLaunchKernelGGL((update_rows_kernel<ITERS, true>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((update_rows_kernel<ITERS, false>), grid, block, 0, stream, a);
}

}  // namespace

// Enqueues the update-only step.  Arguments are already validated by the caller.
hipError_t launch_update_dense(hipStream_t stream, uint8_t* state, float* scale, float* v,
                               const float* grad_w, int C, int in_features, int out_features,
                               float lr, float lr_scale, float rms_beta, float rms_eps,
                               uint32_t seed) {
    UpdateArgs a;
    a.state = state; a.scale = scale; a.v = v; a.grad_w = grad_w;
    a.cd = make_codec(C);
    a.in_features = in_features; a.out_features = out_features;
    a.gpr = in_features / 4;
    a.lr = lr; a.lr_scale = lr_scale; a.rms_beta = rms_beta; a.rms_eps = rms_eps;
    a.seed = seed;

    const int iters = (a.gpr + kWave - 1) / kWave;
    const bool aligned = (reinterpret_cast<uintptr_t>(grad_w) & 15u) == 0;
    if (aligned && iters <= 1) launch_rows<1>(a, stream);
    else if (aligned && iters <= 2) launch_rows<2>(a, stream);
    else if (aligned && iters <= 3) launch_rows<3>(a, stream);
    else if (aligned && iters <= 4) launch_rows<4>(a, stream);
    else if (aligned && iters <= 8) launch_rows<8>(a, stream);
    else if (aligned && iters <= 12) launch_rows<12>(a, stream);
    else if (aligned && iters <= 16) launch_rows<16>(a, stream);
    else if (aligned && iters <= 24) launch_rows<24>(a, stream);
    else if (aligned && iters <= 32) launch_rows<32>(a, stream);
    else if (aligned && iters <= 43) launch_rows<43>(a, stream);
    else {
        const dim3 grid((a.out_features + kWavesPerBlock - 1) / kWavesPerBlock);
        const dim3 block(kWave * kWavesPerBlock);
        if (a.lr_scale != 0.0f)
            hipLaunchKernelGGL((update_rows_generic_kernel<true>), grid, block, 0, stream, a);
        else
            hipLaunchKernelGGL((update_rows_generic_kernel<false>), grid, block, 0, stream, a);
    }
    return hipGetLastError();
}

}  // namespace mcc
