// Main loop of the fp32 MFMA contraction c[m,n] = sum_k a[k,m] * b[k,n], shared by the plain
// contraction kernel and the strip-fused update kernel.
//
// Both operands are stored token-major, which is exactly the operand shape of
// v_mfma_f32_32x32x2_f32: lane l supplies a[k0 + l/32][m0 + l%32] and b[k0 + l/32][n0 + l%32],
// i.e. 32 consecutive floats of one token row per half-wave.  Slabs of kBK tokens are staged
// into LDS in their HBM orientation ([k][m] and [k][n]) with 16-byte loads and read back with
// conflict-free 4-byte reads; no transpose is needed.  A workgroup of 4 waves (2x2) owns a
// BM x BN tile; each wave owns (BM/2) x (BN/2) as 32x32 MFMA tiles whose accumulators stay in
// registers for the whole K loop.  The next slab is fetched from HBM into registers while the
// current one is multiplied.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

namespace mcc {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kGemmThreads = 256;
constexpr int kBK = 16;  // tokens per LDS slab

template <int BM, int BN>
struct TileCfg {
    static constexpr int kWaveM = BM / 2;        // rows of c per wave
    static constexpr int kWaveN = BN / 2;        // cols of c per wave
    static constexpr int kTilesM = kWaveM / 32;  // 32x32 MFMA tiles per wave along m
    static constexpr int kTilesN = kWaveN / 32;
    static constexpr int kLdA = BM + 4;  // padded LDS row strides (floats)
    static constexpr int kLdB = BN + 4;
    static constexpr int kA4 = kBK * BM / 4 / kGemmThreads;  // float4 loads per thread per slab
    static constexpr int kB4 = kBK * BN / 4 / kGemmThreads;
    static constexpr int kLdsFloats = kBK * (kLdA + kLdB);
};

// One slab row segment of 4 floats, zero-filled outside the matrix (`rows` x `cols`, rows
// `stride` floats apart).
template <bool VEC>
__device__ __forceinline__ float4 load4(const float* __restrict__ base, int row, int col, int rows, int cols, int stride) {
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row >= rows) return r;
    const float* p = base + (size_t)row * stride + col;
    if (VEC) {
        if (col + 3 < cols) return *reinterpret_cast<const float4*>(p);
    }
    if (col + 0 < cols) r.x = p[0];
    if (col + 1 < cols) r.y = p[1];
    if (col + 2 < cols) r.z = p[2];
    if (col + 3 < cols) r.w = p[3];
    return r;
}

// Position of the calling thread inside its workgroup's tile.
struct TilePos {
    int tid, l32, half, wm0, wn0;
};

template <int BM, int BN>
__device__ __forceinline__ TilePos tile_pos() {
    using Cfg = TileCfg<BM, BN>;
    TilePos p;
    p.tid = threadIdx.x;
    const int lane = p.tid & 63, wave = p.tid >> 6;
    p.l32 = lane & 31;
    p.half = lane >> 5;
    p.wm0 = (wave >> 1) * Cfg::kWaveM;
    p.wn0 = (wave & 1) * Cfg::kWaveN;
    return p;
}

// Which tile of a tiles_x x tiles_y grid the calling workgroup computes.  Workgroups are dealt to
// the 8 XCDs round-robin by linear id, and each XCD has an L2 of its own: a tile order that
// follows the launch order puts neighbouring tiles -- which share operand panels -- on eight
// different L2s.  Here workgroups w, w + 8, w + 16, ... (one XCD) take consecutive tiles of an
// order that walks bands of `band_rows` tile rows column by column, so the workgroups resident
// together on an XCD cover a compact block of tiles and fetch each panel slab once between them.
// A bijection for any grid; gridDim.x * gridDim.y must equal tiles_x * tiles_y.
struct TileXY {
    int x, y;
};
__device__ __forceinline__ TileXY xcd_tile(int tiles_x, int tiles_y, int band_rows) {
    const uint32_t total = (uint32_t)tiles_x * (uint32_t)tiles_y;
    const uint32_t w = blockIdx.x + blockIdx.y * gridDim.x;
    const uint32_t xcd = w & 7u, local = w >> 3;
    const uint32_t base = total >> 3, rem = total & 7u;
    const uint32_t t = xcd * base + (xcd < rem ? xcd : rem) + local;
    const uint32_t band_tiles = (uint32_t)band_rows * (uint32_t)tiles_x;
    const uint32_t band = t / band_tiles, within = t - band * band_tiles;
    const uint32_t left = (uint32_t)tiles_y - band * (uint32_t)band_rows;
    const uint32_t rows = left < (uint32_t)band_rows ? left : (uint32_t)band_rows;
    TileXY r;
    r.x = (int)(within / rows);
    r.y = (int)(band * (uint32_t)band_rows + within % rows);
    return r;
}

// Accumulates the BM x BN tile at (m0, n0) over all K tokens into acc (zeroed here).  lds holds
// TileCfg::kLdsFloats floats.  Ends with a barrier, so lds may be reused right after.  `a` is
// K x M with rows `lda` floats apart (lda > M when a is a column band of a wider matrix).
// Accumulator layout (v_mfma_f32_32x32x2_f32): acc[i][j][r] is row
// wm0 + 32 i + 8 (r/4) + 4 half + r%4 and column wn0 + 32 j + l32 of the tile.
//
// ROTATE_PRIORITY: the hardware issues from a SIMD's oldest wave first, so of the four workgroups
// resident on a CU the first one runs up to 30 % ahead of the last.  Kernels whose workgroups wait
// for each other want even progress instead: every kPriorityPeriod slabs the wave moves to the
// next of four priority levels, and workgroups resident together start at different levels
// (priority_phase = the workgroup's residency layer), so each leads a quarter of the time.
constexpr int kPriorityPeriod = 16;

__device__ __forceinline__ void set_wave_priority(int level) {
    switch (level) {  // s_setprio takes an immediate
        case 0: __builtin_amdgcn_s_setprio(0); break;
        case 1: __builtin_amdgcn_s_setprio(1); break;
        case 2: __builtin_amdgcn_s_setprio(2); break;
        default: __builtin_amdgcn_s_setprio(3); break;
    }
}

template <int BM, int BN, bool VEC_A, bool VEC_B, bool ROTATE_PRIORITY = false>
__device__ __forceinline__ void gemm_tile_mainloop(const float* __restrict__ a, const float* __restrict__ b,
                                                   int K, int M, int N, int m0, int n0, const TilePos& tp,
                                                   float* lds,
                                                   floatx16 (&acc)[TileCfg<BM, BN>::kTilesM][TileCfg<BM, BN>::kTilesN],
                                                   int lda, int priority_phase = 0) {
    using Cfg = TileCfg<BM, BN>;
    float* lds_a = lds;
    float* lds_b = lds + kBK * Cfg::kLdA;
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
            const int idx = tp.tid + kGemmThreads * p;
            const int row = idx / (BM / 4), c4 = idx % (BM / 4);
            ra[p] = load4<VEC_A>(a, k0 + row, m0 + 4 * c4, K, M, lda);
        }
#pragma unroll
        for (int p = 0; p < Cfg::kB4; ++p) {
            const int idx = tp.tid + kGemmThreads * p;
            const int row = idx / (BN / 4), c4 = idx % (BN / 4);
            rb[p] = load4<VEC_B>(b, k0 + row, n0 + 4 * c4, K, N, N);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int p = 0; p < Cfg::kA4; ++p) {
            const int idx = tp.tid + kGemmThreads * p;
            const int row = idx / (BM / 4), c4 = idx % (BM / 4);
            *reinterpret_cast<float4*>(&lds_a[row * Cfg::kLdA + 4 * c4]) = ra[p];
        }
#pragma unroll
        for (int p = 0; p < Cfg::kB4; ++p) {
            const int idx = tp.tid + kGemmThreads * p;
            const int row = idx / (BN / 4), c4 = idx % (BN / 4);
            *reinterpret_cast<float4*>(&lds_b[row * Cfg::kLdB + 4 * c4]) = rb[p];
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += kBK) {
        if (ROTATE_PRIORITY && (k0 & (kPriorityPeriod * kBK - 1)) == 0)
            set_wave_priority((k0 / (kPriorityPeriod * kBK) + priority_phase) & 3);
        stage();
        __syncthreads();
        if (k0 + kBK < K) fetch(k0 + kBK);
#pragma unroll
        for (int kk = 0; kk < kBK / 2; ++kk) {
            float fa[Cfg::kTilesM], fb[Cfg::kTilesN];
            const int krow = 2 * kk + tp.half;
#pragma unroll
            for (int i = 0; i < Cfg::kTilesM; ++i) fa[i] = lds_a[krow * Cfg::kLdA + tp.wm0 + 32 * i + tp.l32];
#pragma unroll
            for (int j = 0; j < Cfg::kTilesN; ++j) fb[j] = lds_b[krow * Cfg::kLdB + tp.wn0 + 32 * j + tp.l32];
#pragma unroll
            for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
                for (int j = 0; j < Cfg::kTilesN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
}

// The same contraction with the slabs copied from global memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, no LDS store instructions) and two LDS buffers,
// so that a slab costs one barrier: 3 % faster on the 7B shapes.  A wave's 64 lanes write 64
// consecutive 16-byte pieces, so the slab is stored unpadded ([k][m], the MFMA operand read of 32
// consecutive floats is conflict-free without padding).  Whole tiles and whole slabs only:
// K % kBK == 0, the tile lies inside the matrix and the operands are 16-byte aligned (nothing can
// be zero-filled on the way); other shapes use gemm_tile_mainloop.  lds holds
// DirectCfg::kLdsFloats floats.
template <int BM, int BN>
struct DirectCfg {
    static constexpr int kSlabFloats = kBK * (BM + BN);
    static constexpr int kLdsFloats = 2 * kSlabFloats;
    static constexpr int kA4 = kBK * BM / 4 / kGemmThreads;
    static constexpr int kB4 = kBK * BN / 4 / kGemmThreads;
};

template <int BM, int BN, bool ROTATE_PRIORITY = false>
__device__ __forceinline__ void gemm_tile_mainloop_direct(
    const float* __restrict__ a, const float* __restrict__ b, int K, int M, int N, int m0, int n0, const TilePos& tp,
    float* lds, floatx16 (&acc)[TileCfg<BM, BN>::kTilesM][TileCfg<BM, BN>::kTilesN], int lda,
    int priority_phase = 0) {
    using Cfg = TileCfg<BM, BN>;
    using D = DirectCfg<BM, BN>;
#pragma unroll
    for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::kTilesN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    const int lane = tp.tid & 63, wave = tp.tid >> 6;
    typedef __attribute__((address_space(3))) void* lds_ptr;
    typedef const __attribute__((address_space(1))) void* global_ptr;
    auto issue = [&](int k0, int buf) {
        float* dst_a = lds + buf * D::kSlabFloats;
        float* dst_b = dst_a + kBK * BM;
#pragma unroll
        for (int p = 0; p < D::kA4; ++p) {
            const int chunk = p * 4 + wave;         // 64 consecutive float4 of the slab
            const int idx = chunk * 64 + lane;
            const int row = idx / (BM / 4), c4 = idx % (BM / 4);
            __builtin_amdgcn_global_load_lds((global_ptr)(a + (size_t)(k0 + row) * lda + m0 + 4 * c4),
                                             (lds_ptr)(dst_a + chunk * 256), 16, 0, 0);
        }
#pragma unroll
        for (int p = 0; p < D::kB4; ++p) {
            const int chunk = p * 4 + wave;
            const int idx = chunk * 64 + lane;
            const int row = idx / (BN / 4), c4 = idx % (BN / 4);
            __builtin_amdgcn_global_load_lds((global_ptr)(b + (size_t)(k0 + row) * N + n0 + 4 * c4),
                                             (lds_ptr)(dst_b + chunk * 256), 16, 0, 0);
        }
    };
    issue(0, 0);
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += kBK) {
        if (ROTATE_PRIORITY && (k0 & (kPriorityPeriod * kBK - 1)) == 0)
            set_wave_priority((k0 / (kPriorityPeriod * kBK) + priority_phase) & 3);
        __builtin_amdgcn_s_waitcnt(0);  // this wave's part of the slab has landed
        __syncthreads();                // ... and everybody else's; the other buffer is free
        if (k0 + kBK < K) issue(k0 + kBK, buf ^ 1);
        const float* lds_a = lds + buf * D::kSlabFloats;
        const float* lds_b = lds_a + kBK * BM;
#pragma unroll
        for (int kk = 0; kk < kBK / 2; ++kk) {
            float fa[Cfg::kTilesM], fb[Cfg::kTilesN];
            const int krow = 2 * kk + tp.half;
#pragma unroll
            for (int i = 0; i < Cfg::kTilesM; ++i) fa[i] = lds_a[krow * BM + tp.wm0 + 32 * i + tp.l32];
#pragma unroll
            for (int j = 0; j < Cfg::kTilesN; ++j) fb[j] = lds_b[krow * BN + tp.wn0 + 32 * j + tp.l32];
#pragma unroll
            for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
                for (int j = 0; j < Cfg::kTilesN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        buf ^= 1;
    }
    __syncthreads();
}

}  // namespace mcc
