// Weight-gradient contraction on the gfx950 fp32 matrix cores:
//     c[m,n] = sum_k a[k,m] * b[k,n]        (a = grad_out [tokens,out], b = x [tokens,in])
// The main loop lives in gemm_tile.hpp; this file adds the store epilogue and the launch.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <vector>

#include "gemm_tile.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

// Token chunk blockIdx.z of `chunk` tokens goes to slice blockIdx.z of `c` (slices are m*n floats
// apart); with one chunk this is the whole contraction.  Rows of `a` are lda floats apart.
template <int BM, int BN, bool VEC_A, bool VEC_B, bool DIRECT>
__global__ __launch_bounds__(kGemmThreads) void gemm_tn_kernel(const float* __restrict__ a,
                                                                const float* __restrict__ b,
                                                                float* __restrict__ c, int K, int M, int N,
                                                                int chunk, int lda) {
    using Cfg = TileCfg<BM, BN>;
    __shared__ float lds[DIRECT ? DirectCfg<BM, BN>::kLdsFloats : Cfg::kLdsFloats];
    const TilePos tp = tile_pos<BM, BN>();
    const TileXY tile = xcd_tile(gridDim.x, gridDim.y, 8);
    const int m0 = tile.y * BM;
    const int n0 = tile.x * BN;
    const int k_begin = blockIdx.z * chunk;
    const int k_len = K - k_begin < chunk ? K - k_begin : chunk;
    a += (size_t)k_begin * lda;
    b += (size_t)k_begin * N;
    c += (size_t)blockIdx.z * M * N;
    floatx16 acc[Cfg::kTilesM][Cfg::kTilesN];
    if (DIRECT)
        gemm_tile_mainloop_direct<BM, BN>(a, b, k_len, M, N, m0, n0, tp, lds, acc, lda);
    else
        gemm_tile_mainloop<BM, BN, VEC_A, VEC_B>(a, b, k_len, M, N, m0, n0, tp, lds, acc, lda);
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

// ---------------------------------------------------------------------------
// Grouped form: the contractions of several tensors in one launch (and one launch that adds
// their chunk slices).  A small layer is tens of microseconds of work, so a model made of such
// layers is bound by launches when every tensor goes out on its own; here the descriptors
// travel as kernel arguments and a workgroup finds its tensor by scanning their first-workgroup
// indices.  The order of a gradient's token sum depends on the token chunks alone, not on the tile
// size or on how a slab reaches LDS: while every tensor keeps the chunks of its own plan the
// gradients are the same bits as from launch_gemm_tn_f32; a list whose tiles fill the device is
// cut into fewer chunks (list_splits), and its gradients are then those sums.
// ---------------------------------------------------------------------------
struct GemmGroupItem {
    const float* a;
    const float* b;
    float* out;  // slice 0 (the chunk slices are M*N floats apart)
    int K, M, N, chunk, tiles_x, tiles, wg_start, pad;
};
constexpr int kMaxGemmGroup = 56;  // 56 descriptors of 56 bytes: the kernel arguments stay below 4 KiB
struct GemmGroupArgs {
    GemmGroupItem it[kMaxGemmGroup];
    int n;
};
static_assert(sizeof(GemmGroupArgs) <= 4096, "kernel arguments are limited to 4 KiB");

template <int BM, int BN>
__global__ __launch_bounds__(kGemmThreads) void gemm_tn_group_kernel(GemmGroupArgs g) {
    using Cfg = TileCfg<BM, BN>;
    __shared__ float lds[Cfg::kLdsFloats];
    const int wg = blockIdx.x;
    int i = 0;
    while (i + 1 < g.n && wg >= g.it[i + 1].wg_start) ++i;  // uniform: scalar loads of the arguments
    const GemmGroupItem it = g.it[i];
    const int local = wg - it.wg_start;
    const int z = local / it.tiles, t = local - z * it.tiles;
    const int ty = t / it.tiles_x, tx = t - ty * it.tiles_x;
    const TilePos tp = tile_pos<BM, BN>();
    const int m0 = ty * BM, n0 = tx * BN;
    const int k_begin = z * it.chunk;
    const int k_len = it.K - k_begin < it.chunk ? it.K - k_begin : it.chunk;
    const float* a = it.a + (size_t)k_begin * it.M;
    const float* b = it.b + (size_t)k_begin * it.N;
    float* c = it.out + (size_t)z * it.M * it.N;
    floatx16 acc[Cfg::kTilesM][Cfg::kTilesN];
    gemm_tile_mainloop<BM, BN, true, true>(a, b, k_len, it.M, it.N, m0, n0, tp, lds, acc, it.M);
#pragma unroll
    for (int ii = 0; ii < Cfg::kTilesM; ++ii)
#pragma unroll
        for (int j = 0; j < Cfg::kTilesN; ++j) {
            const int col = n0 + tp.wn0 + 32 * j + tp.l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + tp.wm0 + 32 * ii + 8 * (r / 4) + 4 * tp.half + (r % 4);
                if (row < it.M && col < it.N) c[(size_t)row * it.N + col] = acc[ii][j][r];
            }
        }
}

// 96 x 96 tiles for the grouped launch: 288- and 768-wide layers (the 15M-shaped model) are whole
// numbers of them, where 64 x 64 tiles cover 288 as 320 (a fifth of the matrix instructions wasted).
// Three waves, each 32 rows x 96 columns of the tile: four operand reads per three matrix
// instructions where the 2 x 2 waves of a 64 x 64 tile need six.  Same slabs, same order of the
// token sum as the other tiles, so the same bits.  m and n multiples of 96, operands 16-byte
// aligned.
constexpr int kThreads96 = 192;
// DIRECT: every chunk is a whole number of slabs, so the slabs go from global memory straight into
// one of two unpadded LDS buffers (no staging registers, no LDS store instructions, one barrier per
// slab); otherwise through registers with the end of a ragged chunk zero-filled.
template <bool DIRECT>
__global__ __launch_bounds__(kThreads96) void gemm_tn_group96_kernel(GemmGroupArgs g) {
    constexpr int kT96 = 96, kLd = DIRECT ? kT96 : kT96 + 4;
    constexpr int kSlab = kBK * kLd;  // floats of one operand's slab
    __shared__ float lds[(DIRECT ? 4 : 2) * kSlab];
    const int wg = blockIdx.x;
    int i = 0;
    while (i + 1 < g.n && wg >= g.it[i + 1].wg_start) ++i;  // uniform: scalar loads of the arguments
    const GemmGroupItem it = g.it[i];
    const int local = wg - it.wg_start;
    const int z = local / it.tiles, t = local - z * it.tiles;
    const int ty = t / it.tiles_x, tx = t - ty * it.tiles_x;
    const int m0 = ty * kT96, n0 = tx * kT96;
    const int k_begin = z * it.chunk;
    const int k_len = it.K - k_begin < it.chunk ? it.K - k_begin : it.chunk;
    const float* a = it.a + (size_t)k_begin * it.M;
    const float* b = it.b + (size_t)k_begin * it.N;
    float* c = it.out + (size_t)z * it.M * it.N;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    floatx16 acc[3];
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
    auto multiply = [&](const float* lds_a, const float* lds_b) {
#pragma unroll
        for (int kk = 0; kk < kBK / 2; ++kk) {
            const int krow = 2 * kk + half;
            const float fa = lds_a[krow * kLd + 32 * wave + l32];
            float fb[3];
#pragma unroll
            for (int j = 0; j < 3; ++j) fb[j] = lds_b[krow * kLd + 32 * j + l32];
#pragma unroll
            for (int j = 0; j < 3; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb[j], acc[j], 0, 0, 0);
        }
    };
    // 16 x 96 floats per operand and slab = 384 float4: two per thread (row = idx / 24, c4 = idx % 24)
    if constexpr (DIRECT) {
        typedef __attribute__((address_space(3))) void* lds_ptr;
        typedef const __attribute__((address_space(1))) void* global_ptr;
        auto issue = [&](int k0, int buf) {
            float* dst_a = lds + buf * 2 * kSlab;
            float* dst_b = dst_a + kSlab;
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int chunk = 3 * p + wave;  // 64 consecutive float4 of the slab
                const int idx = chunk * 64 + lane;
                const int row = idx / 24, c4 = idx % 24;
                __builtin_amdgcn_global_load_lds((global_ptr)(a + (size_t)(k0 + row) * it.M + m0 + 4 * c4),
                                                 (lds_ptr)(dst_a + chunk * 256), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((global_ptr)(b + (size_t)(k0 + row) * it.N + n0 + 4 * c4),
                                                 (lds_ptr)(dst_b + chunk * 256), 16, 0, 0);
            }
        };
        issue(0, 0);
        int buf = 0;
        for (int k0 = 0; k0 < k_len; k0 += kBK) {
            __builtin_amdgcn_s_waitcnt(0);  // this wave's part of the slab has landed
            __syncthreads();                // ... and everybody else's; the other buffer is free
            if (k0 + kBK < k_len) issue(k0 + kBK, buf ^ 1);
            multiply(lds + buf * 2 * kSlab, lds + buf * 2 * kSlab + kSlab);
            buf ^= 1;
        }
    } else {
        float* lds_a = lds;
        float* lds_b = lds + kSlab;
        float4 ra[2], rb[2];
        auto fetch = [&](int k0) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int idx = tid + kThreads96 * p;
                const int row = idx / 24, c4 = idx % 24;
                // a slab past the end of a chunk that is not a whole number of slabs is zero-filled
                const bool in = k0 + row < k_len;
                ra[p] = in ? *reinterpret_cast<const float4*>(a + (size_t)(k0 + row) * it.M + m0 + 4 * c4)
                           : make_float4(0.f, 0.f, 0.f, 0.f);
                rb[p] = in ? *reinterpret_cast<const float4*>(b + (size_t)(k0 + row) * it.N + n0 + 4 * c4)
                           : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        };
        fetch(0);
        for (int k0 = 0; k0 < k_len; k0 += kBK) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int idx = tid + kThreads96 * p;
                const int row = idx / 24, c4 = idx % 24;
                *reinterpret_cast<float4*>(&lds_a[row * kLd + 4 * c4]) = ra[p];
                *reinterpret_cast<float4*>(&lds_b[row * kLd + 4 * c4]) = rb[p];
            }
            __syncthreads();
            if (k0 + kBK < k_len) fetch(k0 + kBK);
            multiply(lds_a, lds_b);
            __syncthreads();
        }
    }
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int col = n0 + 32 * j + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = m0 + 32 * wave + 8 * (r / 4) + 4 * half + (r % 4);
            c[(size_t)row * it.N + col] = acc[j][r];
        }
    }
}

struct ReduceGroupItem {
    float* slices;  // summed in place into slice 0
    unsigned mn;
    int n_slices, block_start, pad;
};
constexpr int kMaxReduceGroup = 128;
struct ReduceGroupArgs {
    ReduceGroupItem it[kMaxReduceGroup];
    int n;
};
static_assert(sizeof(ReduceGroupArgs) <= 4096, "kernel arguments are limited to 4 KiB");
constexpr int kReduceBlockElems = 256;  // one element per thread: a thread's chunk loads are all in flight at once

__global__ __launch_bounds__(256) void reduce_slices_group_kernel(ReduceGroupArgs g) {
    const int wg = blockIdx.x;
    int i = 0;
    while (i + 1 < g.n && wg >= g.it[i + 1].block_start) ++i;
    const ReduceGroupItem it = g.it[i];
    const unsigned e = (unsigned)(wg - it.block_start) * kReduceBlockElems + threadIdx.x;
    if (e < it.mn) {
        float acc = it.slices[e];
        for (int s = 1; s < it.n_slices; ++s) acc = acc + it.slices[(size_t)s * it.mn + e];
        it.slices[e] = acc;
    }
}

// tiles_x, tiles_y > 0 restrict the launch to that many tiles from a, b, c on (a corner block of
// the matrix: m and n stay the row lengths)
template <int BM, int BN>
hipError_t launch_tile(hipStream_t stream, const float* a, const float* b, float* c, int k, int m, int n,
                       const GemmTnPlan& plan, int tiles_x = 0, int tiles_y = 0, int lda = 0) {
    if (lda == 0) lda = m;
    const dim3 grid(tiles_x > 0 ? tiles_x : (n + BN - 1) / BN, tiles_y > 0 ? tiles_y : (m + BM - 1) / BM, plan.splits);
    // every chunk starts at a multiple of 16 tokens, so it is as aligned as the matrix itself
    const bool vec_a = (m % 4 == 0) && (lda % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15u) == 0);
    const bool vec_b = (n % 4 == 0) && ((reinterpret_cast<uintptr_t>(b) & 15u) == 0);
    // whole tiles and whole slabs (every chunk is a multiple of 16 tokens when k is): direct-to-LDS
    const bool direct = vec_a && vec_b && m % BM == 0 && n % BN == 0 && k % kBK == 0;
    if (direct)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, true, true, true>), grid, dim3(kGemmThreads), 0, stream, a, b, c, k,
                           m, n, plan.chunk, lda);
    else if (vec_a && vec_b)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, true, true, false>), grid, dim3(kGemmThreads), 0, stream, a, b, c,
                           k, m, n, plan.chunk, lda);
    else if (vec_b)
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, false, true, false>), grid, dim3(kGemmThreads), 0, stream, a, b, c,
                           k, m, n, plan.chunk, lda);
    else
        hipLaunchKernelGGL((gemm_tn_kernel<BM, BN, false, false, false>), grid, dim3(kGemmThreads), 0, stream, a, b,
                           c, k, m, n, plan.chunk, lda);
    return hipGetLastError();
}

}  // namespace

// One 256 x 256 tile occupies a CU (8 waves, 64 KiB of LDS, 128 accumulator registers), so the
// wide kernel only pays when the tiles come in whole rounds of the 256 CUs: 4096 x 4096 is
// exactly one round (+4 % over 128 x 128 tiles), 11008 x 4096 is 2.69 rounds and loses 10 % to
// the last one, where the small tiles lose 2 %.
static bool wide_tiles_fill_the_device(int m, int n) {
    if (m % 256 || n % 256) return false;
    const long tiles = (long)(m / 256) * (n / 256);
    const long rounds = (tiles + 255) / 256;
    return tiles >= 256 && tiles * 100 >= rounds * 256 * 97;
}

// A smaller matrix whose token range the plan cuts into chunks: the wide tiles times the chunks
// should come close to whole rounds (2048 x 768 at 16384 tokens: 24 tiles x 10 chunks = 240).
static bool wide_chunks_fill_the_device(int m, int n, int splits) {
    if (m % 256 || n % 256 || splits < 2) return false;
    const long wgs = (long)(m / 256) * (n / 256) * splits;
    const long rounds = (wgs + 255) / 256;
    return wgs * 100 >= rounds * 256 * 85;
}

// For a matrix of `lines` x `across` wide tiles that is more than one round but not whole rounds:
// how many lines make whole rounds of 256 tiles (0: none do).  11008 x 4096 is 43 x 16 tiles:
// 32 lines are two rounds, the other 11 lines go to the small tiles.
static int wide_block(int lines, int across) {
    const long tiles = (long)lines * across;
    if (tiles <= 256 || across <= 0) return 0;
    const long full = tiles / 256 * 256;
    if (full % across) return 0;
    const long block = full / across;
    return block < lines ? (int)block : 0;
}

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

size_t gemm_tn_sync_nbytes(int k, int m, int n) {
    const GemmTnPlan plan = plan_gemm_tn(k, m, n);
    return plan.splits == 1 && plan.tile == 128 && gemm_tn_wide_spans_apply(k, m, n) ? kWideSpanWorkgroups * sizeof(int) : 0;
}

// `slices` holds plan.splits * m * n floats when the plan splits the tokens (it may start at c);
// it is not touched otherwise.
hipError_t launch_gemm_tn_f32(hipStream_t stream, const float* a, const float* b, float* c, int k, int m, int n,
                              float* slices, int mode, int lda, const GemmTnPlan* band_plan, int* sync_words) {
    GemmTnPlan plan = plan_gemm_tn(k, m, n);
    if (band_plan && lda != 0 && lda != m) {
        plan.splits = band_plan->splits;  // the tile size follows the rows at hand (a last, shorter band)
        plan.chunk = band_plan->chunk;
    }
    float* out = plan.splits > 1 ? slices : c;
    if (plan.splits > 1 && !slices) return hipErrorInvalidValue;
    hipError_t e;
    if (lda != 0 && lda != m) {
        // a column band of a wider matrix: the general tiles only
        e = plan.tile == 128 ? launch_tile<128, 128>(stream, a, b, out, k, m, n, plan, 0, 0, lda)
                             : launch_tile<64, 64>(stream, a, b, out, k, m, n, plan, 0, 0, lda);
        if (e != hipSuccess || plan.splits == 1) return e;
        const size_t mn_band = (size_t)m * n;
        const size_t want_band = (mn_band + 255) / 256;
        hipLaunchKernelGGL(reduce_slices_kernel, dim3((unsigned)(want_band < 4096 ? want_band : 4096)), dim3(256), 0, stream,
                           slices, c, mn_band, plan.splits);
        return hipGetLastError();
    }
    const bool wide_ok = plan.tile == 128 && gemm_tn_wide_supports(a, b, k, m, n, plan.chunk);
    // rows or columns of wide tiles that make whole rounds, when the whole matrix does not
    const int wide_rows = wide_ok && plan.splits == 1 ? wide_block(m / 256, n / 256) : 0;
    const int wide_cols = wide_ok && plan.splits == 1 && wide_rows == 0 ? wide_block(n / 256, m / 256) : 0;
    if (mode == 1 && gemm_tn_bf16x6_supports(a, b, k, m, n, plan)) {
        e = launch_gemm_tn_bf16x6(stream, a, b, out, k, m, n, plan);
    } else if (wide_ok && (wide_tiles_fill_the_device(m, n) || wide_chunks_fill_the_device(m, n, plan.splits))) {
        e = launch_gemm_tn_wide(stream, a, b, out, k, m, n, n / 256, m / 256, plan.chunk, plan.splits);
    } else if (wide_ok && plan.splits == 1 && sync_words && gemm_tn_wide_spans_apply(k, m, n)) {
        e = launch_gemm_tn_wide_spans(stream, a, b, out, k, m, n, sync_words);
    } else if (wide_rows > 0) {
        // wide tiles on the first rows, small tiles on the rest
        const int r = 256 * wide_rows;
        e = launch_gemm_tn_wide(stream, a, b, out, k, m, n, n / 256, wide_rows, plan.chunk, 1);
        if (e == hipSuccess)
            e = launch_tile<128, 128>(stream, a + r, b, out + (size_t)r * n, k, m, n, plan, n / 128, (m - r) / 128);
    } else if (wide_cols > 0) {
        const int cw = 256 * wide_cols;
        e = launch_gemm_tn_wide(stream, a, b, out, k, m, n, wide_cols, m / 256, plan.chunk, 1);
        if (e == hipSuccess)
            e = launch_tile<128, 128>(stream, a, b + cw, out + cw, k, m, n, plan, (n - cw) / 128, m / 128);
    } else {
        e = plan.tile == 128 ? launch_tile<128, 128>(stream, a, b, out, k, m, n, plan)
                             : launch_tile<64, 64>(stream, a, b, out, k, m, n, plan);
    }
    if (e != hipSuccess || plan.splits == 1) return e;
    const size_t mn = (size_t)m * n;
    const size_t want = (mn + 255) / 256;
    hipLaunchKernelGGL(reduce_slices_kernel, dim3((unsigned)(want < 4096 ? want : 4096)), dim3(256), 0, stream, slices,
                       c, mn, plan.splits);
    return hipGetLastError();
}

// The contractions of `n` tensors (c = slice 0 of `out`, which holds gemm_tn_slices floats-matrices).
// Tensors whose operands are 16-byte aligned with m, n multiples of 4 are grouped by tile size;
// the others, and very large ones (which fill the device alone), go out one by one.
// Whether job j can share a grouped launch of `tile`-sized tiles, and its plan on its own.
// (tile 96: the small-tile plan on 96 x 96 tiles, for sides that are multiples of 96)
static bool groupable(const GemmTnJob& j, int tile, GemmTnPlan* plan_out, long* tiles_out) {
    const GemmTnPlan plan = plan_gemm_tn(j.k, j.m, j.n);
    const bool vec = j.m % 4 == 0 && j.n % 4 == 0 && (reinterpret_cast<uintptr_t>(j.a) & 15u) == 0 &&
                     (reinterpret_cast<uintptr_t>(j.b) & 15u) == 0;
    const bool fits96 = plan.tile == 64 && j.m % 96 == 0 && j.n % 96 == 0;
    const int side = tile == 96 ? 96 : plan.tile;
    const long tiles = (long)((j.m + side - 1) / side) * ((j.n + side - 1) / side);
    *plan_out = plan;
    *tiles_out = tiles;
    if (tile == 96 ? !fits96 : (plan.tile != tile || fits96)) return false;
    // a tensor of 1024 workgroups or more gains nothing from sharing a launch, and one whose
    // chunks fill the device with wide tiles is faster on those
    if (!vec || tiles * plan.splits >= 1024) return false;
    if (plan.tile == 128 && gemm_tn_wide_supports(j.a, j.b, j.k, j.m, j.n, plan.chunk) &&
        wide_chunks_fill_the_device(j.m, j.n, plan.splits))
        return false;
    return true;
}

// Token chunks of a list: a tensor's own plan cuts its tokens until its tiles alone fill the device
// (32 chunks for a 288 x 288 layer), which is slices to write and to add.  When the tiles of the
// whole list of one class fill the device twice over, the list is cut instead: as many chunks as
// bring the list to about sixteen workgroups a CU, the same for every tensor (0: keep the tensors'
// own plans; measured flat from 13 to 24 a CU).  15M-shaped model, 42 tensors: six chunks of 96 x 96 tiles.
static int list_splits(const GemmTnJob* jobs, size_t n, int tile) {
    long total = 0;
    for (size_t i = 0; i < n; ++i) {
        GemmTnPlan plan;
        long tiles;
        if (groupable(jobs[i], tile, &plan, &tiles)) total += tiles;
    }
    if (total < 512) return 0;  // two tiles for each of the 256 CUs
    const long s = 4096 / total;
    return s < 1 ? 1 : (int)s;
}

hipError_t launch_gemm_tn_group(hipStream_t stream, const GemmTnJob* jobs, size_t n) {
    std::vector<char> grouped(n, 0);
    std::vector<int> splits_used(n, 0);
    for (int tile : {96, 64, 128}) {
        const int of_list = list_splits(jobs, n, tile);
        GemmGroupArgs g;
        g.n = 0;
        int wgs = 0;
        bool whole_slabs = true;  // of the descriptors gathered so far: every chunk a whole number of slabs
        auto flush = [&]() -> hipError_t {
            if (g.n == 0) return hipSuccess;
            if (tile == 96 && whole_slabs)
                hipLaunchKernelGGL(gemm_tn_group96_kernel<true>, dim3(wgs), dim3(kThreads96), 0, stream, g);
            else if (tile == 96)
                hipLaunchKernelGGL(gemm_tn_group96_kernel<false>, dim3(wgs), dim3(kThreads96), 0, stream, g);
            else if (tile == 64)
                hipLaunchKernelGGL((gemm_tn_group_kernel<64, 64>), dim3(wgs), dim3(kGemmThreads), 0, stream, g);
            else
                hipLaunchKernelGGL((gemm_tn_group_kernel<128, 128>), dim3(wgs), dim3(kGemmThreads), 0, stream, g);
            g.n = 0;
            wgs = 0;
            whole_slabs = true;
            return hipGetLastError();
        };
        for (size_t i = 0; i < n; ++i) {
            const GemmTnJob& j = jobs[i];
            GemmTnPlan plan;
            long tiles;
            if (!groupable(j, tile, &plan, &tiles)) continue;
            if (of_list > 0 && of_list < plan.splits) {  // (never more slices than the tensor's region holds)
                const int chunk = (j.k + of_list - 1) / of_list;
                plan.chunk = (chunk + kBK - 1) / kBK * kBK;
                plan.splits = (j.k + plan.chunk - 1) / plan.chunk;
            }
            splits_used[i] = plan.splits;
            if (j.k % kBK != 0 || plan.chunk % kBK != 0) whole_slabs = false;
            if (g.n == kMaxGemmGroup || wgs > (1 << 30)) {
                const hipError_t e = flush();
                if (e != hipSuccess) return e;
            }
            GemmGroupItem& it = g.it[g.n++];
            it.a = j.a; it.b = j.b; it.out = j.out;
            it.K = j.k; it.M = j.m; it.N = j.n;
            it.chunk = plan.chunk;
            it.tiles_x = (j.n + tile - 1) / tile;
            it.tiles = (int)tiles;
            it.wg_start = wgs;
            it.pad = 0;
            wgs += (int)tiles * plan.splits;
            grouped[i] = 1;
        }
        const hipError_t e = flush();
        if (e != hipSuccess) return e;
    }
    // the rest one by one (this also adds their slices)
    for (size_t i = 0; i < n; ++i) {
        if (grouped[i]) continue;
        const hipError_t e = launch_gemm_tn_f32(stream, jobs[i].a, jobs[i].b, jobs[i].out, jobs[i].k, jobs[i].m,
                                                jobs[i].n, jobs[i].out, 0, 0, nullptr, jobs[i].sync_words);
        if (e != hipSuccess) return e;
    }
    // slices of the grouped tensors, in chunk order
    ReduceGroupArgs r;
    r.n = 0;
    int blocks = 0;
    auto flush_reduce = [&]() -> hipError_t {
        if (r.n == 0) return hipSuccess;
        hipLaunchKernelGGL(reduce_slices_group_kernel, dim3(blocks), dim3(256), 0, stream, r);
        r.n = 0;
        blocks = 0;
        return hipGetLastError();
    };
    for (size_t i = 0; i < n; ++i) {
        if (!grouped[i] || splits_used[i] == 1) continue;
        if (r.n == kMaxReduceGroup) {
            const hipError_t e = flush_reduce();
            if (e != hipSuccess) return e;
        }
        ReduceGroupItem& it = r.it[r.n++];
        it.slices = jobs[i].out;
        it.mn = (unsigned)((size_t)jobs[i].m * jobs[i].n);  // below 2^32: the tensor has fewer than 1024 tiles
        it.n_slices = splits_used[i];
        it.block_start = blocks;
        it.pad = 0;
        blocks += (int)((it.mn + kReduceBlockElems - 1) / kReduceBlockElems);
    }
    return flush_reduce();
}

}  // namespace mcc
