// Forward and input-gradient products of the counter layer on the bf16 matrix cores, with fp32
// accuracy.
//
// The weight is W[o,i] = scale[o] * t[o,i] with t a small integer (-1, 0, 1 for every reachable
// code), and a small integer is exact in bf16.  A binary32 activation is the exact sum of three
// bf16 numbers,
//     x = hi + mid + lo,   hi = bf16(x),  mid = bf16(x - hi),  lo = bf16(x - hi - mid)
// (each subtraction is exact: 24 significant bits are peeled off 8 at a time; only numbers within
// 2^16 of the smallest normal lose their tail), and a bf16 x bf16 product is exact in binary32.
// So
//     sum_k x[k] * t[k] = sum_k hi[k] t[k] + sum_k mid[k] t[k] + sum_k lo[k] t[k]
// is three bf16 MFMA passes into one fp32 accumulator whose every product is exact: the same
// mathematical terms as an fp32 contraction, summed in another order, at 16 x the matrix rate
// per pass (v_mfma_f32_32x32x16_bf16 against v_mfma_f32_32x32x2_f32).
//   forward         y[r,o]      = scale[o] * sum_i x[r,i] * t[o,i]
//   backward_input  grad_x[r,i] = sum_o (grad_out[r,o] * scale[o]) * t[o,i]
// (kernels/vulkan/counter_forward_f32_rb4.comp, counter_backward_input_f32_rb4.comp; the second
// line multiplies by the scale first, as kernels/compact_counter.cl:262-267 does).  Non-finite
// activations are outside this kernel's contract (inf - inf in the split).
//
// Tile: 128 rows x 128 or 256 columns per workgroup, 32-deep slabs: 4 or 8 waves of 64 x 64 that
// each stage and multiply (counter_linear_bf16x3_kernel), or, for large products, 16 waves of
// which half stage and half multiply (counter_linear_bf16x3_split_roles_kernel).  LDS holds the three activation planes and the weight tile as [row][32 bf16] = 64-byte
// rows whose four 16-byte chunks are XOR-swizzled with bits 2-3 of the row, which makes the
// 16-byte MFMA operand reads (lane = row, 8 consecutive k) conflict-free without padding:
// 32 or 40 KiB per workgroup.  Splitting and decoding are done by the thread that fetched the
// data, on its way into LDS.  The whole-tile kernel decodes through a table: two neighbouring
// 6-bit codes of a packed word index a 4096-entry LDS table (16 KiB, built once per workgroup)
// whose entries are their two ternary values as a bf16 pair, so a packed group costs two table
// reads and four address instructions instead of 22 instructions of arithmetic -- the vector work
// per slab, which competes with the matrix instructions for issue slots, drops by about a third.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "bf16_split.hpp"
#include "counter_math.hpp"
#include "gemm_tile.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

struct Lin3Args {
    const float* act;      // [rows, K]
    const uint8_t* state;  // packed [out, in/4 * 3]
    const float* scale;    // [out]
    float* c;              // [rows, N]
    Codec cd;
    int rows, in_features, out_features;
};

__device__ __forceinline__ uint32_t fetch_group(const uint8_t* state, size_t group, size_t last_group, bool valid) {
    if (!valid) return 0xffffffffu;  // marks "no weight": decoded to zero below
    const uint8_t* p = state + 3 * group;
    if (group == last_group) return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
    uint32_t w;
    __builtin_memcpy(&w, p, 4);
    return w & 0x00ffffffu;
}

// t = code / lv - 1 of code k of a packed word, as a float (0 for the "no weight" marker).
__device__ __forceinline__ float ternary_of(uint32_t word, int k, const Codec& cd) {
    const float t = (float)(code_q(code_of(word, k), cd) - 1);
    return word == 0xffffffffu ? 0.0f : t;
}

// Whole tiles and whole slabs (rows, N multiples of 128, K a multiple of 32, 16-byte aligned
// activation and scale, buffers below 4 GiB): nothing is checked, every address is a per-thread
// 32-bit offset computed once plus a per-slab constant.
// WN waves side by side (each 64 columns) times 2 waves down: the tile is 128 rows x 64 WN columns
// and the split of an activation slab is shared by that many columns.
template <bool FORWARD, int WN>
__global__ __launch_bounds__(128 * WN, WN == 2 ? 3 : 4) void counter_linear_bf16x3_kernel(Lin3Args a) {
    constexpr int kThreads = 128 * WN;
    constexpr int kTN = 64 * WN;
    constexpr int kA4 = kT * kK / 4 / kThreads;  // float4 of activation per thread and slab
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[3 * kPlaneBytes];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[kTN * kRowBytes];
    // pair_t[c1 << 6 | c0] = bf16(t(c0)) | bf16(t(c1)) << 16 with t = code / lv - 1
    __shared__ uint32_t pair_t[4096];
    const int tid = threadIdx.x;
    for (int i = tid; i < 4096; i += kThreads)
        pair_t[i] = pack_bf16((float)(code_q((uint32_t)i & 63u, a.cd) - 1), (float)(code_q((uint32_t)i >> 6, a.cd) - 1));
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, kh = lane >> 5;
    const int wm0 = (wave / WN) * 64, wn0 = (wave % WN) * 64;
    // the activation panel weighs 4 bytes an element, the packed weight panel 0.75: flat bands
    const TileXY tile = xcd_tile(gridDim.x, gridDim.y, 4);
    const int m0 = tile.y * kT, n0 = tile.x * kTN;
    const int K = FORWARD ? a.in_features : a.out_features;
    const int N = FORWARD ? a.out_features : a.in_features;
    const uint32_t gpr = (uint32_t)a.in_features >> 2;
    const uint32_t last_off = 3u * ((uint32_t)a.out_features * gpr - 1u);

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // thread (row = tid / 8 + (threads / 8) p, c4 = tid % 8) stages 4 activations per p; byte offsets
    const int c4 = tid & 7, row0 = tid >> 3;
    uint32_t off_a[kA4], off_w[4];
    int lds_off_a[kA4], lds_off_b[4];
#pragma unroll
    for (int p = 0; p < kA4; ++p) {
        const int row = row0 + (kThreads / 8) * p;
        off_a[p] = ((uint32_t)(m0 + row) * (uint32_t)K + 4u * c4) * 4u;
        lds_off_a[p] = tile_offset(row, c4 >> 1, c4 & 1);
    }
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        if (FORWARD) {
            // (weight row n = tid / 8 + (threads / 8) p, group c4 of the slab)
            const int n = row0 + (kThreads / 8) * p;
            off_w[p] = 3u * ((uint32_t)(n0 + n) * gpr + (uint32_t)c4);
            lds_off_b[p] = tile_offset(n, c4 >> 1, c4 & 1);
        } else {
            // (weight rows k = 4 oq + p with oq = tid % 8, group g = tid / 8 of the tile's columns)
            off_w[p] = 3u * ((uint32_t)(4 * c4 + p) * gpr + (uint32_t)(n0 >> 2) + (uint32_t)row0);
            // column n = 4 g + p, k = 4 oq ..: a wave writes rows 4 apart, hence the dealt row order
            lds_off_b[p] = dealt_tile_offset<kTN>(4 * row0 + p, c4 >> 1, c4 & 1);
        }
    }
    const uint32_t w_step = FORWARD ? 3u * (kK / 4) : 3u * kK * gpr;  // packed bytes per slab

    float4 ra[kA4];
    uint32_t rw[4];
    auto fetch = [&](int k0, uint32_t w_base) {
        float4 sc = make_float4(1.f, 1.f, 1.f, 1.f);
        if (!FORWARD) sc = *reinterpret_cast<const float4*>(a.scale + k0 + 4 * c4);
#pragma unroll
        for (int p = 0; p < kA4; ++p) {
            const float4 x = *reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(a.act) + off_a[p] +
                                                              4u * (uint32_t)k0);
            // (grad_out * scale) first, as the reference does
            ra[p] = FORWARD ? x : make_float4(x.x * sc.x, x.y * sc.y, x.z * sc.z, x.w * sc.w);
        }
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            // one 4-byte load per packed group; the tensor's last group has no byte after it and
            // is fetched one byte early
            const uint32_t off = off_w[p] + w_base;
            const uint32_t is_last = off == last_off ? 1u : 0u;
            uint32_t w;
            __builtin_memcpy(&w, a.state + (off - is_last), 4);
            rw[p] = w >> (8 * is_last);
        }
    };
    // the ternary values of codes 0, 1 (low pair) and 2, 3 (high pair) of a packed word, as bf16 pairs
    auto pair_lo = [&](uint32_t word) { return pair_t[word & 0xfffu]; };
    auto pair_hi = [&](uint32_t word) { return pair_t[(word >> 12) & 0xfffu]; };
    auto stage = [&]() {
#pragma unroll
        for (int p = 0; p < kA4; ++p) store_split(lds_a, lds_off_a[p], ra[p].x, ra[p].y, ra[p].z, ra[p].w);
        if (FORWARD) {
#pragma unroll
            for (int p = 0; p < 4; ++p)
                *reinterpret_cast<uint2*>(lds_b + lds_off_b[p]) = make_uint2(pair_lo(rw[p]), pair_hi(rw[p]));
        } else {
            // rw[r] is weight row k = 4 oq + r; column 4 g + j takes code j of each: the pairs come
            // out of the table along a row and are transposed two by two (v_perm_b32)
#pragma unroll
            for (int h = 0; h < 2; ++h) {  // codes 2 h, 2 h + 1
                uint32_t pr[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) pr[r] = h == 0 ? pair_lo(rw[r]) : pair_hi(rw[r]);
                // column 2 h: the low halves of rows (0, 1) and (2, 3); column 2 h + 1: the high halves
                const uint32_t lo0 = __builtin_amdgcn_perm(pr[1], pr[0], 0x05040100u);
                const uint32_t hi0 = __builtin_amdgcn_perm(pr[3], pr[2], 0x05040100u);
                const uint32_t lo1 = __builtin_amdgcn_perm(pr[1], pr[0], 0x07060302u);
                const uint32_t hi1 = __builtin_amdgcn_perm(pr[3], pr[2], 0x07060302u);
                *reinterpret_cast<uint2*>(lds_b + lds_off_b[2 * h]) = make_uint2(lo0, hi0);
                *reinterpret_cast<uint2*>(lds_b + lds_off_b[2 * h + 1]) = make_uint2(lo1, hi1);
            }
        }
    };
    int read_a[2], read_b[2];  // operand read offsets for chunk kh; the chunk of step s is 2 s + kh
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        read_a[i] = wm0 + 32 * i + l32;
        read_b[i] = wn0 + 32 * i + l32;
    }

    uint32_t w_base = 0;
    fetch(0, 0);
    __syncthreads();  // the table is complete
    for (int k0 = 0; k0 < K; k0 += kK) {
        stage();
        __syncthreads();
        w_base += w_step;
        if (k0 + kK < K) fetch(k0 + kK, w_base);
#pragma unroll
        for (int s = 0; s < kK / 16; ++s) {
            const int chunk = 2 * s + kh;
            bf16x8 fb[2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
                fb[j] = FORWARD ? read_operand(lds_b, read_b[j], chunk) : read_dealt_operand<kTN>(lds_b, read_b[j], chunk);
#pragma unroll
            for (int plane = 0; plane < 3; ++plane) {
                bf16x8 fa[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) fa[i] = read_operand(lds_a + plane * kPlaneBytes, read_a[i], chunk);
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn0 + 32 * j + l32;
            const float s = FORWARD ? a.scale[col] : 1.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + 32 * i + 8 * (r / 4) + 4 * kh + (r % 4);
                a.c[(size_t)row * N + col] = FORWARD ? acc[i][j][r] * s : acc[i][j][r];
            }
        }
}

// The same tile (128 rows x 256 columns) with the two kinds of work on different waves: one
// workgroup of 16 waves per CU, of which waves 0-7 only multiply (32 rows x 128 columns each: per
// slab 24 matrix instructions and 14 operand reads) and waves 8-15 only stage (the slab between
// them: 8 activations and 4 packed groups per thread), two of each kind on every SIMD.  In the
// kernel above every wave stages and then multiplies, the waves of a SIMD do so in step, and the
// matrix pipe idles while they stage (busy 54 % of the cycles); here the SIMD's matrix pipe and
// its vector ALUs work at the same time on different waves (67-72 %).  Two LDS buffers (the stagers
// fill one while the other is multiplied), one barrier per slab.  What made the difference, in
// the order found:
//   - nothing computed from a loaded value inside the fetch (it would wait for the load there),
//     and a steady-state loop without conditions (the compiler's wait counts are the minimum over
//     all paths into a point: one path with fewer loads in flight and every wait drains them), so
//     the stagers' loads stay three to four slabs ahead;
//   - the multiplying waves read the operands of a 16-deep step while the matrix instructions of
//     the step before run (two register sets), and the slab's barrier sits between its two steps;
//   - 32 x 128 wave tiles: 7 operand reads per 12 matrix instructions where 64 x 64 needs 8 (the
//     activation has three planes, so a wave tile should be wide, not tall); LDS instruction
//     count is what the two kinds of wave compete for;
//   - the last-group handling (a byte early, shifted) only in the slabs that can hold that group.
template <bool FORWARD>
__global__ __launch_bounds__(1024, 4) void counter_linear_bf16x3_split_roles_kernel(Lin3Args a) {
    constexpr int CW = 8;  // multiplying waves; as many staging waves
    constexpr int kTN = 256;
    constexpr int kStagers = 64 * CW;                  // threads of the staging waves
    constexpr int kA4 = kT * kK / 4 / kStagers;        // 2 float4 of activation per stager and slab
    constexpr int kW = kTN * kK / 4 / kStagers;        // 4 packed groups per stager and slab
    constexpr int kBufA = 3 * kPlaneBytes, kBufB = kTN * kRowBytes;
    // One array, the table first: its entries are then addressed by their byte offset alone.
    // pair_t[c1 << 6 | c0] = bf16(t(c0)) | bf16(t(c1)) << 16 with t = code / lv - 1
    constexpr int kTableBytes = 4096 * 4;
    __shared__ __attribute__((aligned(16))) uint8_t lds[kTableBytes + 2 * kBufA + 2 * kBufB];
    uint32_t* pair_t = reinterpret_cast<uint32_t*>(lds);
    auto lds_a = [&](int buf) { return lds + kTableBytes + buf * kBufA; };
    auto lds_b = [&](int buf) { return lds + kTableBytes + 2 * kBufA + buf * kBufB; };
    const int tid = threadIdx.x;
    for (int i = tid; i < 4096; i += 128 * CW)
        pair_t[i] = pack_bf16((float)(code_q((uint32_t)i & 63u, a.cd) - 1), (float)(code_q((uint32_t)i >> 6, a.cd) - 1));
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool stager = wave >= CW;  // wave-uniform
    const TileXY tile = xcd_tile(gridDim.x, gridDim.y, 4);
    const int m0 = tile.y * kT, n0 = tile.x * kTN;
    const int K = FORWARD ? a.in_features : a.out_features;
    const int N = FORWARD ? a.out_features : a.in_features;
    const int slabs = K / kK;

    if (stager) {
        constexpr int kRows = kStagers / 8;  // rows of 8 groups one pass of the stagers covers
        const int st = tid - kStagers;
        const int c4 = st & 7, row0 = st >> 3;  // row0 in [0, kRows)
        const uint32_t gpr = (uint32_t)a.in_features >> 2;
        const uint32_t last_off = 3u * ((uint32_t)a.out_features * gpr - 1u);
        uint32_t off_a[kA4], off_w[kW];
        int lds_off_a[kA4], lds_off_b[kW];
#pragma unroll
        for (int p = 0; p < kA4; ++p) {
            const int row = row0 + kRows * p;
            off_a[p] = ((uint32_t)(m0 + row) * (uint32_t)K + 4u * c4) * 4u;
            lds_off_a[p] = tile_offset(row, c4 >> 1, c4 & 1);
        }
#pragma unroll
        for (int p = 0; p < kW; ++p) {
            if (FORWARD) {
                // (weight row n = row0 + kRows p, group c4 of the slab)
                const int n = row0 + kRows * p;
                off_w[p] = 3u * ((uint32_t)(n0 + n) * gpr + (uint32_t)c4);
                lds_off_b[p] = tile_offset(n, c4 >> 1, c4 & 1);
            } else {
                // p = 4 q + r: weight row k = 4 oq + r (oq = c4), group g = row0 + kRows q of the tile's columns;
                // after the transpose, slot 4 q + j holds column 4 g + j
                const int q = p >> 2, r = p & 3, g = row0 + kRows * q;
                off_w[p] = 3u * ((uint32_t)(4 * c4 + r) * gpr + (uint32_t)(n0 >> 2) + (uint32_t)g);
                lds_off_b[p] = dealt_tile_offset<kTN>(4 * g + r, c4 >> 1, c4 & 1);
            }
        }
        const uint32_t w_step = FORWARD ? 3u * (kK / 4) : 3u * kK * gpr;  // packed bytes per slab
        // What a fetch leaves in registers is exactly what the loads return: anything computed from it
        // here would wait for the load at once instead of kAhead slabs later.
        struct Fetched {
            float4 ra[kA4];
            float4 sc;
            uint32_t rw[kW];
        };
        // Only the tensor's last packed group has no byte after it, and it lies in the last slab: the
        // careful forms (which fetch it one byte early and shift) are used for the last slabs only.
        using Careful = std::true_type;
        using Plain = std::false_type;
        auto fetch = [&](auto careful, int slab, Fetched& f) {
            const int k0 = slab * kK;
            const uint32_t w_base = (uint32_t)slab * w_step;
            if (!FORWARD) f.sc = *reinterpret_cast<const float4*>(a.scale + k0 + 4 * c4);
#pragma unroll
            for (int p = 0; p < kA4; ++p)
                f.ra[p] = *reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(a.act) + off_a[p] +
                                                           4u * (uint32_t)k0);
#pragma unroll
            for (int p = 0; p < kW; ++p) {
                uint32_t off = off_w[p] + w_base;  // one 4-byte load per packed group
                if constexpr (decltype(careful)::value) off -= off == last_off ? 1u : 0u;
                __builtin_memcpy(&f.rw[p], a.state + off, 4);
            }
        };
        auto pair_lo = [&](uint32_t word) { return *reinterpret_cast<const uint32_t*>(lds + ((word << 2) & 0x3ffcu)); };
        auto pair_hi = [&](uint32_t word) { return *reinterpret_cast<const uint32_t*>(lds + ((word >> 10) & 0x3ffcu)); };
        auto stage = [&](auto careful, int buf, int slab, const Fetched& f) {
            uint8_t* pa = lds_a(buf);
            uint8_t* pb = lds_b(buf);
            uint32_t rw[kW];
#pragma unroll
            for (int p = 0; p < kW; ++p) {
                rw[p] = f.rw[p];
                if constexpr (decltype(careful)::value)
                    rw[p] >>= off_w[p] + (uint32_t)slab * w_step == last_off ? 8 : 0;
            }
            // all table reads first (their latency passes under the split of the activations), then the
            // writes: both are in the one LDS array, and a read after a write would wait for it
            uint32_t lo[kW], hi[kW];
#pragma unroll
            for (int p = 0; p < kW; ++p) {
                lo[p] = pair_lo(rw[p]);
                hi[p] = pair_hi(rw[p]);
            }
#pragma unroll
            for (int p = 0; p < kA4; ++p) {
                float4 x = f.ra[p];
                // (grad_out * scale) first, as the reference does
                if (!FORWARD) x = make_float4(x.x * f.sc.x, x.y * f.sc.y, x.z * f.sc.z, x.w * f.sc.w);
                store_split(pa, lds_off_a[p], x.x, x.y, x.z, x.w);
            }
            if (FORWARD) {
#pragma unroll
                for (int p = 0; p < kW; ++p) *reinterpret_cast<uint2*>(pb + lds_off_b[p]) = make_uint2(lo[p], hi[p]);
            } else {
#pragma unroll
                for (int q = 0; q < kW / 4; ++q)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {  // codes 2 h, 2 h + 1 of rows k .. k + 3
                        uint32_t pr[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) pr[r] = h == 0 ? lo[4 * q + r] : hi[4 * q + r];
                        const uint32_t lo0 = __builtin_amdgcn_perm(pr[1], pr[0], 0x05040100u);
                        const uint32_t hi0 = __builtin_amdgcn_perm(pr[3], pr[2], 0x05040100u);
                        const uint32_t lo1 = __builtin_amdgcn_perm(pr[1], pr[0], 0x07060302u);
                        const uint32_t hi1 = __builtin_amdgcn_perm(pr[3], pr[2], 0x07060302u);
                        *reinterpret_cast<uint2*>(pb + lds_off_b[4 * q + 2 * h]) = make_uint2(lo0, hi0);
                        *reinterpret_cast<uint2*>(pb + lds_off_b[4 * q + 2 * h + 1]) = make_uint2(lo1, hi1);
                    }
            }
        };
        // Slabs are fetched kAhead ahead of the one being staged (kAhead register sets), so a load has
        // that many slab times to arrive.
        constexpr int kAhead = FORWARD ? 4 : 3;
        Fetched f[kAhead];
#pragma unroll
        for (int d = 0; d < kAhead; ++d) fetch(Plain{}, d, f[d]);
        __syncthreads();  // the table is complete
        stage(Plain{}, 0, 0, f[0]);
        fetch(Plain{}, kAhead, f[0]);  // slabs > 2 kAhead + 1 (the launcher's condition)
        __syncthreads();               // slab 0 is in buffer 0
        // The steady state has no conditions: every path through it has the same loads in flight, so
        // the compiler's wait counts let the newest kAhead - 1 sets stay in flight.  It stops short
        // of fetching the last slab.
        int s = 0;
        for (; s + 2 * kAhead + 1 < slabs; s += kAhead) {
#pragma unroll
            for (int d = 0; d < kAhead; ++d) {
                // while the other waves multiply slab s + d: slab s + d + 1 into the other buffer
                const int nxt = (d + 1) % kAhead;
                stage(Plain{}, (s + d + 1) & 1, s + d + 1, f[nxt]);
                fetch(Plain{}, s + d + 1 + kAhead, f[nxt]);
                __syncthreads();
            }
        }
        for (; s < slabs; s += kAhead) {
#pragma unroll
            for (int d = 0; d < kAhead; ++d) {
                if (s + d >= slabs) break;
                const int nxt = (d + 1) % kAhead;
                if (s + d + 1 < slabs) stage(Careful{}, (s + d + 1) & 1, s + d + 1, f[nxt]);
                if (s + d + 1 + kAhead < slabs) fetch(Careful{}, s + d + 1 + kAhead, f[nxt]);
                __syncthreads();
            }
        }
        return;
    }

    // The multiplying waves, 32 rows x 128 columns each.  A slab is two 16-deep steps; the operands
    // of a step (3 activation reads, 4 weight reads) are read into registers while the matrix
    // instructions of the step before run, so no read's latency is waited for.  The slab's barrier
    // sits between its two steps: by then this wave has read all of the slab (the stagers may
    // overwrite it) and the stagers have finished the next slab (its first step's operands are read
    // during this slab's second step).
    const int l32 = lane & 31, kh = lane >> 5;
    constexpr int kAcross = 2;                 // multiplying waves side by side
    constexpr int kWaveN = kTN / kAcross;      // columns per wave
    constexpr int kWaveM = kT / (CW / kAcross);  // rows per wave
    constexpr int IB = kWaveM / 32, JB = kWaveN / 32;
    constexpr int kReads = 3 * IB + JB, kMfma = 3 * IB * JB;
    const int wm0 = kWaveM * (wave / kAcross), wn0 = kWaveN * (wave % kAcross);
    floatx16 acc[IB][JB];
#pragma unroll
    for (int i = 0; i < IB; ++i)
#pragma unroll
        for (int j = 0; j < JB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    auto read_step = [&](int buf, int c, bf16x8 (&fa)[3][IB], bf16x8 (&fb)[JB]) {
        const uint8_t* pa = lds_a(buf);
        const uint8_t* pb = lds_b(buf);
        const int chunk = 2 * c + kh;  // lane half kh holds k = 8 chunk .. 8 chunk + 7
#pragma unroll
        for (int j = 0; j < JB; ++j)
            fb[j] = FORWARD ? read_operand(pb, wn0 + 32 * j + l32, chunk)
                            : read_dealt_operand<kTN>(pb, wn0 + 32 * j + l32, chunk);
#pragma unroll
        for (int plane = 0; plane < 3; ++plane)
#pragma unroll
            for (int i = 0; i < IB; ++i) fa[plane][i] = read_operand(pa + plane * kPlaneBytes, wm0 + 32 * i + l32, chunk);
    };
    auto multiply_step = [&](const bf16x8 (&fa)[3][IB], const bf16x8 (&fb)[JB]) {
#pragma unroll
        for (int plane = 0; plane < 3; ++plane)
#pragma unroll
            for (int i = 0; i < IB; ++i)
#pragma unroll
                for (int j = 0; j < JB; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[plane][i], fb[j], acc[i][j], 0, 0, 0);
    };
    // the matrix instructions of a step with the operand reads of the next step between the first of
    // them, so the reads have landed when the step ends
    auto interleave = [&]() {
#pragma unroll
        for (int g = 0; g < kReads; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // matrix
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // LDS read
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kMfma - kReads, 0);
    };
    bf16x8 fa0[3][IB], fb0[JB], fa1[3][IB], fb1[JB];
    __syncthreads();  // the table is complete (the stagers' barrier)
    __syncthreads();  // slab 0 is in buffer 0
    read_step(0, 0, fa0, fb0);
    for (int s = 0; s < slabs; ++s) {
        read_step(s & 1, 1, fa1, fb1);
        multiply_step(fa0, fb0);
        interleave();
        __builtin_amdgcn_sched_barrier(0);  // all of the step before the barrier: its last reads land meanwhile
        __syncthreads();
        read_step((s + 1) & 1, 0, fa0, fb0);  // after the last slab: read and never used
        multiply_step(fa1, fb1);
        interleave();
    }
#pragma unroll
    for (int i = 0; i < IB; ++i)
#pragma unroll
        for (int j = 0; j < JB; ++j) {
            const int col = n0 + wn0 + 32 * j + l32;
            const float sv = FORWARD ? a.scale[col] : 1.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + 32 * i + 8 * (r / 4) + 4 * kh + (r % 4);
                a.c[(size_t)row * N + col] = FORWARD ? acc[i][j][r] * sv : acc[i][j][r];
            }
        }
}

// Any shape: every access is checked and short slabs are zero-filled.
template <bool FORWARD, bool VEC_A>
__global__ __launch_bounds__(kGemmThreads, 3) void counter_linear_bf16x3_edge_kernel(Lin3Args a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[3 * kPlaneBytes];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[kPlaneBytes];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, kh = lane >> 5;
    const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
    const int m0 = blockIdx.y * kT, n0 = blockIdx.x * kT;
    const int K = FORWARD ? a.in_features : a.out_features;
    const int N = FORWARD ? a.out_features : a.in_features;
    const int gpr = a.in_features >> 2;
    const size_t last_group = (size_t)a.out_features * gpr - 1;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // staging registers of one slab: 4 float4 of activation and 4 packed groups per thread
    float4 ra[4];
    uint32_t rw[4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int idx = tid + kGemmThreads * p;
            const int row = idx >> 3, c4 = idx & 7;
            float4 x = load4<VEC_A>(a.act, m0 + row, k0 + 4 * c4, a.rows, K, K);
            if (!FORWARD) {  // (grad_out * scale) first, as the reference does
                const int o = k0 + 4 * c4;
                x.x = x.x * (o + 0 < K ? a.scale[o + 0] : 0.0f);
                x.y = x.y * (o + 1 < K ? a.scale[o + 1] : 0.0f);
                x.z = x.z * (o + 2 < K ? a.scale[o + 2] : 0.0f);
                x.w = x.w * (o + 3 < K ? a.scale[o + 3] : 0.0f);
            }
            ra[p] = x;
        }
        if (FORWARD) {
            // thread -> (output row n, group g of the slab): 4 consecutive k of one weight row
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int idx = tid + kGemmThreads * p;
                const int o = n0 + (idx >> 3), g = (k0 >> 2) + (idx & 7);
                rw[p] = fetch_group(a.state, (size_t)o * gpr + g, last_group, o < a.out_features && g < gpr);
            }
        } else {
            // thread -> (4 consecutive weight rows o = k, group g of the tile's columns)
            const int oq = tid & 7, g = (n0 >> 2) + (tid >> 3);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int o = k0 + 4 * oq + r;
                rw[r] = fetch_group(a.state, (size_t)o * gpr + g, last_group, o < a.out_features && g < gpr);
            }
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int idx = tid + kGemmThreads * p;
            const int row = idx >> 3, c4 = idx & 7;
            store_split(lds_a, tile_offset(row, c4 >> 1, c4 & 1), ra[p].x, ra[p].y, ra[p].z, ra[p].w);
        }
        if (FORWARD) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int idx = tid + kGemmThreads * p;
                const int n = idx >> 3, g = idx & 7;
                const uint32_t lo = pack_bf16(ternary_of(rw[p], 0, a.cd), ternary_of(rw[p], 1, a.cd));
                const uint32_t hi = pack_bf16(ternary_of(rw[p], 2, a.cd), ternary_of(rw[p], 3, a.cd));
                *reinterpret_cast<uint2*>(lds_b + tile_offset(n, g >> 1, g & 1)) = make_uint2(lo, hi);
            }
        } else {
            const int oq = tid & 7, g = tid >> 3;
#pragma unroll
            for (int j = 0; j < 4; ++j) {  // column n = 4 g + j of the tile, k = 4 oq .. 4 oq + 3
                const uint32_t lo = pack_bf16(ternary_of(rw[0], j, a.cd), ternary_of(rw[1], j, a.cd));
                const uint32_t hi = pack_bf16(ternary_of(rw[2], j, a.cd), ternary_of(rw[3], j, a.cd));
                *reinterpret_cast<uint2*>(lds_b + tile_offset(4 * g + j, oq >> 1, oq & 1)) = make_uint2(lo, hi);
            }
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += kK) {
        stage();
        __syncthreads();
        if (k0 + kK < K) fetch(k0 + kK);
#pragma unroll
        for (int s = 0; s < kK / 16; ++s) {
            const int chunk = 2 * s + kh;  // lane half kh holds k = 8 chunk .. 8 chunk + 7
            bf16x8 fb[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) fb[j] = read_operand(lds_b, wn0 + 32 * j + l32, chunk);
#pragma unroll
            for (int plane = 0; plane < 3; ++plane) {
                bf16x8 fa[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) fa[i] = read_operand(lds_a + plane * kPlaneBytes, wm0 + 32 * i + l32, chunk);
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn0 + 32 * j + l32;
            const float s = (FORWARD && col < N) ? a.scale[col] : 1.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + 32 * i + 8 * (r / 4) + 4 * kh + (r % 4);
                if (row < a.rows && col < N) a.c[(size_t)row * N + col] = FORWARD ? acc[i][j][r] * s : acc[i][j][r];
            }
        }
}

template <bool FORWARD>
hipError_t launch_lin3(hipStream_t stream, const float* act, const uint8_t* state, const float* scale, float* c,
                       int C, int rows, int in_features, int out_features) {
    Lin3Args a;
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
    const bool vec_a = (K % 4 == 0) && ((reinterpret_cast<uintptr_t>(act) & 15u) == 0);
    const dim3 edge_block(kGemmThreads);
    auto launch_edge = [&](const Lin3Args& e) {
        const dim3 grid((N + kT - 1) / kT, (e.rows + kT - 1) / kT);
        if (vec_a)
            hipLaunchKernelGGL((counter_linear_bf16x3_edge_kernel<FORWARD, true>), grid, edge_block, 0, stream, e);
        else
            hipLaunchKernelGGL((counter_linear_bf16x3_edge_kernel<FORWARD, false>), grid, edge_block, 0, stream, e);
        return hipGetLastError();
    };
    // whole 128-column tiles and whole slabs, aligned operands, a packed weight below 4 GiB
    const bool shape_whole = N % kT == 0 && K % kK == 0 && vec_a && (reinterpret_cast<uintptr_t>(scale) & 15u) == 0 &&
                             (uint64_t)out_features * (uint64_t)in_features * 3u / 4u < (1ull << 32);
    if (!shape_whole || rows < kT) return launch_edge(a);
    // The unchecked kernels take whole 128-row tiles and address the activations with 32-bit byte
    // offsets: the rows go out in launches of whole tiles below 4 GiB of activations each, and a
    // ragged rest of fewer than 128 rows goes to the checked kernel.
    // (and the grid's y extent is at most 65535 tiles)
    const uint64_t fit_rows = ((1ull << 32) - 1) / ((uint64_t)K * 4u) / kT * kT;
    const int max_rows = (int)(fit_rows < 65535ull * kT ? fit_rows : 65535ull * kT);
    const int whole_rows = rows / kT * kT;
    if (max_rows < kT) return launch_edge(a);
    for (int r0 = 0; r0 < whole_rows; r0 += max_rows) {
        Lin3Args w = a;
        w.rows = whole_rows - r0 < max_rows ? whole_rows - r0 : max_rows;
        w.act = act + (size_t)r0 * K;
        w.c = c + (size_t)r0 * N;
        // 256-column tiles share one split of the activation slab between twice as many columns:
        // +15 % when there are enough of them to fill the device
        if (N % 256 == 0 && (long)(w.rows / kT) * (N / 256) >= 256) {
            // 16 slabs or more: the staging waves run four slabs ahead
            if (K >= 16 * kK)
                hipLaunchKernelGGL((counter_linear_bf16x3_split_roles_kernel<FORWARD>), dim3(N / 256, w.rows / kT),
                                   dim3(1024), 0, stream, w);
            else
                hipLaunchKernelGGL((counter_linear_bf16x3_kernel<FORWARD, 4>), dim3(N / 256, w.rows / kT), dim3(512), 0,
                                   stream, w);
        } else {
            hipLaunchKernelGGL((counter_linear_bf16x3_kernel<FORWARD, 2>), dim3(N / kT, w.rows / kT), dim3(kGemmThreads), 0,
                               stream, w);
        }
        const hipError_t err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    if (rows > whole_rows) {
        Lin3Args e = a;
        e.rows = rows - whole_rows;
        e.act = act + (size_t)whole_rows * K;
        e.c = c + (size_t)whole_rows * N;
        return launch_edge(e);
    }
    return hipSuccess;
}

}  // namespace

hipError_t launch_forward(hipStream_t stream, const float* x, const uint8_t* state, const float* scale, float* y,
                          int C, int batch, int in_features, int out_features) {
    return launch_lin3<true>(stream, x, state, scale, y, C, batch, in_features, out_features);
}

hipError_t launch_backward_input(hipStream_t stream, const float* grad_out, const uint8_t* state,
                                 const float* scale, float* grad_x, int C, int batch, int in_features,
                                 int out_features) {
    return launch_lin3<false>(stream, grad_out, state, scale, grad_x, C, batch, in_features, out_features);
}

}  // namespace mcc
