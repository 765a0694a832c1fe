// Pieces shared by the kernels that run binary32 data on the bf16 matrix cores by splitting each
// number into three bf16 terms:
//     x = hi + mid + lo,   hi = bf16(x),  mid = bf16(x - hi),  lo = bf16(x - hi - mid)
// Each subtraction is exact (24 significant bits are peeled off 8 at a time; only numbers within
// 2^16 of the smallest normal lose their tail), and a bf16 x bf16 product is exact in binary32.
// Operand tiles live in LDS as [row][32 bf16] = 64-byte rows whose four 16-byte chunks are
// XOR-swizzled with bits 2-3 of the row.  A 16-byte operand read (lane = row, 8 consecutive k) is
// served 16 lanes a cycle, all 64 banks at once: rows r, r + 4, r + 8, r + 12 start in the same
// banks and the swizzle sends them to four different chunks, so the read is conflict-free
// without padding (measured: SQ_LDS_BANK_CONFLICT drops from half of the LDS cycles to none).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mcc {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kT = 128;        // tile rows
constexpr int kK = 32;         // slab depth
constexpr int kRowBytes = 64;  // 32 bf16
constexpr int kPlaneBytes = kT * kRowBytes;

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    const bf16x2 p = {(__bf16)a, (__bf16)b};  // round to nearest even
    return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ float bf16_lo(uint32_t p) { return __uint_as_float(p << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t p) { return __uint_as_float(p & 0xffff0000u); }

// Byte offset of 8-byte piece `half` of 16-byte chunk `chunk` of row `row` in a swizzled tile.
__device__ __forceinline__ int tile_offset(int row, int chunk, int half) {
    return row * kRowBytes + ((chunk ^ ((row >> 2) & 3)) << 4) + (half << 3);
}

// The same for a stager that transposes: its wave writes, in one instruction, 8-byte pieces of
// rows r, r + 4, ..., r + 28.  In the layout above those rows are 256 bytes -- one sweep of the
// banks -- apart and the write is an 8-way bank conflict.  Here row r sits at position
// (r % 4) * 32 + r / 4, so the eight rows are 512 contiguous bytes; the chunk swizzle (r % 4, and
// bit 4 of r so that rows 16 apart differ) keeps both those writes and the operand reads
// (consecutive rows, one chunk) conflict-free.
template <int ROWS = kT>
__device__ __forceinline__ int dealt_tile_offset(int row, int chunk, int half) {
    static_assert(ROWS % 16 == 0, "a quarter of the tile must be whole bank sweeps");
    const int swizzle = (row & 3) ^ ((row >> 3) & 2);
    return (((row & 3) * (ROWS / 4)) + (row >> 2)) * kRowBytes + ((chunk ^ swizzle) << 4) + (half << 3);
}

// Splits four activations into their three bf16 planes and stores each as 8 bytes.
__device__ __forceinline__ void store_split(uint8_t* planes, int offset, float x0, float x1, float x2, float x3) {
    const uint32_t h01 = pack_bf16(x0, x1), h23 = pack_bf16(x2, x3);
    const float r0 = x0 - bf16_lo(h01), r1 = x1 - bf16_hi(h01), r2 = x2 - bf16_lo(h23), r3 = x3 - bf16_hi(h23);
    const uint32_t m01 = pack_bf16(r0, r1), m23 = pack_bf16(r2, r3);
    const float s0 = r0 - bf16_lo(m01), s1 = r1 - bf16_hi(m01), s2 = r2 - bf16_lo(m23), s3 = r3 - bf16_hi(m23);
    const uint32_t l01 = pack_bf16(s0, s1), l23 = pack_bf16(s2, s3);
    *reinterpret_cast<uint2*>(planes + offset) = make_uint2(h01, h23);
    *reinterpret_cast<uint2*>(planes + kPlaneBytes + offset) = make_uint2(m01, m23);
    *reinterpret_cast<uint2*>(planes + 2 * kPlaneBytes + offset) = make_uint2(l01, l23);
}

__device__ __forceinline__ bf16x8 read_operand(const uint8_t* tile, int row, int chunk) {
    const uint4 v = *reinterpret_cast<const uint4*>(tile + tile_offset(row, chunk, 0));
    return __builtin_bit_cast(bf16x8, v);
}
template <int ROWS = kT>
__device__ __forceinline__ bf16x8 read_dealt_operand(const uint8_t* tile, int row, int chunk) {
    const uint4 v = *reinterpret_cast<const uint4*>(tile + dealt_tile_offset<ROWS>(row, chunk, 0));
    return __builtin_bit_cast(bf16x8, v);
}

}  // namespace mcc
