// The 256 x 256 tile of the fp32 matrix-core contraction c[m,n] = sum_k a[k,m] * b[k,n]: lane
// layout, accumulators and the main loop, shared by the contraction kernels
// (gemm_tn_f32_wide.hip) and the fused strip kernel on wide tiles (counter_fused_strip.hip).
// 8 waves (2 down x 4 across, 128 x 64 each); slabs of 16 tokens are copied straight into one of
// four LDS buffers (global_load_lds_dwordx4).
//
// Operand layout.  v_mfma_f32_32x32x2_f32 takes one float per lane from each operand; which matrix
// row a lane's float belongs to is the kernel's choice.  Here lane l of the wave's four 32-row
// blocks supplies rows 4 l .. 4 l + 3 (one per block) and columns 2 l, 2 l + 1, so a step's six
// operand floats are one 16-byte and one 8-byte LDS read instead of six 4-byte ones; the
// accumulators then hold a permuted tile: acc[i][j][r] is row wm0 + 4 (8 (r/4) + 4 half + r%4) + i,
// column wn0 + 2 l32 + j of the tile.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "gemm_tile.hpp"

namespace mcc {

constexpr int kWide = 256;
constexpr int kWideThreads = 512;
constexpr int kWideSlabFloats = kBK * 2 * kWide;  // 16 tokens of both operands: 32 KiB
constexpr int kWideBuffers = 4;                   // slabs in LDS: 128 KiB of the CU's 160

struct WideLane {
    int tid, lane, wave, l32, half, wm0, wn0;
};

__device__ __forceinline__ WideLane wide_lane() {
    WideLane t;
    t.tid = threadIdx.x;
    t.lane = t.tid & 63;
    t.wave = t.tid >> 6;
    t.l32 = t.lane & 31;
    t.half = t.lane >> 5;
    t.wm0 = (t.wave >> 2) * 128;
    t.wn0 = (t.wave & 3) * 64;
    return t;
}

typedef floatx16 WideAcc[4][2];

#define MCC_WIDE_KERNEL __global__ __launch_bounds__(kWideThreads, 2)

__device__ __forceinline__ void wide_zero(WideAcc& acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
}

// ------------------------------------------------------------------------------ main loop
// The slab loop is written in assembly.  Left to the compiler, every step's operand reads are
// followed at once by s_waitcnt lgkmcnt(0), whatever read-ahead the source spells out, each slab
// begins with a barrier followed by a full LDS latency with the matrix pipes idle, and the copies
// of the next slab are issued between two slabs by both waves of a SIMD at the same moment, whose
// address arithmetic leaves the matrix pipe idle.  Measured on 4096 x 4096 at 32768 tokens: the
// compiler's loop 91.8 % of the peak; matrix instructions, operand reads and barriers alone (no
// copies, no operands from memory) 98.5 %; this loop 96.6 %, and 98 % with its copies left out.
//
// Registers.  A step's operands sit in fixed registers -- set 0 in v[232:235] (a) and v[240:241]
// (b), set 1 in v[236:239] and v[242:243] -- because an assembly operand cannot name one register
// of a tuple that a 16-byte LDS read fills.  They are clobbers of the one statement that holds the
// whole loop, so nothing of them is live outside it.
//
// The eight matrix instructions of one step (two tokens): accumulator (i, j) takes operand row
// block i and column block j.
#define MCC_WIDE_MFMA(C, A, B) "v_mfma_f32_32x32x2_f32 %[" C "], " A ", " B ", %[" C "]\n"
#define MCC_WIDE_USE0                                                                               \
    MCC_WIDE_MFMA("c00", "v232", "v240") MCC_WIDE_MFMA("c01", "v232", "v241") MCC_WIDE_MFMA("c10", "v233", "v240") \
    MCC_WIDE_MFMA("c11", "v233", "v241") MCC_WIDE_MFMA("c20", "v234", "v240") MCC_WIDE_MFMA("c21", "v234", "v241") \
    MCC_WIDE_MFMA("c30", "v235", "v240") MCC_WIDE_MFMA("c31", "v235", "v241")
#define MCC_WIDE_USE1                                                                               \
    MCC_WIDE_MFMA("c00", "v236", "v242") MCC_WIDE_MFMA("c01", "v236", "v243") MCC_WIDE_MFMA("c10", "v237", "v242") \
    MCC_WIDE_MFMA("c11", "v237", "v243") MCC_WIDE_MFMA("c20", "v238", "v242") MCC_WIDE_MFMA("c21", "v238", "v243") \
    MCC_WIDE_MFMA("c30", "v239", "v242") MCC_WIDE_MFMA("c31", "v239", "v243")
// Operand reads of step STEP of the buffer at byte offset BUF from the address registers VA / VB
// into a set: 16 bytes of a and 8 bytes of b per lane, 2048 bytes on per step, b 16 KiB after a.
#define MCC_WIDE_READ0(VA, VB, BUF, STEP)                               \
    "ds_read_b128 v[232:235], " VA " offset:" #BUF "+2048*" #STEP "\n" \
    "ds_read_b64 v[240:241], " VB " offset:" #BUF "+16384+2048*" #STEP "\n"
#define MCC_WIDE_READ1(VA, VB, BUF, STEP)                               \
    "ds_read_b128 v[236:239], " VA " offset:" #BUF "+2048*" #STEP "\n" \
    "ds_read_b64 v[242:243], " VB " offset:" #BUF "+16384+2048*" #STEP "\n"
#define MCC_WIDE_AHEAD "s_waitcnt lgkmcnt(2)\n"  // all reads but the two just issued have returned
// A step's matrix instructions with two of the wave's copies in their shadow: 16 bytes per lane
// from the addresses in P0 and P1 to the LDS addresses dst + D0 and dst + D1.
#define MCC_WIDE_MFMA8_COPY(A0, A1, A2, A3, B0, B1, D0, P0, D1, P1)          \
    "s_add_u32 m0, %[dst], " #D0 "\n"                                        \
    MCC_WIDE_MFMA("c00", A0, B0)                                             \
    "global_load_lds_dwordx4 " P0 ", off\n"                                  \
    "s_add_u32 m0, %[dst], " #D1 "\n"                                        \
    MCC_WIDE_MFMA("c01", A0, B1) MCC_WIDE_MFMA("c10", A1, B0)                \
    "global_load_lds_dwordx4 " P1 ", off\n"                                  \
    MCC_WIDE_MFMA("c11", A1, B1) MCC_WIDE_MFMA("c20", A2, B0) MCC_WIDE_MFMA("c21", A2, B1) \
    MCC_WIDE_MFMA("c30", A3, B0) MCC_WIDE_MFMA("c31", A3, B1)
#define MCC_WIDE_USE0_COPY(D0, P0, D1, P1) MCC_WIDE_MFMA8_COPY("v232", "v233", "v234", "v235", "v240", "v241", D0, P0, D1, P1)
#define MCC_WIDE_USE1_COPY(D0, P0, D1, P1) MCC_WIDE_MFMA8_COPY("v236", "v237", "v238", "v239", "v242", "v243", D0, P0, D1, P1)
// USE (a set's eight matrix instructions), with the two copies if this wave's turn (%[go]) is TURN
#define MCC_WIDE_USE_OR_COPY(ID, K, TURN, USE, USE_COPY)                  \
    "s_cmp_eq_u32 %[go], " #TURN "\n"                                     \
    "s_cbranch_scc0 .Lmcc_wide_plain" #ID #K "_%=\n"                      \
    USE_COPY                                                              \
    "s_branch .Lmcc_wide_join" #ID #K "_%=\n"                             \
    ".Lmcc_wide_plain" #ID #K "_%=:\n"                                    \
    USE                                                                   \
    ".Lmcc_wide_join" #ID #K "_%=:\n"
// One slab out of the buffer (VA, VB, BUF); the next one is in (VAN, VBN, BUFN), and DST is the
// byte offset of the buffer three on, which held the slab before this one.  On entry the reads
// of step 0 are in flight (set 0); every step first issues the reads of the step after it into
// the other set and then waits for its own, so a wave never waits for a read it has only just
// issued.  Before the last step every wave waits for its own reads, for its copies of the next
// slab (those of the two slabs after it may stay in flight) and for the other waves; the last
// step's read-ahead is step 0 of the next slab.  The barrier therefore also says that nobody
// reads this slab's buffer any more, and the next slab may fill it: if there is a slab three
// ahead, the wave issues its four copies of it (rows wave and wave + 8 of a from pa0 and pa1, of
// b from pb0 and pb1, to LDS address dst + DST + 0, 8, 16, 24 KiB) in the first four steps, each
// in the shadow of a matrix instruction.  The copy unit takes a few dozen cycles per instruction
// and a wave that waits for it issues nothing else, so the two waves of a SIMD take turns: waves
// 0-3 copy in steps 0 and 2, waves 4-7 in steps 1 and 3 (%[ph]), and the matrix pipe always has
// one wave that is not copying.  (All eight waves copying in the same step: 1 % slower; copies
// between the slabs, outside the matrix instructions: 3 % slower.)
#define MCC_WIDE_SLAB(ID, VA, VB, BUF, VAN, VBN, BUFN, DST)                            \
    "s_add_u32 %[t], %[i], 3\n"                                                        \
    "s_cmp_lt_u32 %[t], %[n]\n"                                                        \
    "s_cselect_b32 %[go], %[ph], 2\n"                                                  \
    MCC_WIDE_READ1(VA, VB, BUF, 1) MCC_WIDE_AHEAD                                      \
    MCC_WIDE_USE_OR_COPY(ID, 0, 0, MCC_WIDE_USE0, MCC_WIDE_USE0_COPY(DST, "%[pa0]", DST+0x2000, "%[pa1]")) \
    MCC_WIDE_READ0(VA, VB, BUF, 2) MCC_WIDE_AHEAD                                      \
    MCC_WIDE_USE_OR_COPY(ID, 1, 1, MCC_WIDE_USE1, MCC_WIDE_USE1_COPY(DST, "%[pa0]", DST+0x2000, "%[pa1]")) \
    MCC_WIDE_READ1(VA, VB, BUF, 3) MCC_WIDE_AHEAD                                      \
    MCC_WIDE_USE_OR_COPY(ID, 2, 0, MCC_WIDE_USE0, MCC_WIDE_USE0_COPY(DST+0x4000, "%[pb0]", DST+0x6000, "%[pb1]")) \
    MCC_WIDE_READ0(VA, VB, BUF, 4) MCC_WIDE_AHEAD                                      \
    MCC_WIDE_USE_OR_COPY(ID, 3, 1, MCC_WIDE_USE1, MCC_WIDE_USE1_COPY(DST+0x4000, "%[pb0]", DST+0x6000, "%[pb1]")) \
    "v_lshl_add_u64 %[pa0], %[pa0], 0, %[sa]\n"                                        \
    "v_lshl_add_u64 %[pa1], %[pa1], 0, %[sa]\n"                                        \
    "v_lshl_add_u64 %[pb0], %[pb0], 0, %[sb]\n"                                        \
    "v_lshl_add_u64 %[pb1], %[pb1], 0, %[sb]\n"                                        \
    MCC_WIDE_READ1(VA, VB, BUF, 5) MCC_WIDE_AHEAD MCC_WIDE_USE0                        \
    MCC_WIDE_READ0(VA, VB, BUF, 6) MCC_WIDE_AHEAD MCC_WIDE_USE1                        \
    MCC_WIDE_READ1(VA, VB, BUF, 7) MCC_WIDE_AHEAD MCC_WIDE_USE0                        \
    "s_cmp_lt_u32 %[t], %[n]\n"                                                        \
    "s_cbranch_scc0 .Lmcc_wide_two" #ID "_%=\n"                                        \
    "s_waitcnt vmcnt(8) lgkmcnt(0)\n"                                                  \
    "s_branch .Lmcc_wide_landed" #ID "_%=\n"                                           \
    ".Lmcc_wide_two" #ID "_%=:\n"                                                      \
    "s_add_u32 %[t], %[i], 2\n"                                                        \
    "s_cmp_lt_u32 %[t], %[n]\n"                                                        \
    "s_cbranch_scc0 .Lmcc_wide_one" #ID "_%=\n"                                        \
    "s_waitcnt vmcnt(4) lgkmcnt(0)\n"                                                  \
    "s_branch .Lmcc_wide_landed" #ID "_%=\n"                                           \
    ".Lmcc_wide_one" #ID "_%=:\n"                                                      \
    "s_waitcnt vmcnt(0) lgkmcnt(0)\n"                                                  \
    ".Lmcc_wide_landed" #ID "_%=:\n"                                                   \
    "s_barrier\n"                                                                      \
    MCC_WIDE_READ0(VAN, VBN, BUFN, 0)                                                  \
    MCC_WIDE_USE1                                                                      \
    "s_add_u32 %[i], %[i], 1\n"                                                        \
    "s_cmp_lt_u32 %[i], %[n]\n"

// acc += the products of k_len tokens (a multiple of 16, at least 16); a and b point at the first
// token's row, at the tile's first column.  The caller separates two calls by __syncthreads():
// the first copies of a call go to buffers that waves still in the previous call's last slab may
// read.
//
// LDS holds kWideBuffers = 4 slabs.  The barrier of slab s says that slab s + 1 has landed and
// that nobody reads slab s any more, so the copies of slab s + 4 go into that buffer during the
// first steps of slab s + 1 and have two and a half slabs' time to land.  Buffers 0 and 1 are addressed from one
// pair of address registers, 2 and 3 from another 64 KiB on (the offset field of an LDS read has
// 16 bits), so the loop body is four slabs with constant offsets and the per-slab work outside
// the matrix instructions is a handful of scalar instructions.
__device__ __forceinline__ void wide_accumulate(const float* __restrict__ a, const float* __restrict__ b, int M, int N,
                                                int k_len, WideAcc& acc, float* lds, const WideLane& t) {
    typedef __attribute__((address_space(3))) void* lds_ptr;
    typedef const __attribute__((address_space(1))) void* global_ptr;
    static_assert(kWideBuffers == 4 && kWideSlabFloats * 4 == 32768, "the assembly below spells these out");
    const int slabs = __builtin_amdgcn_readfirstlane(k_len / kBK);
    // a slab is 32 rows of 1 KiB (16 token rows of a, then 16 of b); wave w copies rows w and
    // w + 8 of each, lane l the floats 4 l .. 4 l + 3 of the row
    const float* a_next = a + (size_t)t.wave * M + 4 * t.lane;
    const float* b_next = b + (size_t)t.wave * N + 4 * t.lane;
    // the waits below count this call's copies: nothing older may be in flight (loads and stores
    // share the counter and are not ordered against each other)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    for (int s = 0; s < kWideBuffers - 1 && s < slabs; ++s) {
        float* dst = lds + s * kWideSlabFloats + t.wave * kWide;
        __builtin_amdgcn_global_load_lds((global_ptr)a_next, (lds_ptr)dst, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((global_ptr)(a_next + (size_t)8 * M), (lds_ptr)(dst + 8 * kWide), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((global_ptr)b_next, (lds_ptr)(dst + kBK * kWide), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((global_ptr)(b_next + (size_t)8 * N), (lds_ptr)(dst + (kBK + 8) * kWide), 16, 0,
                                         0);
        a_next += (size_t)kBK * M;
        b_next += (size_t)kBK * N;
    }
    // four copy instructions per wave and slab: wait for slab 0 only
    if (slabs >= 3) asm volatile("s_waitcnt vmcnt(8)\n s_barrier" ::: "memory");
    else if (slabs == 2) asm volatile("s_waitcnt vmcnt(4)\n s_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");

    // LDS byte addresses of this lane's operands in step 0 of buffers 0 and 2: token 2 kk + half of
    // step kk, rows wm0 + 4 l32 .. + 3 of a, columns wn0 + 2 l32, + 1 of b
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr)lds;
    const uint32_t va = lds0 + 4u * (uint32_t)(t.half * kWide + t.wm0 + 4 * t.l32);
    const uint32_t vb = lds0 + 4u * (uint32_t)(t.half * kWide + t.wn0 + 2 * t.l32);
    const uint32_t dst = lds0 + (uint32_t)__builtin_amdgcn_readfirstlane(t.wave) * (4u * kWide);
    uint64_t pa0 = (uint64_t)a_next, pa1 = (uint64_t)(a_next + (size_t)8 * M);
    uint64_t pb0 = (uint64_t)b_next, pb1 = (uint64_t)(b_next + (size_t)8 * N);
    const uint64_t sa = (uint64_t)kBK * (uint64_t)M * 4u, sb = (uint64_t)kBK * (uint64_t)N * 4u;
    const int turn = __builtin_amdgcn_readfirstlane(t.wave >> 2);
    int i, tmp, go;
    asm volatile(
        "s_mov_b32 %[i], 0\n"
        MCC_WIDE_READ0("%[va]", "%[vb]", 0, 0)
        ".Lmcc_wide_loop_%=:\n"
        MCC_WIDE_SLAB(0, "%[va]", "%[vb]", 0, "%[va]", "%[vb]", 32768, 98304)
        "s_cbranch_scc0 .Lmcc_wide_exit_%=\n"
        MCC_WIDE_SLAB(1, "%[va]", "%[vb]", 32768, "%[va2]", "%[vb2]", 0, 0)
        "s_cbranch_scc0 .Lmcc_wide_exit_%=\n"
        MCC_WIDE_SLAB(2, "%[va2]", "%[vb2]", 0, "%[va2]", "%[vb2]", 32768, 32768)
        "s_cbranch_scc0 .Lmcc_wide_exit_%=\n"
        MCC_WIDE_SLAB(3, "%[va2]", "%[vb2]", 32768, "%[va]", "%[vb]", 0, 65536)
        "s_cbranch_scc1 .Lmcc_wide_loop_%=\n"
        ".Lmcc_wide_exit_%=:\n"
        // the read-ahead of the last slab (nothing uses it), and the results of the last matrix
        // instructions: 18 wait states before another kind of instruction may read them
        "s_waitcnt lgkmcnt(0)\n"
        "s_nop 15\n"
        "s_nop 7\n"
        : [c00] "+v"(acc[0][0]), [c01] "+v"(acc[0][1]), [c10] "+v"(acc[1][0]), [c11] "+v"(acc[1][1]),
          [c20] "+v"(acc[2][0]), [c21] "+v"(acc[2][1]), [c30] "+v"(acc[3][0]), [c31] "+v"(acc[3][1]), [pa0] "+v"(pa0),
          [pa1] "+v"(pa1), [pb0] "+v"(pb0), [pb1] "+v"(pb1), [i] "=&s"(i), [t] "=&s"(tmp), [go] "=&s"(go)
        : [va] "v"(va), [vb] "v"(vb), [va2] "v"(va + 65536u), [vb2] "v"(vb + 65536u), [n] "s"(slabs), [dst] "s"(dst),
          [sa] "s"(sa), [sb] "s"(sb), [ph] "s"(turn)
        : "memory", "scc", "m0", "v232", "v233", "v234", "v235", "v236", "v237", "v238", "v239", "v240", "v241", "v242",
          "v243");
}

}  // namespace mcc
