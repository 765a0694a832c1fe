// Fused step without a weight-sized gradient buffer: the fp32 MFMA contraction
//     G[o,i] = sum_r grad_out[r,o] * x[r,i]
// keeps each 128 x 128 tile of G in its accumulators and applies the counter update to the
// packed state straight from them.
//
// The obstacle is that every tick needs its row's denominator, i.e. the sum of squares over the
// WHOLE row of G (kernels/compact_counter.cl:92-99 before :118), while a tile sees 128 columns.
// The tiles of one 128-row strip therefore cooperate through a small strip scratch:
//
//   * The reference sums a row as 64 strided chains (chain l takes packed groups l, l+64, ...,
//     kernels/compact_counter.cl:75-83) and then a binary tree (:88-91).  A tile's 128 columns
//     are 32 consecutive groups, so tile ct of a strip holds exactly step ct/2 of the chains
//     32*(ct%2) .. 32*(ct%2)+31 of its 128 rows.  Tile ct waits until tile ct-2 has published
//     those chains, adds its four squares per group in element order, and publishes them for
//     tile ct+2.  The even and the odd tiles form two independent hand-off sequences.
//   * When both sequences have reached the end of the strip, every tile reads the 64 final chain
//     values of each of its rows, runs the binary tree and the row epilogue itself, and applies
//     the ticks to its own columns.  Tile 0 of the strip commits v and scale.
//
// The sums are the reference's, operation for operation, so the result is bit-identical to the
// two-kernel path (contraction into a workspace, then the update kernel) on the same inputs.
//
// Workgroups are persistent: workgroup b takes tiles b, b + grid, b + 2 grid, ... of the
// strip-major tile order.  A tile waits only for tiles of its own strip; a strip's tiles have
// consecutive indices and a strip has no more tiles than the grid has workgroups, so the
// workgroups that hold the lowest unfinished strip are all running and it always completes,
// provided the whole grid is resident (the launch sizes it from the occupancy query).  Every
// wait is bounded: a workgroup that exhausts its spin budget raises the status word, which
// ends all waits, and the host reports the failure.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <mutex>

#include "counter_math.hpp"
#include "gemm_tile.hpp"
#include "gemm_wide_tile.hpp"
#include "launch.hpp"
#include "wave_ops.hpp"

namespace mcc {
namespace {

constexpr int kTile = 128;             // rows and columns of G per tile
constexpr int kGroupsPerTile = kTile / 4;
constexpr int kNapsPerHandOff = 2;  // s_sleep(32) units (about 0.9 us each) slept per pending hand-off
constexpr int kChainSetFloats = 2 * kTile * kGroupsPerTile;  // both parities, 128 rows x 32 chains
constexpr int kStripChainFloats = 2 * kChainSetFloats;       // the sums of g^2 and of g*t

// Per-strip control words.  A strip is updated all or nothing: `decision` goes from 0 to +1 when
// both hand-off sequences have reached the end of the strip (set by the tile that completes the
// second one) or to -1 when a tile gives up; no tile writes a tick, v or scale before it has read +1.
struct StripControl {
    int published[2];  // tiles of each parity that have published their chains
    int sequences_done;
    int decision;
};

struct StripArgs {
    uint8_t* state;
    float* scale;
    float* v;
    const float* grad_out;
    const float* x;
    int* status;            // launch-local: raised by the first workgroup that gives up, ends all waits
    int* failures;          // the library's per-device count of strip launches' workgroups that gave up
    StripControl* control;  // [strip]
    float* chain;           // [strip][g^2, g*t][parity][128][32]
    float* park;            // wide tiles: slots for tiles whose strip ends in a later pass (nullptr: none)
    int park_first_wg;      // ... the first workgroup that has slots (two each)
    int tokens, in_features, out_features;
    int tiles_per_strip, total_tiles;
    int layer_wgs;  // workgroups the device takes in per residency layer (its CU count)
    unsigned spin_limit;
    Codec cd;
    LutGeom geom;
    float lr, lr_scale, rms_beta, rms_eps;
    uint32_t seed;
};

// Tables and per-row constants of the epilogue.
struct EpilogueLds {
    int q_off[64];
    float c_f[64];          // residual counter of each code, before the rebase
    float dn[kTile];        // denominator of each row of the strip
    float k[kTile];         // Cf / scale_new
    float ratio[kTile];     // scale_old / scale_new
    uint8_t fin[kLutFinMaxBytes];
    int ok;
};

// c_reb[code] of the update kernel, evaluated on the fly: (float)c * ratio.
struct RebasedCounter {
    const float* c_f;
    float ratio;
    __device__ __forceinline__ float operator[](uint32_t code) const { return c_f[code] * ratio; }
};

__device__ __forceinline__ int load_relaxed(const int* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Data that crosses workgroups (the chain blocks) moves with device-scope atomic accesses, which
// are coherent between the per-XCD L2 caches by themselves, instead of ordinary accesses bracketed
// by device-scope fences: a fence writes back or invalidates the whole L2 and costs tens of
// microseconds when a thousand workgroups do it, and a strip has up to 43 hand-offs in sequence.
// Ordering comes from completion: the producer waits until its stores have been acknowledged
// (stores_done) before it raises the flag, and the consumer issues its loads only after it has
// seen the flag.
__device__ __forceinline__ float load_shared_f32(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void store_shared_f32(float* p, float x) {
    __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void stores_done() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt = expcnt = lgkmcnt = 0
}

// Value of lane (4 * (lane / 4) + K) of the calling lane's quad.
template <int K>
__device__ __forceinline__ float quad_lane(float x) {
    constexpr int ctrl = K | (K << 2) | (K << 4) | (K << 6);  // quad_perm:[K,K,K,K]
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), ctrl, 0xf, 0xf, false));
}

// OR over the four lanes of each quad.
__device__ __forceinline__ uint32_t quad_or(uint32_t x) {
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xb1, 0xf, 0xf, false);  // quad_perm:[1,0,3,2]
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4e, 0xf, 0xf, false);  // quad_perm:[2,3,0,1]
    return x;
}

// Parks the tile in the accumulation registers (AGPRs): between the phases of the epilogue the 64
// accumulators are only kept, not used, and the vector registers are needed for the phase's own
// working set.  Without this the compiler keeps them in vector registers and spills to scratch.
template <int TM, int TN>
__device__ __forceinline__ void park_accumulators(floatx16 (&acc)[TM][TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float t = acc[i][j][r];
                asm volatile("" : "+a"(t));
                acc[i][j][r] = t;
            }
}

// The thread's tile coordinates recomputed from an index the compiler cannot see through: each
// phase of the epilogue derives its addresses afresh instead of keeping hundreds of them, hoisted
// out of the persistent tile loop, alive across the contraction.
__device__ __forceinline__ TilePos fresh_tile_pos() {
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    TilePos p;
    p.tid = tid;
    const int lane = tid & 63, wave = tid >> 6;
    p.l32 = lane & 31;
    p.half = lane >> 5;
    p.wm0 = (wave >> 1) * (kTile / 2);
    p.wn0 = (wave & 1) * (kTile / 2);
    return p;
}

__device__ __forceinline__ bool cas_relaxed(int* p, int expected, int desired) {
    return __hip_atomic_compare_exchange_strong(p, &expected, desired, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
}

// A workgroup that cannot go on: the strip is marked aborted unless it has been committed already,
// the launch-local status ends every other wait, and the library's failure count remembers it.
// Returns the strip's final decision (+1 if the commit came first).
__device__ __forceinline__ int give_up(const StripArgs& a, StripControl* c) {
    cas_relaxed(&c->decision, 0, -1);
    const int d = load_relaxed(&c->decision);
    if (d < 0) {
        if (__hip_atomic_exchange(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
            __hip_atomic_fetch_add(a.failures, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return d;
}

// Thread 0 polls until *word >= want (a hand-off counter) or, with DECISION, until *word != 0,
// the status word is raised, or the spin budget is spent; ok_word (in LDS) tells the workgroup
// whether the condition came true.  All threads of the workgroup call it.
template <bool DECISION>
__device__ __forceinline__ bool wait_for(const StripArgs& a, const int* word, int want, int& ok_word,
                                         int decision_naps = 0) {
    if (threadIdx.x == 0) {
        int ok = 1;
        unsigned spins = 0, polls = 0;
        for (;;) {
            const int seen = load_relaxed(word);
            if (DECISION ? seen != 0 : seen >= want) break;
            // A hand-off counter counts hand-offs, each of which takes a few microseconds: sleep in
            // proportion to the hand-offs still to come instead of polling at full rate.  A
            // thousand workgroups polling a handful of words slow the contractions that are
            // still running by a third.
            const int naps = DECISION ? decision_naps : (want - seen - 1) * kNapsPerHandOff;
            __builtin_amdgcn_s_sleep(8);
            for (int n = 0; n < naps; ++n) __builtin_amdgcn_s_sleep(32);
            spins += 1u + (unsigned)naps;
            if (((++polls & 15u) == 0 && load_relaxed(a.status) != 0) || spins >= a.spin_limit) {
                ok = 0;
                break;
            }
        }
        ok_word = ok;
    }
    __syncthreads();
    const bool ok = ok_word != 0;
    __syncthreads();  // the word may be rewritten by the next wait
    return ok;
}

// One chain step of the hand-off for one of the two sums: every lane adds the four values of its
// packed group to the chain slot of (row, group) in element order.  `value(i, j, r)` is this
// lane's value for accumulator element (i, j, r).
template <typename Value>
__device__ __forceinline__ void chain_step(float* lds, const TilePos& tp, int kq, Value value) {
    using Cfg = TileCfg<kTile, kTile>;
#pragma unroll
    for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = tp.wm0 + 32 * i + 8 * (r / 4) + 4 * tp.half + (r % 4);
#pragma unroll
            for (int j = 0; j < Cfg::kTilesN; ++j) {
                const int gi = (tp.wn0 + 32 * j + tp.l32) >> 2;
                float* slot = lds + row * kGroupsPerTile + gi;  // owned by this lane's quad
                float c = *slot;
                const float val = value(i, j, r);
                c = c + quad_lane<0>(val);  // element order inside the group
                c = c + quad_lane<1>(val);
                c = c + quad_lane<2>(val);
                c = c + quad_lane<3>(val);
                if (kq == 0) *slot = c;
            }
        }
}

// DIRECT: tokens % 16 == 0 and grad_out 16-byte aligned, so the slabs can go straight to LDS.
// WITH_GS: lr_scale != 0, the row sums of g * t travel beside the sums of squares.
template <bool VEC_A, bool DIRECT, bool WITH_GS>
__global__ __launch_bounds__(kGemmThreads, 4) void fused_strip_kernel(StripArgs a) {
    using Cfg = TileCfg<kTile, kTile>;
    __shared__ float lds[DIRECT ? DirectCfg<kTile, kTile>::kLdsFloats : Cfg::kLdsFloats];
    __shared__ EpilogueLds e;
    const TilePos tp0 = tile_pos<kTile, kTile>();
    for (int i = tp0.tid; i < 64; i += kGemmThreads) {
        e.q_off[i] = q_off_entry((uint32_t)i, a.cd, a.geom);
        e.c_f[i] = (float)code_c((uint32_t)i, a.cd);
    }
    for (int i = tp0.tid, n = fin_size(a.geom); i < n; i += kGemmThreads) fill_fin_entry(i, a.cd, a.geom, e.fin);
    __syncthreads();

    const int groups_per_row = a.in_features >> 2;
    const uint32_t last_group_off = 3u * ((uint32_t)a.out_features * (uint32_t)groups_per_row - 1u);
    const uint32_t row_bytes = 3u * (uint32_t)groups_per_row;

    for (int tile = blockIdx.x; tile < a.total_tiles; tile += gridDim.x) {
        // once a workgroup has given up nothing new is started: a strip whose tiles have not all
        // published cannot have been committed, and this tile has not published yet
        if (threadIdx.x == 0) e.ok = load_relaxed(a.status) == 0 ? 1 : 0;
        __syncthreads();
        const bool healthy = e.ok != 0;
        __syncthreads();
        if (!healthy) return;
        const int strip = tile / a.tiles_per_strip;
        const int ct = tile - strip * a.tiles_per_strip;
        const int m0 = strip * kTile, n0 = ct * kTile;
        const int parity = ct & 1, step = ct >> 1;
        StripControl* control = a.control + strip;
        float* chain = a.chain + (size_t)strip * kStripChainFloats;

        floatx16 acc[Cfg::kTilesM][Cfg::kTilesN];
        // even progress of the workgroups that share a CU: a strip is as slow as its slowest tile
        if (DIRECT)
            gemm_tile_mainloop_direct<kTile, kTile, true>(a.grad_out, a.x, a.tokens, a.out_features, a.in_features,
                                                          m0, n0, tp0, lds, acc, a.out_features,
                                                          (int)blockIdx.x / a.layer_wgs);
        else
            gemm_tile_mainloop<kTile, kTile, VEC_A, true, true>(a.grad_out, a.x, a.tokens, a.out_features,
                                                                a.in_features, m0, n0, tp0, lds, acc,
                                                                a.out_features, (int)blockIdx.x / a.layer_wgs);

        park_accumulators(acc);
        // the hand-off sequence is latency-bound and other workgroups of this CU are still in
        // their contraction: let the epilogue's few instructions issue first
        __builtin_amdgcn_s_setprio(3);
        TilePos tp = fresh_tile_pos();
        int lane = tp.tid & 63, wave = tp.tid >> 6;
        int kq = tp.l32 & 3;  // position of this lane's column inside its packed group

        // Old per-row values, read before anything of this strip is written: tile 0 overwrites
        // them only after the strip has been committed, and commits happen after every tile of
        // the strip has been here.
        float s_old = 0.0f, v_old = 0.0f;
        if (tp.tid < kTile) {
            s_old = a.scale[m0 + tp.tid];
            v_old = a.v[m0 + tp.tid];
        }
        // byte offsets of this thread's accumulator elements from the state base (the launch checks
        // that the state is smaller than 2 GiB) and their element indices
        const uint32_t my_state = (uint32_t)(m0 + tp.wm0 + 4 * tp.half) * row_bytes +
                                  3u * ((uint32_t)(n0 + tp.wn0 + tp.l32) >> 2);
        // One 4-byte load per lane and element; the tensor's last group has no byte after it, so it
        // is fetched one byte early and shifted down.
        auto load_word = [&](int i, int j, int r) {
            const uint32_t off = my_state + (uint32_t)(32 * i + 8 * (r / 4) + (r % 4)) * row_bytes + 24u * j;
            const uint32_t is_last = off == last_group_off ? 1u : 0u;
            uint32_t word;
            __builtin_memcpy(&word, a.state + (off - is_last), 4);
            return word >> (8 * is_last);
        };

        // ---- chain hand-off: step `step` of chains 32*parity .. 32*parity+31 -------------
        // The 128 x 32 chain block (16 KiB per sum) is staged in the contraction's LDS slab buffer,
        // which is free by now; each thread moves 16 floats, 256 contiguous bytes per wave and access.
        if (!wait_for<false>(a, &control->published[parity], step, e.ok)) {
            if (threadIdx.x == 0) give_up(a, control);
            return;
        }
        park_accumulators(acc);
        static_assert(Cfg::kLdsFloats >= kTile * kGroupsPerTile, "chain block must fit the slab buffer");
        constexpr int kChainPerThread = kTile * kGroupsPerTile / kGemmThreads;
#pragma unroll
        for (int set = 0; set < (WITH_GS ? 2 : 1); ++set) {
            float* my_chain = chain + set * kChainSetFloats + parity * (kTile * kGroupsPerTile);
            {
                float in[kChainPerThread];
#pragma unroll
                for (int p = 0; p < kChainPerThread; ++p)
                    in[p] = step > 0 ? load_shared_f32(my_chain + tp.tid + kGemmThreads * p) : 0.0f;
#pragma unroll
                for (int p = 0; p < kChainPerThread; ++p) lds[tp.tid + kGemmThreads * p] = in[p];
            }
            __syncthreads();
            if (set == 0) {
                chain_step(lds, tp, kq, [&](int i, int j, int r) { return acc[i][j][r] * acc[i][j][r]; });
            } else {
                // g * t (kernels/compact_counter.cl:81-82): t from this element's code
                chain_step(lds, tp, kq, [&](int i, int j, int r) {
                    const uint32_t code = (load_word(i, j, r) >> (6 * kq)) & 0x3fu;
                    return acc[i][j][r] * (float)(code_q(code, a.cd) - 1);
                });
            }
            __syncthreads();
#pragma unroll
            for (int p = 0; p < kChainPerThread; ++p)
                store_shared_f32(my_chain + tp.tid + kGemmThreads * p, lds[tp.tid + kGemmThreads * p]);
            stores_done();
            __syncthreads();
        }
        const int n_even = (a.tiles_per_strip + 1) >> 1, n_odd = a.tiles_per_strip >> 1;
        if (tp.tid == 0) {
            __hip_atomic_store(&control->published[parity], step + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // the tile that ends its sequence counts it; the one that ends the second commits the strip
            if (step + 1 == (parity ? n_odd : n_even)) {
                __builtin_amdgcn_s_waitcnt(0);
                const int done = __hip_atomic_fetch_add(&control->sequences_done, 1, __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT) + 1;
                if (done == (n_odd > 0 ? 2 : 1)) cas_relaxed(&control->decision, 0, 1);
            }
        }

        // ---- wait for the strip's decision ---------------------------------------------
        park_accumulators(acc);
        tp = fresh_tile_pos();
        lane = tp.tid & 63, wave = tp.tid >> 6;
        bool committed = wait_for<true>(a, &control->decision, 0, e.ok);
        if (tp.tid == 0) {
            int d = committed ? load_relaxed(&control->decision) : give_up(a, control);
            if (d < 0 && committed) give_up(a, control);  // aborted by another tile: count this launch as failed
            e.ok = d > 0 ? 1 : 0;
        }
        __syncthreads();
        committed = e.ok != 0;
        __syncthreads();
        if (!committed) return;

        // ---- row statistics: every tile finishes the rows of its strip itself ---------------
        {
            // wave w finishes rows 32 w .. 32 w + 31: lane l holds chain l of the row
            constexpr int kRowsPerWave = kTile / 4;
            const bool have = lane < 32 || n_odd > 0;
#pragma unroll
            for (int set = 0; set < (WITH_GS ? 2 : 1); ++set) {
                const float* mine = chain + set * kChainSetFloats + (lane >> 5) * (kTile * kGroupsPerTile) + (lane & 31);
                float part[kRowsPerWave];
#pragma unroll
                for (int rr = 0; rr < kRowsPerWave; ++rr)
                    part[rr] = have ? load_shared_f32(mine + (wave * kRowsPerWave + rr) * kGroupsPerTile) : 0.0f;
#pragma unroll
                for (int rr = 0; rr < kRowsPerWave; ++rr) {
                    const float sum = tree_sum(part[rr], lane);
                    if (lane == 0) (set == 0 ? e.dn : e.k)[wave * kRowsPerWave + rr] = sum;  // parked; replaced below
                }
            }
        }
        __syncthreads();
        if (tp.tid < kTile) {
            const RowStats rs = finish_row_stats(e.dn[tp.tid], WITH_GS ? e.k[tp.tid] : 0.0f, v_old, s_old, a.in_features,
                                                 WITH_GS ? a.lr_scale : 0.0f, a.rms_beta, a.rms_eps);
            e.dn[tp.tid] = rs.denom;
            e.k[tp.tid] = a.cd.Cf / rs.scale_new;
            e.ratio[tp.tid] = s_old / rs.scale_new;
            if (ct == 0) {
                a.v[m0 + tp.tid] = rs.v_new;
                a.scale[m0 + tp.tid] = rs.scale_new;
            }
        }
        __syncthreads();

        park_accumulators(acc);
        tp = fresh_tile_pos();
        kq = tp.l32 & 3;
        // ---- ticks straight from the accumulators -----------------------------------------
        TickConsts tc;
        tc.rd = 0.0;
        tc.neg_lr = -a.lr;
        tc.neg_lim_neg = -(float)a.geom.lim_neg;
        tc.lim_pos = (float)a.geom.lim_pos;
        tc.two_m24 = 1.0f / 16777216.0f;
        tc.seed_mix = seed_mix(a.seed);
        const uint32_t my_state2 = (uint32_t)(m0 + tp.wm0 + 4 * tp.half) * row_bytes +
                                   3u * ((uint32_t)(n0 + tp.wn0 + tp.l32) >> 2);
        const uint32_t my_elem = (uint32_t)(m0 + tp.wm0 + 4 * tp.half) * (uint32_t)a.in_features +
                                 (uint32_t)(n0 + tp.wn0 + tp.l32);
        const int my_row = tp.wm0 + 4 * tp.half;
#pragma unroll
        for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
            for (int j = 0; j < Cfg::kTilesN; ++j) {
                // all 16 state loads are issued before the first tick
                uint32_t word[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t off = my_state2 + (uint32_t)(32 * i + 8 * (r / 4) + (r % 4)) * row_bytes + 24u * j;
                    const uint32_t is_last = off == last_group_off ? 1u : 0u;
                    __builtin_memcpy(&word[r], a.state + (off - is_last), 4);
                    word[r] >>= 8 * is_last;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = my_row + 32 * i + 8 * (r / 4) + (r % 4);
                    tc.dn = e.dn[row];
                    tc.k = e.k[row];
                    const RebasedCounter c_reb{e.c_f, e.ratio[row]};
                    const uint32_t dr = (uint32_t)(32 * i + 8 * (r / 4) + (r % 4));
                    const uint32_t elem = my_elem + dr * (uint32_t)a.in_features + 32u * j;
                    const uint32_t off = my_state2 + dr * row_bytes + 24u * j;
                    const uint32_t code = (word[r] >> (6 * kq)) & 0x3fu;
                    const uint32_t nc = tick_code<false>(code, acc[i][j][r], tc, hash_first(elem), c_reb, e.q_off,
                                                         e.fin);
                    const uint32_t nw = quad_or(nc << (6 * kq));
                    if (kq < 3) a.state[off + kq] = (uint8_t)(nw >> (8 * kq));
                }
            }
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();  // the row constants are rewritten by the next tile
    }
}

// ------------------------------------------------------------------------------ wide tiles
// The same step on the 256 x 256 tiles of gemm_wide_tile.hpp, one workgroup per CU.  A strip is 256
// rows and a tile covers 64 consecutive packed groups of its rows -- one step of all 64 chains --
// so the tiles of a strip form a single hand-off sequence: tile ct waits for tile ct - 1.  In the
// permuted accumulator layout a lane holds two neighbouring columns of each of its 64 rows, so a
// packed group is a pair of lanes: the even lane adds elements 0 and 1 to the chain value, hands
// the sum to the odd lane (DPP), which adds elements 2 and 3 and stores it; the four adds are the
// reference's, in its order.  Chain values go straight between registers and the chain block
// (device-scope atomic accesses, 64 contiguous bytes per 16 lanes).  A wide strip uses the chain
// storage and the first control block of the two 128-row strips it covers, so the workspace is
// the same for both kernels.
constexpr int kWideChainSetFloats = kWide * 64;  // 256 rows x 64 chains
static_assert(2 * kWideChainSetFloats == 2 * kStripChainFloats, "a wide strip takes the room of two 128-row strips");

struct WideEpilogueLds {
    int q_off[64];
    float c_f[64];
    float dn[kWide];     // denominator of each row of the strip
    float k[kWide];      // Cf / scale_new
    float ratio[kWide];  // scale_old / scale_new
    uint8_t fin[kLutFinMaxBytes];
    int ok;
};

// Value of the even lane of the calling lane's pair (lanes 2 n and 2 n + 1).
__device__ __forceinline__ float from_even_lane(float x) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), 0xa0, 0xf, 0xf, false));  // quad_perm:[0,0,2,2]
}
// OR over the two lanes of each pair.
__device__ __forceinline__ uint32_t pair_or(uint32_t x) {
    return x | (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xb1, 0xf, 0xf, false);  // quad_perm:[1,0,3,2]
}

// A parked tile: its 65536 accumulators in the order (register, thread), then the old scale and v of
// the strip's 256 rows.  Only the workgroup that wrote a slot reads it, every thread its own values.
constexpr int kParkSlotFloats = kWide * kWide + 2 * kWide;

// The thread's coordinates recomputed from an index the compiler cannot see through: what the
// epilogue derives from them (row offsets, state addresses) is then computed where it is used
// instead of being hoisted over the tile loop and kept alive -- spilled -- across the contraction.
struct WideEpiloguePos {
    WideLane t;
    int pair_half;  // 0: elements 0, 1 of the packed group; 1: elements 2, 3
    int slot;       // the group's place in the tile = its chain
    int row0;       // accumulator (i, j, r) is row row0 + 32 (r / 4) + 4 (r % 4) + i,
                    // column 4 slot + 2 pair_half + j of the tile
};
__device__ __forceinline__ WideEpiloguePos fresh_wide_pos() {
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    WideEpiloguePos p;
    p.t.tid = tid;
    p.t.lane = tid & 63;
    p.t.wave = tid >> 6;
    p.t.l32 = p.t.lane & 31;
    p.t.half = p.t.lane >> 5;
    p.t.wm0 = (p.t.wave >> 2) * 128;
    p.t.wn0 = (p.t.wave & 3) * 64;
    p.pair_half = p.t.l32 & 1;
    p.slot = (p.t.wn0 >> 2) + (p.t.l32 >> 1);
    p.row0 = p.t.wm0 + 16 * p.t.half;
    return p;
}

template <bool WITH_GS>
MCC_WIDE_KERNEL void fused_strip_wide_kernel(StripArgs a) {
    __shared__ __attribute__((aligned(1024))) float lds[kWideBuffers * kWideSlabFloats];
    __shared__ WideEpilogueLds e;
    const WideLane t = wide_lane();
    for (int i = t.tid; i < 64; i += kWideThreads) {
        e.q_off[i] = q_off_entry((uint32_t)i, a.cd, a.geom);
        e.c_f[i] = (float)code_c((uint32_t)i, a.cd);
    }
    for (int i = t.tid, n = fin_size(a.geom); i < n; i += kWideThreads) fill_fin_entry(i, a.cd, a.geom, e.fin);
    __syncthreads();

    const int groups_per_row = a.in_features >> 2;
    const uint32_t last_group_off = 3u * ((uint32_t)a.out_features * (uint32_t)groups_per_row - 1u);
    const uint32_t row_bytes = 3u * (uint32_t)groups_per_row;
    // the epilogue's view of the thread, taken afresh at the start of each of its phases
    WideLane te = t;
    int pair_half = 0, slot = 0, row0 = 0;
    auto refresh = [&]() __attribute__((always_inline)) {
        const WideEpiloguePos p = fresh_wide_pos();
        te = p.t;
        pair_half = p.pair_half;
        slot = p.slot;
        row0 = p.row0;
    };
    auto row_of = [&](int i, int r) { return row0 + 32 * (r / 4) + 4 * (r % 4) + i; };

    // One 4-byte load per lane and group; the tensor's last group has no byte after it, so it
    // is fetched one byte early and shifted down.  my_state: byte offset of this lane's packed
    // group in row row0 of the strip (the launch checks that the state is smaller than 2 GiB).
    auto load_word = [&](uint32_t my_state, int i, int r) {
        const uint32_t off = my_state + (uint32_t)(32 * (r / 4) + 4 * (r % 4) + i) * row_bytes;
        const uint32_t is_last = off == last_group_off ? 1u : 0u;
        uint32_t word;
        __builtin_memcpy(&word, a.state + (off - is_last), 4);
        return word >> (8 * is_last);
    };

    // Everything after a tile's hand-off: wait for the strip's decision, finish the rows of the
    // strip, apply the ticks to the tile's columns.  False: the strip was not committed (the launch
    // has failed) and nothing of it was written by this tile.
    auto finish = [&](WideAcc& acc, int strip, int ct, float s_old, float v_old, int decision_naps)
                      __attribute__((always_inline)) -> bool {
        refresh();
        const int m0 = strip * kWide, n0 = ct * kWide;
        StripControl* control = a.control + 2 * strip;
        const float* chain = a.chain + (size_t)strip * (2 * kWideChainSetFloats);
        bool committed = wait_for<true>(a, &control->decision, 0, e.ok, decision_naps);
        if (te.tid == 0) {
            int d = committed ? load_relaxed(&control->decision) : give_up(a, control);
            if (d < 0 && committed) give_up(a, control);  // aborted by another tile: count this launch as failed
            e.ok = d > 0 ? 1 : 0;
        }
        __syncthreads();
        committed = e.ok != 0;
        __syncthreads();
        if (!committed) return false;

        // ---- row statistics: every tile finishes the rows of its strip itself ---------------
        {
            // wave w finishes rows 32 w .. 32 w + 31: lane l holds chain l of the row
            constexpr int kRowsPerWave = kWide / 8;
#pragma unroll
            for (int set = 0; set < (WITH_GS ? 2 : 1); ++set) {
                const float* mine = chain + set * kWideChainSetFloats + te.lane;
                float part[kRowsPerWave];
#pragma unroll
                for (int rr = 0; rr < kRowsPerWave; ++rr)
                    part[rr] = load_shared_f32(mine + (te.wave * kRowsPerWave + rr) * 64);
#pragma unroll
                for (int rr = 0; rr < kRowsPerWave; ++rr) {
                    const float sum = tree_sum(part[rr], te.lane);
                    if (te.lane == 0) (set == 0 ? e.dn : e.k)[te.wave * kRowsPerWave + rr] = sum;  // parked; replaced below
                }
            }
        }
        __syncthreads();
        if (te.tid < kWide) {
            const RowStats rs = finish_row_stats(e.dn[te.tid], WITH_GS ? e.k[te.tid] : 0.0f, v_old, s_old, a.in_features,
                                                 WITH_GS ? a.lr_scale : 0.0f, a.rms_beta, a.rms_eps);
            e.dn[te.tid] = rs.denom;
            e.k[te.tid] = a.cd.Cf / rs.scale_new;
            e.ratio[te.tid] = s_old / rs.scale_new;
            if (ct == 0) {
                a.v[m0 + te.tid] = rs.v_new;
                a.scale[m0 + te.tid] = rs.scale_new;
            }
        }
        __syncthreads();

        // ---- ticks straight from the accumulators -----------------------------------------
        TickConsts tc;
        tc.rd = 0.0;
        tc.neg_lr = -a.lr;
        tc.neg_lim_neg = -(float)a.geom.lim_neg;
        tc.lim_pos = (float)a.geom.lim_pos;
        tc.two_m24 = 1.0f / 16777216.0f;
        tc.seed_mix = seed_mix(a.seed);
        const uint32_t my_state = (uint32_t)(m0 + row0) * row_bytes + 3u * (uint32_t)((n0 >> 2) + slot);
        const uint32_t my_elem = (uint32_t)(m0 + row0) * (uint32_t)a.in_features +
                                 (uint32_t)(n0 + 4 * slot + 2 * pair_half);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // all 16 state loads are issued before the first tick
            uint32_t word[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) word[r] = load_word(my_state, i, r);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = row_of(i, r);
                tc.dn = e.dn[row];
                tc.k = e.k[row];
                const RebasedCounter c_reb{e.c_f, e.ratio[row]};
                const uint32_t dr = (uint32_t)(32 * (r / 4) + 4 * (r % 4) + i);
                const uint32_t elem = my_elem + dr * (uint32_t)a.in_features;
                const uint32_t off = my_state + dr * row_bytes;
                const uint32_t codes = word[r] >> (12 * pair_half);
                const uint32_t nc0 = tick_code<false>(codes & 0x3fu, acc[i][0][r], tc, hash_first(elem), c_reb, e.q_off,
                                                      e.fin);
                const uint32_t nc1 = tick_code<false>((codes >> 6) & 0x3fu, acc[i][1][r], tc, hash_first(elem + 1u),
                                                      c_reb, e.q_off, e.fin);
                const uint32_t nw = pair_or((nc0 | (nc1 << 6)) << (12 * pair_half));
                // bytes 0 and 1 of the group from the even lane, byte 2 from the odd one
                if (pair_half) {
                    a.state[off + 2] = (uint8_t)(nw >> 16);
                } else {
                    a.state[off] = (uint8_t)nw;
                    a.state[off + 1] = (uint8_t)(nw >> 8);
                }
            }
        }
        __syncthreads();  // the row constants are rewritten by the next tile
        return true;
    };

    // A tile whose strip ends in a later pass of the grid cannot be finished now without idling for
    // the length of a pass: after its hand-off its accumulators go to one of the workgroup's two
    // slots (two, because the next tile may have to be parked before this one can be finished)
    // and the workgroup takes its next tile.  A parked tile is finished after the next tile has
    // been dealt with -- by then the rest of its strip, which runs in that same pass, has published
    // -- or, when there is no next tile, at the end.
    float* my_slots = a.park ? a.park + (size_t)2 * ((int)blockIdx.x - a.park_first_wg) * kParkSlotFloats : nullptr;
    int parked_strip = -1, parked_ct = 0, parked_slot = 0, next_slot = 0;
    auto finish_parked = [&](int decision_naps) __attribute__((always_inline)) {
        refresh();
        float* p = my_slots + (size_t)parked_slot * kParkSlotFloats;
        WideAcc acc;
#pragma unroll
        for (int q = 0; q < 128; ++q) acc[q / 32][(q / 16) % 2][q % 16] = p[q * kWideThreads + te.tid];
        float s_old = 0.0f, v_old = 0.0f;
        if (te.tid < kWide) {
            s_old = p[kWide * kWide + te.tid];
            v_old = p[kWide * kWide + kWide + te.tid];
        }
        const bool ok = finish(acc, parked_strip, parked_ct, s_old, v_old, decision_naps);
        parked_strip = -1;
        return ok;
    };

    bool alive = true;
    for (int tile = blockIdx.x; alive && tile < a.total_tiles; tile += gridDim.x) {
        // once a workgroup has given up nothing new is started: a strip whose tiles have not all
        // published cannot have been committed, and this tile has not published yet
        if (te.tid == 0) e.ok = load_relaxed(a.status) == 0 ? 1 : 0;
        __syncthreads();
        const bool healthy = e.ok != 0;
        __syncthreads();
        if (!healthy) break;
        const int strip = tile / a.tiles_per_strip;
        const int ct = tile - strip * a.tiles_per_strip;
        const int m0 = strip * kWide, n0 = ct * kWide;
        StripControl* control = a.control + 2 * strip;
        float* chain = a.chain + (size_t)strip * (2 * kWideChainSetFloats);

        WideAcc acc;
        wide_zero(acc);
        wide_accumulate(a.grad_out + m0, a.x + n0, a.out_features, a.in_features, a.tokens, acc, lds, t);
        refresh();

        // Old per-row values, read before anything of this strip is written: tile 0 overwrites
        // them only after the strip has been committed, and commits happen after every tile of
        // the strip has been here.
        float s_old = 0.0f, v_old = 0.0f;
        if (te.tid < kWide) {
            s_old = a.scale[m0 + te.tid];
            v_old = a.v[m0 + te.tid];
        }
        const uint32_t my_state = (uint32_t)(m0 + row0) * row_bytes + 3u * (uint32_t)((n0 >> 2) + slot);

        // ---- chain hand-off: step ct of all 64 chains of the strip's rows -------------------
        if (!wait_for<false>(a, &control->published[0], ct, e.ok)) {
            if (te.tid == 0) give_up(a, control);
            break;
        }
#pragma unroll
        for (int set = 0; set < (WITH_GS ? 2 : 1); ++set) {
            float* my_chain = chain + set * kWideChainSetFloats + slot;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float in[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) in[r] = ct > 0 ? load_shared_f32(my_chain + row_of(i, r) * 64) : 0.0f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float v0, v1;
                    if (set == 0) {
                        v0 = acc[i][0][r] * acc[i][0][r];
                        v1 = acc[i][1][r] * acc[i][1][r];
                    } else {
                        // g * t (kernels/compact_counter.cl:81-82): t from the element's code
                        const uint32_t word = load_word(my_state, i, r) >> (12 * pair_half);
                        v0 = acc[i][0][r] * (float)(code_q(word & 0x3fu, a.cd) - 1);
                        v1 = acc[i][1][r] * (float)(code_q((word >> 6) & 0x3fu, a.cd) - 1);
                    }
                    const float first = (in[r] + v0) + v1;          // elements 0 and 1: the even lane's
                    const float second = (from_even_lane(first) + v0) + v1;  // then 2 and 3: the odd lane's
                    if (pair_half) store_shared_f32(my_chain + row_of(i, r) * 64, second);
                }
            }
        }
        stores_done();
        __syncthreads();
        if (te.tid == 0) {
            __hip_atomic_store(&control->published[0], ct + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // the last tile of the sequence commits the strip
            if (ct + 1 == a.tiles_per_strip) {
                __builtin_amdgcn_s_waitcnt(0);
                cas_relaxed(&control->decision, 0, 1);
            }
        }

        const int pass = tile / (int)gridDim.x;
        const int strip_last_pass = (strip * a.tiles_per_strip + a.tiles_per_strip - 1) / (int)gridDim.x;
        if (my_slots && strip_last_pass > pass && (int)blockIdx.x >= a.park_first_wg) {
            float* p = my_slots + (size_t)next_slot * kParkSlotFloats;
#pragma unroll
            for (int q = 0; q < 128; ++q) p[q * kWideThreads + te.tid] = acc[q / 32][(q / 16) % 2][q % 16];
            if (te.tid < kWide) {
                p[kWide * kWide + te.tid] = s_old;
                p[kWide * kWide + kWide + te.tid] = v_old;
            }
            // the tile parked before this one: its strip ended in this pass
            if (parked_strip >= 0) alive = finish_parked(0);
            parked_strip = strip;
            parked_ct = ct;
            parked_slot = next_slot;
            next_slot ^= 1;
            continue;
        }
        alive = finish(acc, strip, ct, s_old, v_old, 0);
        if (parked_strip >= 0) alive = finish_parked(0) && alive;
    }
    // the rest of a parked tile's strip may still be a whole tile's time away: poll slowly
    if (parked_strip >= 0) finish_parked(8);
}

__global__ void strip_clear_kernel(int* words, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) words[i] = 0;
}

constexpr size_t kHeaderBytes = 256;  // launch-local status word, padded

size_t control_bytes(size_t strips) { return (strips * sizeof(StripControl) + 255) / 256 * 256; }

// Workgroups of strip launches that gave up since the last mcc_compact_counter_fused_check, one
// counter per GPU.  It lives in the library, not in the caller's workspace: workspaces are shared
// between layers, and the next layer's step would wipe a status word kept there.
static __device__ int g_failures;

constexpr int kMaxDevices = 64;
struct DeviceState {
    int* failures = nullptr;          // device address of g_failures on this device
    hipEvent_t last_launch = nullptr; // recorded after the most recent strip launch
    hipStream_t last_stream = nullptr;
    bool launched = false;
};
std::mutex g_mu;
DeviceState g_devices[kMaxDevices];

// The calling thread's current device with its state resolved (nullptr + *err on failure).
DeviceState* current_device_state(hipError_t* err) {
    int device = -1;
    *err = hipGetDevice(&device);
    if (*err != hipSuccess) return nullptr;
    if (device < 0 || device >= kMaxDevices) {
        *err = hipErrorInvalidDevice;
        return nullptr;
    }
    DeviceState& d = g_devices[device];
    if (!d.failures) {
        void* p = nullptr;
        *err = hipGetSymbolAddress(&p, HIP_SYMBOL(g_failures));
        if (*err != hipSuccess) return nullptr;
        d.failures = static_cast<int*>(p);
    }
    return &d;
}

}  // namespace

// Polls (about 0.25 us each) a workgroup spends on one wait before it gives up: roughly four
// seconds, far above any wait a healthy launch can see.
constexpr unsigned kDefaultSpinLimit = 1u << 24;
// The test aids below belong to the calling thread: a thread that never sets them runs on the
// defaults whatever other threads do, and no setting can change under a running call.
static thread_local unsigned g_spin_limit = kDefaultSpinLimit;

// Which tiles a strip launch uses: 0 the wide ones where they keep the device busy, 1 the wide ones
// whenever the shape allows them, 2 never (tests compare the two kernels).
static thread_local int g_wide_mode = 0;
// Test aid: the wide kernel's grid is held to this many workgroups (0: what the device holds), so
// that small layers run in several passes and park tiles.
static thread_local int g_wide_grid_cap = 0;
void set_fused_strip_wide_mode(int mode, int grid_cap) {
    g_wide_mode = mode >= 0 && mode <= 2 ? mode : 0;
    g_wide_grid_cap = grid_cap > 0 ? grid_cap : 0;
}

unsigned fused_strip_spin_limit() { return g_spin_limit; }
void set_fused_strip_spin_limit(unsigned spins) { g_spin_limit = spins ? spins : kDefaultSpinLimit; }

bool fused_strip_supports(size_t in_features, size_t out_features, size_t batch) {
    return batch > 0 && in_features >= kTile && out_features >= kTile && in_features % kTile == 0 &&
           out_features % kTile == 0 && in_features <= (size_t(1) << 31) / out_features;  // 32-bit element offsets
}

// Workgroups of the wide kernel the current device holds at once (one per CU); 256 when no device
// can be asked (a size query on a machine without a GPU).
static long wide_device_capacity() {
    static std::atomic<long> cached[kMaxDevices];
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
        (void)hipGetLastError();
        return 256;
    }
    long c = cached[device].load();
    if (c > 0) return c;
    int cus = 0, per_cu = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0 ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fused_strip_wide_kernel<false>, kWideThreads, 0) != hipSuccess ||
        per_cu <= 0) {
        (void)hipGetLastError();
        return 256;
    }
    c = (long)cus * per_cu;
    cached[device].store(c);
    return c;
}

// Slots for parked tiles of the wide kernel: layers of more wide tiles than one pass of the
// persistent grid holds (`capacity` workgroups), so that strips can straddle passes, get two slots
// for each of the tiles_per_strip - 1 workgroups that may park (1 MiB per 4 slots).
static size_t park_bytes(size_t in_features, size_t out_features, size_t batch, long capacity) {
    if (in_features % kWide || out_features % kWide || batch < (size_t)kBK || batch % kBK) return 0;
    const size_t tiles_x = in_features / kWide, tiles = tiles_x * (out_features / kWide);
    if (tiles <= (size_t)capacity || tiles_x < 2) return 0;
    return 2 * (tiles_x - 1) * (size_t)kParkSlotFloats * sizeof(float);
}

static size_t strip_base_bytes(size_t out_features) {
    const size_t strips = out_features / kTile;
    return kHeaderBytes + control_bytes(strips) + strips * kStripChainFloats * sizeof(float);
}

size_t fused_strip_workspace_nbytes(size_t in_features, size_t out_features, size_t batch) {
    if (!fused_strip_supports(in_features, out_features, batch)) return 0;
    return strip_base_bytes(out_features) + park_bytes(in_features, out_features, batch, wide_device_capacity());
}

size_t fused_strip_workspace_nbytes_for_grid(size_t in_features, size_t out_features, size_t batch, int grid_cap) {
    if (!fused_strip_supports(in_features, out_features, batch)) return 0;
    const long device = wide_device_capacity();
    const long capacity = grid_cap > 0 && grid_cap < device ? grid_cap : device;
    return strip_base_bytes(out_features) + park_bytes(in_features, out_features, batch, capacity);
}

hipError_t fused_strip_take_failures(int* count) {
    std::lock_guard<std::mutex> lock(g_mu);
    hipError_t err;
    DeviceState* d = current_device_state(&err);
    if (!d) return err;
    err = hipMemcpy(count, d->failures, sizeof(int), hipMemcpyDeviceToHost);
    if (err != hipSuccess || *count == 0) return err;
    const int zero = 0;
    return hipMemcpy(d->failures, &zero, sizeof(int), hipMemcpyHostToDevice);
}

hipError_t launch_fused_strip(hipStream_t stream, uint8_t* state, float* scale, float* v, const float* grad_out,
                              const float* x, void* workspace, int C, int in_features, int out_features, int tokens,
                              float lr, float lr_scale, float rms_beta, float rms_eps, uint32_t seed,
                              unsigned spin_limit, size_t workspace_nbytes) {
    const int strips = out_features / kTile;
    StripArgs a;
    a.state = state;
    a.scale = scale;
    a.v = v;
    a.grad_out = grad_out;
    a.x = x;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    a.status = reinterpret_cast<int*>(ws);
    a.control = reinterpret_cast<StripControl*>(ws + kHeaderBytes);
    a.chain = reinterpret_cast<float*>(ws + kHeaderBytes + control_bytes((size_t)strips));
    a.park = nullptr;
    a.park_first_wg = 0;
    a.tokens = tokens;
    a.in_features = in_features;
    a.out_features = out_features;
    a.tiles_per_strip = in_features / kTile;
    a.total_tiles = strips * a.tiles_per_strip;
    a.spin_limit = spin_limit;
    a.cd = make_codec(C);
    a.geom = lut_geom(a.cd);
    a.lr = lr;
    a.lr_scale = lr_scale;
    a.rms_beta = rms_beta;
    a.rms_eps = rms_eps;
    a.seed = seed;

    const bool vec_a = (reinterpret_cast<uintptr_t>(grad_out) & 15u) == 0;  // out_features % 4 == 0 holds
    if ((reinterpret_cast<uintptr_t>(x) & 15u) != 0) return hipErrorInvalidValue;
    // measured: with the rotating priority the direct-to-LDS main loop is 2 % slower here (it is
    // 3 % faster in the plain contraction), so the staged loop stays
    const bool gs = lr_scale != 0.0f;
    typedef void (*StripKernel)(StripArgs);
    StripKernel kernel = vec_a ? (gs ? fused_strip_kernel<true, false, true> : fused_strip_kernel<true, false, false>)
                               : (gs ? fused_strip_kernel<false, false, true> : fused_strip_kernel<false, false, false>);
    int threads = kGemmThreads;

    std::lock_guard<std::mutex> lock(g_mu);
    hipError_t err;
    DeviceState* dev = current_device_state(&err);
    if (!dev) return err;
    a.failures = dev->failures;

    // Tiles of a strip wait for each other, so every workgroup of the launch has to be resident:
    // a second strip launch running beside this one on another stream could starve both.  A launch
    // on another stream than the last one is therefore ordered behind it on the device (the
    // stream waits for the event recorded after that launch; nothing is allocated, the host does
    // not wait).  A stream under capture is left alone: what its graph later runs beside is the
    // caller's to order.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) capture = hipStreamCaptureStatusNone;
    const bool capturing = capture != hipStreamCaptureStatusNone;
    if (!capturing && dev->launched && dev->last_stream != stream) {
        err = hipStreamWaitEvent(stream, dev->last_launch, 0);
        if (err != hipSuccess) return err;
    }

    // the whole grid must be resident at once: size it from what the device can hold
    int device = 0, cus = 0, per_cu = 0;
    err = hipGetDevice(&device);
    if (err != hipSuccess) return err;
    err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
    if (err != hipSuccess) return err;

    // Wide tiles: whole 256 x 256 tiles, whole slabs, aligned operands -- and, unless forced, a shape
    // whose tiles come in rounds that keep at least four fifths of the CUs busy.  With slots for
    // parked tiles in the workspace a round is any 256 tiles (4096 x 11008: 688 tiles, three
    // rounds for 2.69); without them a round is whole strips (4096 x 4096 is one round of 16 strips
    // of 16 tiles; 4096 x 11008 would be four rounds of five strips of 43 tiles).
    const int wide_mode = g_wide_mode;
    const int grid_cap = g_wide_grid_cap;  // read once: sizing and launch agree
    bool parking = false;
    if (wide_mode != 2 && vec_a && in_features % kWide == 0 && out_features % kWide == 0 && tokens >= kBK &&
        tokens % kBK == 0) {
        StripKernel wide = gs ? fused_strip_wide_kernel<true> : fused_strip_wide_kernel<false>;
        int wide_per_cu = 0;
        err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&wide_per_cu, wide, kWideThreads, 0);
        if (err != hipSuccess) return err;
        const long capacity = grid_cap && grid_cap < (long)cus * wide_per_cu ? grid_cap : (long)cus * wide_per_cu;
        const long tiles_x = in_features / kWide, wide_strips = out_features / kWide, tiles = tiles_x * wide_strips;
        if (capacity >= tiles_x) {
            const size_t park = park_bytes((size_t)in_features, (size_t)out_features, (size_t)tokens, capacity);
            parking = park != 0;
            // the caller sized the workspace without the test aid's grid: tiles cannot be parked
            if (parking && workspace_nbytes < strip_base_bytes((size_t)out_features) + park) return hipErrorInvalidValue;
            const long per_round = parking ? capacity : capacity / tiles_x * tiles_x;
            const long rounds = (tiles + per_round - 1) / per_round;
            if (wide_mode == 1 || tiles * 5 >= rounds * capacity * 4) {
                kernel = wide;
                threads = kWideThreads;
                a.tiles_per_strip = (int)tiles_x;
                a.total_tiles = (int)tiles;
            } else {
                parking = false;
            }
        }
    }

    err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0);
    if (err != hipSuccess) return err;
    long capacity = (long)cus * per_cu;
    if (threads == kWideThreads && grid_cap && grid_cap < capacity) capacity = grid_cap;
    a.layer_wgs = cus;
    if (capacity < a.tiles_per_strip) return hipErrorLaunchOutOfResources;
    // a whole number of strips per pass of the persistent grid: a strip that straddled two passes
    // would park its early tiles' workgroups for the length of a pass
    const long whole = parking ? capacity : capacity / a.tiles_per_strip * a.tiles_per_strip;
    const int grid = (int)(whole < a.total_tiles ? whole : a.total_tiles);
    if (parking) {
        // a tile is parked when its strip ends in a later pass: such tiles are the last ones of a
        // pass and fewer than a strip has, so they sit on the last tiles_per_strip - 1 workgroups
        a.park = reinterpret_cast<float*>(ws + strip_base_bytes((size_t)out_features));
        a.park_first_wg = grid - (a.tiles_per_strip - 1);
    }

    const int clear_words = (int)((kHeaderBytes + control_bytes((size_t)strips)) / sizeof(int));
    hipLaunchKernelGGL(strip_clear_kernel, dim3((clear_words + 255) / 256), dim3(256), 0, stream,
                       reinterpret_cast<int*>(ws), clear_words);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), 0, stream, a);
    err = hipGetLastError();
    if (err != hipSuccess || capturing) return err;
    if (!dev->last_launch) {
        err = hipEventCreateWithFlags(&dev->last_launch, hipEventDisableTiming);
        if (err != hipSuccess) return err;
    }
    err = hipEventRecord(dev->last_launch, stream);
    if (err != hipSuccess) return err;
    dev->last_stream = stream;
    dev->launched = true;
    return hipSuccess;
}

}  // namespace mcc
