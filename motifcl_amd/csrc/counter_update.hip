// Update-only step of the compact-counter layer on gfx950: row statistics,
// stochastic-rounding tick and scale commit in ONE kernel, one wave64 per
// output row, for one tensor or a batch of tensors per launch.
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
//
// Why one row per wave and no persistent grid: the workgroups of a launch are
// dispatched in row order, so at any moment the rows in flight are a compact,
// advancing window of the gradient and the state, and neighbouring rows --
// whose bytes share DRAM pages -- are fetched at about the same time.  A
// persistent grid striding over the rows loses that: its waves drift apart,
// the window spreads over hundreds of megabytes, and the same loads and stores
// run at 0.65 instead of 0.73 of the HBM peak (measured on the bare access
// pattern; two rows per wave 0.72, four 0.68, eight 0.64).  The batched entry
// point puts the tensor index on the grid's y axis.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <vector>

#include "counter_math.hpp"
#include "launch.hpp"
#include "wave_ops.hpp"

namespace mcc {
namespace {

constexpr int kWave = 64;
constexpr int kThreads = kWave;  // one wave per workgroup: the row index is a function of blockIdx alone

struct BatchArgs {
    UpdateTensor t[kMaxUpdateBatch];
    int n_tensors;
    int total_rows;  // persistent kernels: rows of all tensors; dispatched kernels: unused
    Codec cd;
    LutGeom geom;
    float lr_scale, rms_beta, rms_eps;
};
static_assert(sizeof(BatchArgs) <= 4096, "kernel arguments are limited to 4 KiB");

// Per-workgroup tables in LDS (see counter_math.hpp).  All three depend on C only: c_f[code] is
// the residual counter as a float, and the rebased counter of kernels/compact_counter.cl:124 is
// c_f[code] * (s_old / s_new) -- the product c_reb_entry forms.  The tables of every valid C
// (3 (2C - 1) <= 64, i.e. C <= 11) are built at compile time and sit in the code object; a
// workgroup copies the ones of its C into LDS (16 bytes per thread) instead of computing them.
struct alignas(16) Luts {
    int q_off[64];   // first, so that the decode reads need no base-address add
    float c_f[64];   // 256 bytes behind q_off: one ds_read2st64_b32 fetches both
    uint8_t fin[kLutFinMaxBytes];
};
static_assert(sizeof(Luts) % 16 == 0, "copied in 16-byte pieces");

constexpr int kMaxC = 11;

struct LutsByC {
    Luts c[kMaxC];
};

constexpr LutsByC make_all_luts() {
    LutsByC all{};
    for (int C = 1; C <= kMaxC; ++C) {
        Luts& l = all.c[C - 1];
        const Codec cd = make_codec(C);
        const LutGeom geom = lut_geom(cd);
        for (int i = 0; i < 64; ++i) {
            l.q_off[i] = q_off_entry((uint32_t)i, cd, geom);
            l.c_f[i] = (float)code_c((uint32_t)i, cd);
        }
        for (int i = 0, n = fin_size(geom); i < n; ++i) fill_fin_entry(i, cd, geom, l.fin);
    }
    return all;
}

__device__ const LutsByC kLutsByC = make_all_luts();

__device__ __forceinline__ void build_luts(Luts& l, const Codec& cd, const LutGeom& geom) {
    const int pieces = (2 * 64 * 4 + fin_size(geom) + 15) / 16;
    const uint4* src = reinterpret_cast<const uint4*>(&kLutsByC.c[cd.C - 1]);
    uint4* dst = reinterpret_cast<uint4*>(&l);
    for (int i = threadIdx.x; i < pieces; i += blockDim.x) dst[i] = src[i];
    __syncthreads();
}

// c_reb[code] of the tick for a row whose scale changed: (float)c * (s_old / s_new).
struct RebasedCounters {
    const float* c_f;
    float ratio;
    __device__ __forceinline__ float operator[](uint32_t code) const { return c_f[code] * ratio; }
};

// A gradient element is read exactly once by the register-resident kernels: a non-temporal load
// keeps it from displacing the state words (whose overlapping 4-byte loads do want the cache) and
// measured +1.8 % on 4096-wide rows.  State loads and stores gained nothing from the hint.
__device__ __forceinline__ float4 load_grad4_once(const float4* p) {
    typedef float f4v __attribute__((ext_vector_type(4)));
    const f4v v = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}

// Byte-granular access to one packed group (any alignment, any position).
__device__ __forceinline__ uint32_t load_group(const uint8_t* p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
}

__device__ __forceinline__ void store_group(uint8_t* p, uint32_t w) {
    // a 2-byte and a 1-byte store straight out of the word's register (global memory takes the
    // unaligned 2-byte store); no repacking
    const uint16_t lo = (uint16_t)w;
    __builtin_memcpy(p, &lo, 2);
    p[2] = (uint8_t)(w >> 16);
}

// One group's 24-bit word fetched with a single 4-byte load (global memory takes unaligned
// dword accesses); the byte above the word belongs to the next group and is never looked
// at.  The caller guarantees that byte exists, i.e. the group is not the tensor's last.
__device__ __forceinline__ uint32_t load_group_dword(const uint8_t* p) {
    uint32_t w;
    __builtin_memcpy(&w, p, 4);
    return w;
}

// The forms the register-resident kernels use: every state byte is read once and written once per
// step, and marking BOTH the load and the stores non-temporal lets the bare access pattern run at
// 0.79 instead of 0.74 of the HBM peak (the hint on the loads alone costs 12 %, on the stores
// alone nothing).
typedef uint32_t __attribute__((aligned(1))) unaligned_u32;
typedef uint16_t __attribute__((aligned(1))) unaligned_u16;

__device__ __forceinline__ uint32_t load_group_dword_once(const uint8_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const unaligned_u32*>(p));
}

__device__ __forceinline__ void store_group_once(uint8_t* p, uint32_t w) {
    __builtin_nontemporal_store((uint16_t)w, reinterpret_cast<unaligned_u16*>(p));
    __builtin_nontemporal_store((uint8_t)(w >> 16), p + 2);
}

// The same for a group that may be the tensor's last (`tail`): that one has no byte after it, so
// it is fetched one byte early and shifted down.  The tensor holds at least two groups (the
// launch sends smaller ones to the byte-granular kernel), so the byte before exists.
__device__ __forceinline__ uint32_t load_group_dword_or_tail(const uint8_t* p, bool tail) {
    const uint32_t back = tail ? 1u : 0u;
    return load_group_dword(p - back) >> (8u * back);
}

__device__ __forceinline__ uint32_t load_group_dword_or_tail_once(const uint8_t* p, bool tail) {
    const uint32_t back = tail ? 1u : 0u;
    return load_group_dword_once(p - back) >> (8u * back);
}

// Row statistics of one group (kernels/compact_counter.cl:78-83) plus what decides whether the
// row may use the reciprocal-based division: the smallest |g| of the row (zeros included, one
// v_min3_f32 per two elements) in the register-resident kernels, the exact magnitude key (zero
// mapped above everything) in the streamed ones.
struct RowAcc {
    float g_sq = 0.0f, grad_s = 0.0f;
    float min_abs = __builtin_inff();
    uint32_t min_key = 0xffffffffu;
};

__device__ __forceinline__ uint32_t umin3(uint32_t a, uint32_t b, uint32_t c) {
    const uint32_t ab = b < a ? b : a;
    return c < ab ? c : ab;  // one v_min3_u32
}

__device__ __forceinline__ float fmin3_abs(float a, float b, float c) {
    return __builtin_fminf(__builtin_fminf(a, __builtin_fabsf(b)), __builtin_fabsf(c));  // one v_min3_f32 with |.| modifiers
}

// Smallest magnitude key of one group (zero counts as large).
__device__ __forceinline__ uint32_t group_min_key(uint32_t key, const float g[4]) {
    key = umin3(key, range_key(g[0]), range_key(g[1]));
    return umin3(key, range_key(g[2]), range_key(g[3]));
}

// `g` holds zeros for a group past the end of the row (they add +0.0 to the squares and -+0.0 to
// the products with t, which leaves both sums unchanged); `live` keeps such a group out of the
// minimum as well.
template <bool WITH_GS, bool EXACT_KEY>
__device__ __forceinline__ void accumulate(RowAcc& acc, const float g[4], bool live, uint32_t w, const Codec& cd) {
    if (EXACT_KEY) {
        acc.min_key = group_min_key(acc.min_key, g);
    } else {
        const float m = fmin3_abs(fmin3_abs(acc.min_abs, g[0], g[1]), g[2], g[3]);
        acc.min_abs = live ? m : acc.min_abs;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float sq = g[k] * g[k];
        acc.g_sq = acc.g_sq + sq;
        if (WITH_GS) {
            const int t = code_q(code_of(w, k), cd) - 1;
            const float gt = g[k] * (float)t;
            acc.grad_s = acc.grad_s + gt;
        }
    }
}

__device__ __forceinline__ uint32_t umin(uint32_t a, uint32_t b) { return b < a ? b : a; }

// Minimum over the wave, taken at lane 0 (same pairing as tree_sum; any order would do).
__device__ __forceinline__ uint32_t wave_min(uint32_t a, int lane) {
    a = umin(a, (uint32_t)__builtin_amdgcn_ds_bpermute((lane + 32) << 2, (int)a));
    a = umin(a, (uint32_t)__builtin_amdgcn_ds_bpermute((lane + 16) << 2, (int)a));
    a = umin(a, row_from_above<8>(a));
    a = umin(a, row_from_above<4>(a));
    a = umin(a, row_from_above<2>(a));
    a = umin(a, row_from_above<1>(a));
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)a);
}

// Non-negative floats order like their bit patterns.
__device__ __forceinline__ float wave_min_nonneg(float a, int lane) { return __uint_as_float(wave_min(__float_as_uint(a), lane)); }

struct RowCtx {
    TickConsts tc;
    float s_old, s_new;  // the rebase factor of the residual counters is s_old / s_new
    bool fast_div;       // wave-uniform
};

// The rebase factor s_old / s_new; a division, so only where a row needs it (lr_scale != 0, or a
// scale that sat outside its clamp range).
__device__ __forceinline__ float rebase_ratio(const RowCtx& rc) { return rc.s_old / rc.s_new; }
// Whether the scale stays as it is (then the factor is exactly 1); wave-uniform.
__device__ __forceinline__ bool scale_unchanged(const RowCtx& rc) {
    return __builtin_amdgcn_readfirstlane(rc.s_old == rc.s_new ? 1 : 0) != 0;
}

// Tree reduction, row epilogue and commit of v/scale.  `exact_key()` returns the lane's exact
// magnitude key over the row; it is called (by the whole wave) only when the smallest magnitude
// cannot decide, i.e. when the row holds an exact zero.
template <bool WITH_GS, bool EXACT_KEY, typename KeyFn>
__device__ __forceinline__ RowCtx finish_row(const BatchArgs& a, const UpdateTensor& t, int row, int lane,
                                             const RowAcc& acc, KeyFn exact_key) {
    const float g_sq = tree_sum(acc.g_sq, lane);
    const float grad_s = WITH_GS ? tree_sum(acc.grad_s, lane) : 0.0f;
    const float s_old = t.scale[row];
    const float v_old = t.v[row];
    const RowStats rs = finish_row_stats(g_sq, grad_s, v_old, s_old, t.in_features, a.lr_scale,
                                         a.rms_beta, a.rms_eps);
    int fast;
    if (EXACT_KEY) {
        fast = row_takes_fast_division(rs.denom, g_sq, wave_min(acc.min_key, lane)) ? 1 : -1;
    } else {
        fast = fast_division_from_min_abs(rs.denom, g_sq, wave_min_nonneg(acc.min_abs, lane));
        fast = __builtin_amdgcn_readfirstlane(fast);
        if (fast == 0) fast = row_takes_fast_division(rs.denom, g_sq, wave_min(exact_key(), lane)) ? 1 : -1;
    }
    if (lane == 0) {
        t.v[row] = rs.v_new;
        t.scale[row] = rs.scale_new;  // commit (kernels/basic.cl:6-9); s_old stays in a register
    }
    RowCtx rc;
    rc.s_old = s_old;
    rc.s_new = rs.scale_new;
    rc.tc.dn = rs.denom;
    rc.tc.rd = row_reciprocal(rs.denom);
    rc.tc.k = a.cd.Cf / rs.scale_new;
    rc.tc.neg_lr = -t.lr;
    rc.tc.neg_lim_neg = -(float)a.geom.lim_neg;
    rc.tc.lim_pos = (float)a.geom.lim_pos;
    rc.tc.seed_mix = seed_mix(t.seed);
    rc.tc.two_m24 = 1.0f / 16777216.0f;
    // two-register VOP2 forms issue faster than forms with a scalar or literal operand: keep the
    // per-row operands of the per-element instructions in vector registers
    asm volatile("" : "+v"(rc.tc.neg_lr), "+v"(rc.tc.k), "+v"(rc.tc.two_m24), "+v"(rc.tc.seed_mix), "+v"(rc.tc.rd));
    rc.fast_div = __builtin_amdgcn_readfirstlane(fast > 0 ? 1 : 0) != 0;
    return rc;
}

__device__ __forceinline__ uint32_t no_exact_key() { return 0xffffffffu; }

// Four 6-bit codes -> the group's 24-bit word, as three shift-or instructions.
__device__ __forceinline__ uint32_t pack_codes(const uint32_t nc[4]) {
    uint32_t nw = nc[0];
    asm("v_lshl_or_b32 %0, %1, 6, %0" : "+v"(nw) : "v"(nc[1]));
    asm("v_lshl_or_b32 %0, %1, 12, %0" : "+v"(nw) : "v"(nc[2]));
    asm("v_lshl_or_b32 %0, %1, 18, %0" : "+v"(nw) : "v"(nc[3]));
    return nw;
}

template <bool FAST_DIV, typename CReb>
__device__ __forceinline__ uint32_t tick_group(uint32_t w, const float g[4], const TickConsts& tc, CReb c_reb,
                                               const Luts& l, uint32_t elem0) {
    uint32_t nc[4];
    const uint32_t x0 = hash_first(elem0);  // elem0 is a multiple of 4: elements k share it up to ^k
#pragma unroll
    for (int k = 0; k < 4; ++k)
        nc[k] = tick_code<FAST_DIV>(code_of(w, k), g[k], tc, x0 ^ (uint32_t)k, c_reb, l.q_off, l.fin);
    return pack_codes(nc);
}

// The same for a group whose first products come by addition (hash_delta): p0 is
// hash_first(elem0) * kHashMul1 and d[k-1] the wave-uniform delta of element k.
template <bool FAST_DIV, typename CReb>
__device__ __forceinline__ uint32_t tick_group_deltas(uint32_t w, const float g[4], const TickConsts& tc, CReb c_reb,
                                                      const Luts& l, uint32_t p0, const uint32_t d[3]) {
    uint32_t nc[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t p = k == 0 ? p0 : p0 + d[k - 1];
        nc[k] = tick_code_from_product<FAST_DIV>(code_of(w, k), g[k], tc, p, c_reb, l.q_off, l.fin);
    }
    return pack_codes(nc);
}

// Tick pass over a row re-read from memory with byte-granular state access: the fallback for
// rows of any length and alignment, for rows that need the plain division, and for rows whose
// scale changes although lr_scale is zero (a scale outside its clamp range).
__device__ __forceinline__ void apply_streamed(const UpdateTensor& t, int row, int lane, const RowCtx& rc,
                                               const Luts& l, int group_begin = 0, int group_end = 0x7fffffff) {
    const int gpr = t.in_features >> 2;
    const int g_end = group_end < gpr ? group_end : gpr;
    const float* g_row = t.grad_w + (size_t)row * t.in_features;
    uint8_t* s_row = t.state + (size_t)row * gpr * 3;
    const uint32_t row_elem = (uint32_t)(row + t.first_row) * (uint32_t)t.in_features;
    const RebasedCounters c_reb{l.c_f, rebase_ratio(rc)};
    for (int gi = group_begin + lane; gi < g_end; gi += kWave) {
        float g[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) g[k] = g_row[4 * gi + k];
        const uint32_t nw = tick_group<false>(load_group(s_row + 3 * gi), g, rc.tc, c_reb, l, row_elem + 4u * (uint32_t)gi);
        store_group(s_row + 3 * gi, nw);
    }
}

// A row held in registers: ITERS == ceil(gpr / 64) exactly and grad_w 16-byte aligned.  State words
// are fetched with 4-byte loads that reach one byte past their group.
// Every iteration but the last covers 64 full groups, so its loads, sums and stores need no masks
// and all addresses are one per-lane base plus a compile-time offset; in the last iteration lanes
// past the end of the row re-read the row's last group and are masked out of the sums and of the
// store.  EXACT: the row is exactly 256 * ITERS weights, no lane is ever masked, and every
// iteration's 256 elements are an aligned span of the element index, so the first products of
// the inner hash come by addition (hash_delta).
template <int ITERS, bool EXACT>
__device__ __forceinline__ void load_row(const UpdateTensor& t, int row, int lane, float4 (&q)[ITERS],
                                         uint32_t (&w)[ITERS]) {
    constexpr int kLast = ITERS - 1;
    const uint32_t gpr = (uint32_t)t.in_features >> 2;
    const float4* g_row = reinterpret_cast<const float4*>(t.grad_w + (size_t)row * t.in_features);
    const uint8_t* s_row = t.state + (size_t)row * gpr * 3;
    const uint32_t gi_last = (uint32_t)lane + kWave * kLast;
    const uint32_t gc_last = EXACT || gi_last < gpr ? gi_last : gpr - 1;
    const bool last_row = row == t.out_features - 1;  // wave-uniform
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
        const uint32_t gc = j < kLast ? (uint32_t)lane + kWave * j : gc_last;
        q[j] = load_grad4_once(g_row + gc);
        // only the row's last iteration can hold the tensor's last group
        w[j] = j < kLast ? load_group_dword_once(s_row + 3u * gc)
                         : load_group_dword_or_tail_once(s_row + 3u * gc, last_row && gc == gpr - 1);
    }
}

// One register-resident row whose loads have been issued (one contiguous burst per row): statistics,
// row epilogue and ticks.  SCALED: the rebase factor multiplies the residual counters (lr_scale != 0).
template <int ITERS, bool WITH_GS, bool EXACT>
__device__ __forceinline__ void update_row_resident(const BatchArgs& a, const UpdateTensor& t, int row, int lane,
                                                    const Luts& luts, const float4 (&q)[ITERS],
                                                    const uint32_t (&w)[ITERS]) {
    constexpr int kLast = ITERS - 1;
    const uint32_t gpr = (uint32_t)t.in_features >> 2;
    uint8_t* s_row = t.state + (size_t)row * gpr * 3;
    const bool last_live = EXACT || (uint32_t)lane + kWave * kLast < gpr;

    RowAcc acc;
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
        const bool live = j < kLast || last_live;
        const float g[4] = {live ? q[j].x : 0.0f, live ? q[j].y : 0.0f, live ? q[j].z : 0.0f,
                            live ? q[j].w : 0.0f};
        accumulate<WITH_GS, false>(acc, g, live, w[j], a.cd);
    }
    const RowCtx rc = finish_row<WITH_GS, false>(a, t, row, lane, acc, [&]() {
        uint32_t key = 0xffffffffu;
#pragma unroll
        for (int j = 0; j < ITERS; ++j) {
            const bool live = j < kLast || last_live;
            const float g[4] = {live ? q[j].x : 0.0f, live ? q[j].y : 0.0f, live ? q[j].z : 0.0f,
                                live ? q[j].w : 0.0f};
            key = group_min_key(key, g);
        }
        return key;
    });
    // without lr_scale the scale only moves when it sits outside its clamp range
    if (!rc.fast_div || (!WITH_GS && !scale_unchanged(rc))) {
        apply_streamed(t, row, lane, rc, luts);
        return;
    }
    const RebasedCounters rebased{luts.c_f, WITH_GS ? rebase_ratio(rc) : 1.0f};
    const uint32_t row_elem = (uint32_t)(row + t.first_row) * (uint32_t)t.in_features;
    // EXACT rows: deltas of the first hash products, wave-uniform per 256-element span and the same
    // for every span with equal bits 16..17 of the element index (a whole row, when it is short):
    // they live in vector registers and are rewritten only when those bits change
    uint32_t dv[3] = {0u, 0u, 0u};
    uint32_t dv_bits = 4u;
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
        const uint32_t gi = (uint32_t)lane + kWave * j;
        const float g[4] = {q[j].x, q[j].y, q[j].z, q[j].w};
        uint32_t nw;
        if (EXACT) {
            const uint32_t span = row_elem + 4u * kWave * j;
            const uint32_t sbits = (span >> 16) & 3u;  // wave-uniform
            if (sbits != dv_bits) {
                dv_bits = sbits;
                dv[0] = hash_delta(sbits, 1);
                dv[1] = hash_delta(sbits, 2);
                dv[2] = hash_delta(sbits, 3);
                // opaque: the products stay products (x * M + d, not (x + d') * M)
                asm volatile("" : "+v"(dv[0]), "+v"(dv[1]), "+v"(dv[2]));
            }
            const uint32_t p0 = hash_first(span + 4u * (uint32_t)lane) * kHashMul1;
            nw = WITH_GS ? tick_group_deltas<true>(w[j], g, rc.tc, rebased, luts, p0, dv)
                         : tick_group_deltas<true>(w[j], g, rc.tc, luts.c_f, luts, p0, dv);
        } else {
            nw = WITH_GS ? tick_group<true>(w[j], g, rc.tc, rebased, luts, row_elem + 4u * gi)
                         : tick_group<true>(w[j], g, rc.tc, luts.c_f, luts, row_elem + 4u * gi);
        }
        if (j < kLast || last_live) store_group_once(s_row + 3u * gi, nw);
    }
}

// One row of any length and alignment: read twice (the second read hits L2).
template <bool WITH_GS>
__device__ __forceinline__ void update_row_streamed(const BatchArgs& a, const UpdateTensor& t, int row,
                                                    int lane, const Luts& luts) {
    const int gpr = t.in_features >> 2;
    const float* g_row = t.grad_w + (size_t)row * t.in_features;
    const uint8_t* s_row = t.state + (size_t)row * gpr * 3;
    RowAcc acc;
    for (int gi = lane; gi < gpr; gi += kWave) {
        float g[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) g[k] = g_row[4 * gi + k];
        accumulate<WITH_GS, true>(acc, g, true, load_group(s_row + 3 * gi), a.cd);
    }
    const RowCtx rc = finish_row<WITH_GS, true>(a, t, row, lane, acc, no_exact_key);
    apply_streamed(t, row, lane, rc, luts);
}

// State word of group gc of a row; `last_row` (wave-uniform) tells that the row is the tensor's
// last, whose final group needs the early fetch.
__device__ __forceinline__ uint32_t load_row_word(const uint8_t* s_row, uint32_t gc, uint32_t gpr, bool last_row) {
    if (last_row) return load_group_dword_or_tail(s_row + 3u * gc, gc == gpr - 1);
    return load_group_dword(s_row + 3u * gc);
}

// One row of any length, 16-byte aligned, by one wave in two passes
// over the row: statistics first, ticks second.  The second pass finds the row in L2 or in the
// memory-side cache as long as the rows in flight fit there (5 waves per SIMD: 5120 rows, i.e.
// 100-230 MB at 5120-11008 weights a row); what the two passes buy is a register footprint of
// one chunk instead of one row, i.e. the occupancy of a short row at any length, and no
// hand-off between waves.  A chunk is kChunk iterations whose loads are issued back to back
// (8 measured best against 4, 6 and 11).
constexpr int kChunk = 8;

template <bool WITH_GS>
__device__ __forceinline__ void update_row_two_pass(const BatchArgs& a, const UpdateTensor& t, int row,
                                                    int lane, const Luts& luts) {
    const uint32_t gpr = (uint32_t)t.in_features >> 2;
    const int iters = (int)((gpr + kWave - 1) / kWave);
    const float4* g_row = reinterpret_cast<const float4*>(t.grad_w + (size_t)row * t.in_features);
    uint8_t* s_row = t.state + (size_t)row * gpr * 3;
    const bool last_row = row == t.out_features - 1;
    RowAcc acc;
    for (int c0 = 0; c0 < iters; c0 += kChunk) {
        float4 q[kChunk];
        uint32_t w[WITH_GS ? kChunk : 1];
#pragma unroll
        for (int j = 0; j < kChunk; ++j) {
            const uint32_t gi = (uint32_t)lane + (uint32_t)kWave * (uint32_t)(c0 + j);
            const uint32_t gc = gi < gpr ? gi : gpr - 1;
            q[j] = g_row[gc];
            if (WITH_GS) w[j] = load_row_word(s_row, gc, gpr, last_row);
        }
#pragma unroll
        for (int j = 0; j < kChunk; ++j) {
            // groups past the end add +0.0 (squares) and -+0.0 (0 * t): the sums do not change
            const bool live = (uint32_t)lane + (uint32_t)kWave * (uint32_t)(c0 + j) < gpr;
            const float g[4] = {live ? q[j].x : 0.0f, live ? q[j].y : 0.0f, live ? q[j].z : 0.0f,
                                live ? q[j].w : 0.0f};
            accumulate<WITH_GS, true>(acc, g, live, WITH_GS ? w[j] : 0u, a.cd);
        }
    }
    const RowCtx rc = finish_row<WITH_GS, true>(a, t, row, lane, acc, no_exact_key);
    if (!rc.fast_div) {
        apply_streamed(t, row, lane, rc, luts);
        return;
    }
    const RebasedCounters rebased{luts.c_f, rebase_ratio(rc)};
    const uint32_t row_elem = (uint32_t)(row + t.first_row) * (uint32_t)t.in_features;
    for (int c0 = 0; c0 < iters; c0 += kChunk) {
        float4 q[kChunk];
        uint32_t w[kChunk];
#pragma unroll
        for (int j = 0; j < kChunk; ++j) {
            const uint32_t gi = (uint32_t)lane + (uint32_t)kWave * (uint32_t)(c0 + j);
            const uint32_t gc = gi < gpr ? gi : gpr - 1;
            q[j] = load_grad4_once(g_row + gc);
            w[j] = load_row_word(s_row, gc, gpr, last_row);
        }
#pragma unroll
        for (int j = 0; j < kChunk; ++j) {
            if (c0 + j < iters) {  // wave-uniform
                const uint32_t gi = (uint32_t)lane + (uint32_t)kWave * (uint32_t)(c0 + j);
                const float g[4] = {q[j].x, q[j].y, q[j].z, q[j].w};
                const uint32_t nw = tick_group<true>(w[j], g, rc.tc, rebased, luts, row_elem + 4u * gi);
                if (gi < gpr) store_group(s_row + 3u * gi, nw);
            }
        }
    }
}

// Minimum waves per SIMD the compiler must leave room for: the tick arithmetic has long
// dependent chains, so the row's registers are budgeted to keep 3-4 waves resident for short
// rows and 2 for the longest.
constexpr int min_waves(int iters) { return iters <= 10 ? 4 : (iters <= 16 ? 3 : 2); }

// Waves (= rows) per workgroup of the dispatched kernels: the workgroup builds the tables once.
constexpr int kRowsPerGroup = 4;

// Register-resident rows, one per wave; blockIdx.y is the tensor, blockIdx.x * kRowsPerGroup the
// workgroup's first row.  Every tensor of a launch has the same out_features.
template <int ITERS, bool WITH_GS, bool EXACT>
__global__ __launch_bounds__(kWave* kRowsPerGroup, min_waves(ITERS)) void update_rows_kernel(BatchArgs a) {
    __shared__ Luts luts;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const UpdateTensor t = a.t[blockIdx.y];
    const int row_v = blockIdx.x * kRowsPerGroup + wave;
    const bool valid = row_v < t.out_features;  // wave-uniform
    const int row = valid ? row_v : t.out_features - 1;
    // the row's loads go out first; the tables are built while they are in flight
    float4 q[ITERS];
    uint32_t w[ITERS];
    load_row<ITERS, EXACT>(t, row, lane, q, w);
    build_luts(luts, a.cd, a.geom);
    if (!valid) return;
    update_row_resident<ITERS, WITH_GS, EXACT>(a, t, row, lane, luts, q, w);
}

// The tensor that holds row `grow` of the launch's concatenated row space; ti only moves forward.
// Everything here depends on blockIdx and kernel arguments only, so it lives in scalar registers.
__device__ __forceinline__ UpdateTensor locate_row(const BatchArgs& a, int grow, int& ti) {
    ti = __builtin_amdgcn_readfirstlane(ti);
    while (grow >= a.t[ti].row_start + a.t[ti].out_features) ++ti;  // monotonic
    ti = __builtin_amdgcn_readfirstlane(ti);
    return a.t[ti];
}

// Rows of any length and alignment, streamed (read twice); persistent one-wave workgroups.
template <bool WITH_GS>
__global__ __launch_bounds__(kThreads, 4) void update_rows_streamed_kernel(BatchArgs a) {
    __shared__ Luts luts;
    build_luts(luts, a.cd, a.geom);
    const int lane = threadIdx.x;
    int ti = 0;
    for (int grow_v = blockIdx.x; grow_v < a.total_rows; grow_v += gridDim.x) {
        const int grow = __builtin_amdgcn_readfirstlane(grow_v);
        const UpdateTensor t = locate_row(a, grow, ti);
        update_row_streamed<WITH_GS>(a, t, grow - t.row_start, lane, luts);
    }
}

template <bool WITH_GS>
__global__ __launch_bounds__(kThreads, 4) void update_rows_long_kernel(BatchArgs a) {
    __shared__ Luts luts;
    build_luts(luts, a.cd, a.geom);
    const int lane = threadIdx.x;
    int ti = 0;
    for (int grow_v = blockIdx.x; grow_v < a.total_rows; grow_v += gridDim.x) {
        const int grow = __builtin_amdgcn_readfirstlane(grow_v);
        const UpdateTensor t = locate_row(a, grow, ti);
        update_row_two_pass<WITH_GS>(a, t, grow - t.row_start, lane, luts);
    }
}

// ---------------------------------------------------------------------------
// Long rows: W cooperating waves per row, one row per workgroup (blockIdx.x the row, blockIdx.y
// the tensor).  Wave w keeps iterations [w*J, (w+1)*J) of the row in its registers, so a row of
// up to 64*J*W groups is register-resident with J*5 instead of ITERS*5 row registers per lane,
// and three or four waves per SIMD still fit.  The reference's per-lane partial sums are
// sequential in the iteration index, so the running sums are handed from wave to wave through
// LDS (W-1 barriers); the last wave owns the tree, the row epilogue and the commit, and
// publishes the tick constants for everybody's share of the tick pass.
// ---------------------------------------------------------------------------
struct SplitShared {
    Luts luts;
    float part_sq[kWave];
    float part_gs[kWave];
    uint32_t part_key[kWave];
    RowCtx rc;
    int fast_div;
};

constexpr int min_waves_split(int j) { return j <= 6 ? 4 : j <= 11 ? 3 : 2; }

// ALIGNED: rows of a whole number of 256-weight iterations (11008 = 43 * 256): no lane is ever
// masked, an iteration past the row's end is skipped by the whole wave, and every iteration is an
// aligned span of the element index, so the first hash products come by addition (hash_delta).
template <int J, int W, bool WITH_GS, bool ALIGNED, bool EVEN>
__global__ __launch_bounds__(kWave* W, min_waves_split(J)) void update_rows_split_kernel(BatchArgs a) {
    __shared__ SplitShared sh;
    const int lane = threadIdx.x & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const UpdateTensor t = a.t[blockIdx.y];
    const int row = blockIdx.x;
    const bool last_row = row == t.out_features - 1;
    const uint32_t gpr = (uint32_t)t.in_features >> 2;
    const int iters = (int)((gpr + kWave - 1) / kWave);
    // the row's iterations in W stretches: of J (EVEN false: the class of one row length, whose
    // stretches of J are even already and whose loops then carry no second bound), or of jn <= J,
    // as even as the row's length allows
    const int jn = EVEN ? (iters + W - 1) / W : J;
    const int j0 = w * jn;
    const float4* g_row = reinterpret_cast<const float4*>(t.grad_w + (size_t)row * t.in_features);
    uint8_t* s_row = t.state + (size_t)row * gpr * 3;
    // whether iteration j0 + jj is this wave's and inside the row (wave-uniform)
    auto mine = [&](int jj) { return (!EVEN || jj < jn) && j0 + jj < iters; };
    // whether lane's group of iteration j0 + jj exists: per iteration when ALIGNED
    auto live_at = [&](int jj) {
        return mine(jj) && (ALIGNED || (uint32_t)lane + (uint32_t)kWave * (uint32_t)(j0 + jj) < gpr);
    };

    float4 q[J];
    uint32_t words[J];
#pragma unroll
    for (int jj = 0; jj < J; ++jj) {
        const uint32_t gi = (uint32_t)lane + (uint32_t)kWave * (uint32_t)(j0 + jj);
        if (mine(jj)) {
            // lanes past the end of a ragged row re-read its last group and are masked below
            const uint32_t gc = ALIGNED || gi < gpr ? gi : gpr - 1;
            q[jj] = load_grad4_once(g_row + gc);
            words[jj] = last_row ? load_group_dword_or_tail_once(s_row + 3u * gc, gc == gpr - 1)
                                 : load_group_dword_once(s_row + 3u * gc);
        } else {
            q[jj] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            words[jj] = 0u;
        }
    }
    build_luts(sh.luts, a.cd, a.geom);  // while the row is in flight
    // What does not depend on the order happens before the hand-off, in all waves at once: the
    // squares, the products with t, and the minimum of the magnitude keys (a minimum may be
    // taken in any order).  Only the additions travel wave 0 -> 1 -> ... -> W-1.  (Long
    // per-wave stretches have no registers to spare for the squares and do it all in turn.)
    constexpr bool kPre = J <= 11;
    float sq[kPre ? J : 1][4], gt[kPre && WITH_GS ? J : 1][4];
    uint32_t my_key = 0xffffffffu;
    if (kPre) {
#pragma unroll
        for (int jj = 0; jj < J; ++jj) {
            // a skipped iteration holds zeros: +0.0 to the sums, the largest key to the minimum
            const bool live = ALIGNED || live_at(jj);  // (a skipped iteration of a whole row holds zeros already)
            const float g[4] = {live ? q[jj].x : 0.0f, live ? q[jj].y : 0.0f, live ? q[jj].z : 0.0f,
                                live ? q[jj].w : 0.0f};
            my_key = umin3(my_key, range_key(g[0]), range_key(g[1]));
            my_key = umin3(my_key, range_key(g[2]), range_key(g[3]));
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                sq[jj][k] = g[k] * g[k];
                if (WITH_GS) gt[jj][k] = g[k] * (float)(code_q(code_of(words[jj], k), a.cd) - 1);
            }
        }
    }
    RowAcc acc;
#pragma unroll
    for (int step = 0; step < W; ++step) {
        if (w == step) {
            if (step > 0) {
                acc.g_sq = sh.part_sq[lane];
                acc.grad_s = sh.part_gs[lane];
                acc.min_key = sh.part_key[lane];
            }
            if (kPre) {
                acc.min_key = umin(acc.min_key, my_key);
#pragma unroll
                for (int jj = 0; jj < J; ++jj)
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        acc.g_sq = acc.g_sq + sq[jj][k];
                        if (WITH_GS) acc.grad_s = acc.grad_s + gt[jj][k];
                    }
            } else {
#pragma unroll
                for (int jj = 0; jj < J; ++jj) {
                    const bool live = live_at(jj);
                    const float g[4] = {live ? q[jj].x : 0.0f, live ? q[jj].y : 0.0f, live ? q[jj].z : 0.0f,
                                        live ? q[jj].w : 0.0f};
                    accumulate<WITH_GS, true>(acc, g, live, words[jj], a.cd);
                }
            }
            if (step < W - 1) {
                sh.part_sq[lane] = acc.g_sq;
                sh.part_gs[lane] = acc.grad_s;
                sh.part_key[lane] = acc.min_key;
            }
        }
        if (step < W - 1) __syncthreads();
    }
    if (w == W - 1) {
        const RowCtx rc = finish_row<WITH_GS, true>(a, t, row, lane, acc, no_exact_key);
        if (lane == 0) {
            sh.rc = rc;
            sh.fast_div = rc.fast_div ? 1 : 0;
        }
    }
    __syncthreads();
    RowCtx rc = sh.rc;
    asm volatile("" : "+v"(rc.tc.neg_lr), "+v"(rc.tc.k), "+v"(rc.tc.two_m24), "+v"(rc.tc.seed_mix));  // VGPR operands
    const bool fast = __builtin_amdgcn_readfirstlane(sh.fast_div) != 0;
    if (!fast || (!WITH_GS && !scale_unchanged(rc))) {
        apply_streamed(t, row, lane, rc, sh.luts, j0 * kWave, (j0 + jn) * kWave);
        return;
    }
    const RebasedCounters rebased{sh.luts.c_f, WITH_GS ? rebase_ratio(rc) : 1.0f};
    const uint32_t row_elem = (uint32_t)(row + t.first_row) * (uint32_t)t.in_features;
    uint32_t dv[3] = {0u, 0u, 0u};
    uint32_t dv_bits = 4u;
#pragma unroll
    for (int jj = 0; jj < J; ++jj) {
        if (mine(jj)) {
            const uint32_t gi = (uint32_t)lane + (uint32_t)kWave * (uint32_t)(j0 + jj);
            const float g[4] = {q[jj].x, q[jj].y, q[jj].z, q[jj].w};
            uint32_t nw;
            if (ALIGNED) {
                const uint32_t span = row_elem + 4u * kWave * (uint32_t)(j0 + jj);
                const uint32_t sbits = (span >> 16) & 3u;  // wave-uniform
                if (sbits != dv_bits) {
                    dv_bits = sbits;
                    dv[0] = hash_delta(sbits, 1);
                    dv[1] = hash_delta(sbits, 2);
                    dv[2] = hash_delta(sbits, 3);
                    asm volatile("" : "+v"(dv[0]), "+v"(dv[1]), "+v"(dv[2]));  // the products stay products
                }
                const uint32_t p0 = hash_first(span + 4u * (uint32_t)lane) * kHashMul1;
                nw = WITH_GS ? tick_group_deltas<true>(words[jj], g, rc.tc, rebased, sh.luts, p0, dv)
                             : tick_group_deltas<true>(words[jj], g, rc.tc, sh.luts.c_f, sh.luts, p0, dv);
            } else {
                nw = WITH_GS ? tick_group<true>(words[jj], g, rc.tc, rebased, sh.luts, row_elem + 4u * gi)
                             : tick_group<true>(words[jj], g, rc.tc, sh.luts.c_f, sh.luts, row_elem + 4u * gi);
            }
            if (ALIGNED || gi < gpr) store_group_once(s_row + 3u * gi, nw);
        }
    }
}

int device_cu_count() {
    static int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
        return n;
    }();
    return cus;
}

// Every tensor of `a` has the rows of a.t[0]: one workgroup per kRowsPerGroup rows and tensor.
template <int ITERS, bool WITH_GS, bool EXACT>
hipError_t launch_variant(hipStream_t stream, const BatchArgs& a) {
    const dim3 grid((unsigned)((a.t[0].out_features + kRowsPerGroup - 1) / kRowsPerGroup), (unsigned)a.n_tensors);
    hipLaunchKernelGGL((update_rows_kernel<ITERS, WITH_GS, EXACT>), grid, dim3(kWave * kRowsPerGroup), 0, stream, a);
    return hipGetLastError();
}

template <bool WITH_GS>
hipError_t launch_streamed_variant(hipStream_t stream, const BatchArgs& a) {
    static int blocks_per_cu = [] {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, update_rows_streamed_kernel<WITH_GS>, kThreads, 0) != hipSuccess ||
            n <= 0)
            n = 2;
        return n;
    }();
    const int resident = device_cu_count() * blocks_per_cu;
    const dim3 grid(a.total_rows < resident ? a.total_rows : resident);
    hipLaunchKernelGGL(update_rows_streamed_kernel<WITH_GS>, grid, dim3(kThreads), 0, stream, a);
    return hipGetLastError();
}

template <int J, int W, bool WITH_GS, bool ALIGNED>
hipError_t launch_split_variant(hipStream_t stream, const BatchArgs& a) {
    const dim3 grid((unsigned)a.t[0].out_features, (unsigned)a.n_tensors);
    // 11008-wide rows (43 iterations) fall into four stretches of 11 as they are
    hipLaunchKernelGGL((update_rows_split_kernel<J, W, WITH_GS, ALIGNED, J != 11>), grid, dim3(kWave * W), 0, stream, a);
    return hipGetLastError();
}

template <bool WITH_GS>
hipError_t launch_long_variant(hipStream_t stream, const BatchArgs& a) {
    static int blocks_per_cu = [] {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, update_rows_long_kernel<WITH_GS>, kThreads, 0) != hipSuccess ||
            n <= 0)
            n = 2;
        return n;
    }();
    const int resident = device_cu_count() * blocks_per_cu;
    const dim3 grid(a.total_rows < resident ? a.total_rows : resident);
    hipLaunchKernelGGL(update_rows_long_kernel<WITH_GS>, grid, dim3(kThreads), 0, stream, a);
    return hipGetLastError();
}

constexpr int kLongClass = 2000;

template <int J, int W, bool ALIGNED>
hipError_t launch_split(hipStream_t stream, const BatchArgs& a) {
    return a.lr_scale != 0.0f ? launch_split_variant<J, W, true, ALIGNED>(stream, a)
                              : launch_split_variant<J, W, false, ALIGNED>(stream, a);
}

template <int ITERS, bool EXACT>
hipError_t launch_iters(hipStream_t stream, const BatchArgs& a) {
    return a.lr_scale != 0.0f ? launch_variant<ITERS, true, EXACT>(stream, a) : launch_variant<ITERS, false, EXACT>(stream, a);
}

// Row lengths (in units of 64 groups = 256 weights, rounded up) with a one-wave
// register-resident variant: every length up to 4096 weights.  Longer rows, up to 32768 weights,
// are shared register-resident by 4, 8 or 16 cooperating waves; beyond that one wave reads the
// row twice.
#define MCC_RESIDENT_ITERS(X) \
    X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15) X(16)

// Classes of the split kernel are encoded as 1000 + 10*J + W; a register-resident class is the
// row's iteration count, plus kExactClass when the row is exactly 256 weights per iteration.
constexpr int split_class(int j, int w) { return 1000 + 10 * j + w; }
constexpr int kExactClass = 100;

// Register-resident variant of a row of `in_features` (0 = streamed fallback).
int iters_class(const UpdateTensor& t) {
    const int iters = ((t.in_features >> 2) + kWave - 1) / kWave;
    const bool aligned = (reinterpret_cast<uintptr_t>(t.grad_w) & 15u) == 0;
    // a one-group tensor has no byte before its last group for the early fetch of that group
    if (!aligned || (long)t.out_features * (t.in_features >> 2) < 2) return 0;
    switch (iters) {
#define MCC_CASE(N) case N:
        MCC_RESIDENT_ITERS(MCC_CASE)
#undef MCC_CASE
        return iters + (t.in_features == 4 * kWave * iters ? kExactClass : 0);
        default: break;
    }
    // Cooperating waves, one row per workgroup, each wave a stretch of at most 8 iterations (11 for
    // the 7B FFN width): 4 waves up to 8192 weights, 8 up to 16384, 16 up to 32768.  Measured at
    // 4096 rows against the two-pass wave: 5120-wide 0.60 against 0.48 of the HBM peak, 8192-wide
    // 0.66 / 0.49, 14336-wide 0.58 / 0.46, 28672-wide 0.44 / 0.37, 20480-wide 0.40 either way.
    const int exact = t.in_features % (4 * kWave) == 0 ? kExactClass : 0;
    if (iters <= 32) return split_class(8, 4) + exact;
    if (iters <= 44) return split_class(11, 4) + exact;
    if (iters <= 64) return split_class(8, 8) + exact;
    if (iters <= 128) return split_class(8, 16) + exact;
    if (iters > 16) return kLongClass;
    return 0;
}

// Dispatched classes put the tensor on the grid's y axis and need equal out_features per launch;
// the persistent fallbacks walk one concatenated row space.
bool class_is_dispatched(int cls) { return cls != 0 && cls != kLongClass; }

hipError_t launch_class(hipStream_t stream, int cls, const BatchArgs& a) {
    switch (cls) {
#define MCC_CASE(N)                                  \
    case N: return launch_iters<N, false>(stream, a); \
    case N + kExactClass: return launch_iters<N, true>(stream, a);
        MCC_RESIDENT_ITERS(MCC_CASE)
#undef MCC_CASE
        case kLongClass:
            return a.lr_scale != 0.0f ? launch_long_variant<true>(stream, a) : launch_long_variant<false>(stream, a);
#define MCC_SPLIT_CASE(J, W)                                               \
    case split_class(J, W): return launch_split<J, W, false>(stream, a); \
    case split_class(J, W) + kExactClass: return launch_split<J, W, true>(stream, a);
        MCC_SPLIT_CASE(8, 4)
        MCC_SPLIT_CASE(11, 4)
        MCC_SPLIT_CASE(8, 8)
        MCC_SPLIT_CASE(8, 16)
#undef MCC_SPLIT_CASE
        default:
            return a.lr_scale != 0.0f ? launch_streamed_variant<true>(stream, a) : launch_streamed_variant<false>(stream, a);
    }
}

}  // namespace

// Enqueues the update-only step for `n` tensors (already validated).  Tensors are grouped by
// the kernel variant their row length needs (and, for the dispatched variants, by their row
// count); each group goes out in launches of at most kMaxUpdateBatch tensors.
hipError_t launch_update_batch(hipStream_t stream, const UpdateTensor* tensors, size_t n, int C,
                               float lr_scale, float rms_beta, float rms_eps) {
    BatchArgs a;
    a.cd = make_codec(C);
    a.geom = lut_geom(a.cd);
    a.lr_scale = lr_scale; a.rms_beta = rms_beta; a.rms_eps = rms_eps;
    // short lists (one tensor, a layer, a small model) are sorted on the stack: no host allocation
    constexpr size_t kOnStack = 256;
    int cls_stack[kOnStack];
    char done_stack[kOnStack];
    std::vector<int> cls_heap;
    std::vector<char> done_heap;
    int* cls = cls_stack;
    char* done = done_stack;
    if (n > kOnStack) {
        cls_heap.resize(n);
        done_heap.resize(n);
        cls = cls_heap.data();
        done = done_heap.data();
    }
    for (size_t i = 0; i < n; ++i) {
        cls[i] = iters_class(tensors[i]);
        done[i] = 0;
    }
    for (size_t i = 0; i < n; ++i) {
        if (done[i]) continue;
        const bool by_rows = class_is_dispatched(cls[i]);
        a.n_tensors = 0;
        a.total_rows = 0;
        for (size_t j = i; j < n; ++j) {
            if (done[j] || cls[j] != cls[i]) continue;
            if (by_rows && tensors[j].out_features != tensors[i].out_features) continue;
            // total_rows stays below 2^31: flush before the row space of one launch gets there
            if (a.n_tensors == kMaxUpdateBatch || a.total_rows > (1 << 30) - tensors[j].out_features) {
                const hipError_t e = launch_class(stream, cls[i], a);
                if (e != hipSuccess) return e;
                a.n_tensors = 0;
                a.total_rows = 0;
            }
            a.t[a.n_tensors] = tensors[j];
            a.t[a.n_tensors].row_start = a.total_rows;
            a.total_rows += tensors[j].out_features;
            ++a.n_tensors;
            done[j] = 1;
        }
        if (a.n_tensors > 0) {
            const hipError_t e = launch_class(stream, cls[i], a);
            if (e != hipSuccess) return e;
        }
    }
    return hipSuccess;
}

hipError_t launch_update_dense(hipStream_t stream, uint8_t* state, float* scale, float* v,
                               const float* grad_w, int C, int in_features, int out_features,
                               float lr, float lr_scale, float rms_beta, float rms_eps,
                               uint32_t seed, int first_row) {
    UpdateTensor t;
    t.state = state; t.scale = scale; t.v = v; t.grad_w = grad_w;
    t.in_features = in_features; t.out_features = out_features;
    t.row_start = 0; t.seed = seed; t.lr = lr; t.first_row = first_row;
    return launch_update_batch(stream, &t, 1, C, lr_scale, rms_beta, rms_eps);
}

}  // namespace mcc
