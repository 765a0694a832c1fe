// Counter-synapse arithmetic shared by the HIP kernels.
//
// Every float operation below is one IEEE-754 binary32 round-to-nearest-even
// operation: translation units that include this header are compiled with
// -ffp-contract=off and correctly rounded division / square root.  The
// formulas follow kernels/compact_counter.cl:7-36,118-137 of MotifCL.
//
// The header also compiles as plain C++ (MCC_HD expands to nothing) so that the
// arithmetic can be checked exhaustively on the CPU.
#pragma once

#include <cstdint>
#include <cmath>

#if defined(__HIPCC__)
#define MCC_HD __host__ __device__ __forceinline__
#else
#define MCC_HD inline
#endif
#define MCC_HDC constexpr MCC_HD  // also usable in constant expressions (the tables are built at compile time)

namespace mcc {

// lowbias32 (kernels/compact_counter.cl:17-21), split after its first xor-shift: the four
// elements of a packed group have indices e, e+1, e+2, e+3 with e a multiple of 4, and
// (e + k) ^ ((e + k) >> 16) == (e ^ (e >> 16)) ^ k for k < 4, so the first step is shared.
constexpr uint32_t kHashMul1 = 0x7feb352du, kHashMul2 = 0x846ca68bu;

MCC_HD uint32_t hash_first(uint32_t x) { return x ^ (x >> 16); }

MCC_HD uint32_t hash_rest(uint32_t x) {
    x *= kHashMul1;
    x ^= x >> 15;
    x *= kHashMul2;
    x ^= x >> 16;
    return x;
}

MCC_HD uint32_t hash_u32(uint32_t x) { return hash_rest(hash_first(x)); }

// hash_rest without its last xor-shift, given its first product p = x * kHashMul1:
// hash_rest(x) == u ^ (u >> 16) with u = hash_open_from_product(x * kHashMul1).
MCC_HD uint32_t hash_open_from_product(uint32_t p) {
    p ^= p >> 15;
    p *= kHashMul2;
    return p;
}

MCC_HD uint32_t hash_open(uint32_t x) { return hash_open_from_product(x * kHashMul1); }

// The four elements of a group enter the inner hash as x ^ k, k = 0..3, with x = hash_first of
// the group's first element.  x ^ k == x + ((s ^ k) - s) for s = x & 3, so their first products
// are (x ^ k) * kHashMul1 == x * kHashMul1 + hash_delta(s, k) (mod 2^32): one multiplication and
// three additions per group, and s -- bits 16..17 of the element index -- is the same for every
// group of a 256-element aligned span.
MCC_HD uint32_t hash_delta(uint32_t s, uint32_t k) { return ((s ^ k) - s) * kHashMul1; }

// The draw of kernels/compact_counter.cl:127 is hash(seed ^ hash(elem)).  With h = u ^ (u >> 16)
// the inner hash and y = seed ^ h, the outer hash starts with y ^ (y >> 16), and
//   y >> 16 = (seed >> 16) ^ (h >> 16) = (seed >> 16) ^ (u >> 16)        ((u >> 16) >> 16 == 0)
//   y ^ (y >> 16) = seed ^ u ^ (u >> 16) ^ (seed >> 16) ^ (u >> 16) = (seed ^ (seed >> 16)) ^ u
// so the inner hash's last step, the xor with the seed and the outer hash's first step collapse
// into one xor with a per-tensor constant.
MCC_HD uint32_t seed_mix(uint32_t seed) { return seed ^ (seed >> 16); }

// hash_u32(seed ^ hash_rest(x)) given mix = seed_mix(seed), from x or from p = x * kHashMul1
MCC_HD uint32_t draw_hash_from_product(uint32_t mix, uint32_t p) { return hash_rest(mix ^ hash_open_from_product(p)); }
MCC_HD uint32_t draw_hash(uint32_t mix, uint32_t x) { return draw_hash_from_product(mix, x * kHashMul1); }

// 24-bit word of one packed group -> code k (kernels/compact_counter.cl:25-31)
MCC_HD uint32_t code_of(uint32_t word, int k) { return (word >> (6 * k)) & 0x3fu; }

// Constants of the state encoding for one counter depth C (lv = 2C-1 levels per
// ternary value).  (code * magic) >> 16 == code / lv for every code < 64.
struct Codec {
    int C, lv;
    uint32_t magic;    // (code * magic) >> 16 == code / lv for code < 64
    uint32_t c_magic;  // (n * c_magic) >> 16 == n / C for n < 5000 (C <= 11)
    float Cf, inv_c;
};

MCC_HDC Codec make_codec(int C) {
    Codec cd{};
    cd.C = C;
    cd.lv = 2 * C - 1;
    cd.magic = 65536u / (uint32_t)cd.lv + 1u;
    cd.c_magic = 65536u / (uint32_t)C + 1u;
    cd.Cf = (float)C;
    cd.inv_c = 1.0f / (float)C;
    return cd;
}

// t + 1 = code / lv  (kernels/compact_counter.cl:10)
MCC_HDC int code_q(uint32_t code, const Codec& cd) { return (int)((code * cd.magic) >> 16); }

// ---------------------------------------------------------------------------
// The tick after val = c_reb + tick is a function of three small integers:
// q = t + 1 (from the old code), total = floor(val) + [rnd < frac], and C
// (kernels/compact_counter.cl:126-136).  It is tabulated once per kernel launch:
//
//   fin[q * width + (total + lim_neg)] = new 6-bit code
//
// Range of `total` that can matter: with t = q - 1 in [-1, rows - 2]
// (rows = 63/lv + 1 distinct q values) the ternary value saturates upward as
// soon as carry >= 3, i.e. total >= 3C, and downward as soon as
// carry <= -rows, i.e. total <= -rows*C.  floor(val) is therefore clamped to
// [-lim_neg, lim_pos] = [-(rows*C + 1), 3C] first: every clamped value, with or
// without the +1 of the stochastic round, lies in the same saturated region as
// the unclamped one.  Valid for finite val (|val| < 2^31 in the reference's
// own terms, where its float->int conversions stop being defined).
// ---------------------------------------------------------------------------
struct LutGeom {
    int rows;      // distinct q = code / lv values
    int lim_neg;   // clamp of floor(val) below, as a positive number
    int lim_pos;   // clamp of floor(val) above
    int width;     // number of distinct totals: lim_neg + lim_pos + 2
    uint32_t width_magic;  // (idx * width_magic) >> 20 == idx / width for idx < rows * width
};

constexpr int kLutFinMaxBytes = 4480;  // C = 1: 64 rows x width 70

MCC_HDC LutGeom lut_geom(const Codec& cd) {
    LutGeom g{};
    g.rows = 63 / cd.lv + 1;
    g.lim_neg = g.rows * cd.C + 1;
    g.lim_pos = 3 * cd.C;
    g.width = g.lim_neg + g.lim_pos + 2;
    g.width_magic = (1u << 20) / (uint32_t)g.width + 1u;
    return g;
}

// New code for old q = t + 1 and integer total = ccv (kernels/compact_counter.cl:129-136).
MCC_HDC uint32_t fin_entry(int total, int q, const Codec& cd) {
    const int C = cd.C;
    const int mag = total < 0 ? -total : total;
    const int mq = (int)(((uint32_t)mag * cd.c_magic) >> 16);  // mag / C (mag <= rows * C + 2)
    const int carry = total < 0 ? -mq : mq;               // trunc(ccv / Cf)
    int rem = total - carry * C;                          // ccv - carry * Cf
    const int nt = (q - 1) + carry;
    const int ct = nt < -1 ? -1 : (nt > 1 ? 1 : nt);
    if (ct != nt) rem = (total > 0 ? 1 : (total < 0 ? -1 : 0)) * (C - 1);
    return (uint32_t)((ct + 1) * cd.lv + rem + (C - 1));
}

// Decode tables, indexed by the 6-bit code:
//   q_off[code] = (code / lv) * width + lim_neg     (row of the fin table, pre-biased so that
//                                                     fin index = q_off + total)
//   c_reb[code] = (float)(code % lv - (C-1)) * (s_old / s_new)
// c_reb is the rebased residual counter of kernels/compact_counter.cl:124; it depends on the
// row through the scale ratio only, so it is tabulated once per row (64 products) instead of
// once per weight.
MCC_HDC int code_c(uint32_t code, const Codec& cd) {
    return (int)code - code_q(code, cd) * cd.lv - (cd.C - 1);
}

MCC_HDC int q_off_entry(uint32_t code, const Codec& cd, const LutGeom& g) {
    return code_q(code, cd) * g.width + g.lim_neg;
}

MCC_HD float c_reb_entry(uint32_t code, const Codec& cd, float ratio) {
    return (float)code_c(code, cd) * ratio;
}

MCC_HDC int fin_size(const LutGeom& g) { return g.rows * g.width; }

MCC_HDC void fill_fin_entry(int idx, const Codec& cd, const LutGeom& g, uint8_t* fin) {
    const int q = (int)(((uint32_t)idx * g.width_magic) >> 20);  // idx / width
    const int til = idx - q * g.width;
    fin[idx] = (uint8_t)fin_entry(til - g.lim_neg, q, cd);
}

// Division by the per-row denominator, gw / dn, without a per-element division: with
// rd = RN64(1 / (double)dn) computed once per row,
//     q = RN32(RN64((double)gw * rd))
// is RN32(gw / dn) whenever that quotient is a normal binary32 number or zero.  Proof sketch: the
// double product is q* (1 + e) with q* = gw / dn and |e| < 2^-51.9.  A rounding boundary of
// binary32 next to q* is an odd multiple m of 2^(k-24) for q* in [2^k, 2^(k+1)); with the
// significands G, D of gw and dn (integers below 2^24), |q* - m| = 2^(k-24) |G 2^s - M D| / D with
// s in {24, 25} and M odd, and G 2^s = M D is impossible (D would need 24 factors of two), so
// |q* - m| > 2^(k-48), sixteen times the error of the double product: both round to the same
// binary32 number.  For subnormal quotients exact ties exist and the argument fails, so the row
// statistics pass collects what bounds the quotients: dn in [2^-40, 2^40], the sum of squares
// (|gw| from above) and the minimum over the row of range_key(gw) (non-zero |gw| from below,
// 2^-60).  Rows that fail take the plain division.  Three instructions per element
// (v_cvt_f64_f32, v_mul_f64, v_cvt_f32_f64) instead of a reciprocal product and four fmas.
MCC_HD uint32_t float_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __float_as_uint(f);
#else
    uint32_t u;
    __builtin_memcpy(&u, &f, 4);
    return u;
#endif
}

// Orders floats by magnitude with zero mapped above everything: (bits << 1) - 1.
MCC_HD uint32_t range_key(float gw) { return (float_bits(gw) << 1) - 1u; }

MCC_HD bool row_takes_fast_division(float dn, float row_sum_sq, uint32_t row_min_key) {
    return dn >= 0x1p-40f && dn <= 0x1p40f && row_sum_sq < 0x1p100f && row_min_key >= range_key(0x1p-60f);
}

// The same decision from the smallest |gw| of the row, zeros included (one v_min3_f32 per two
// elements instead of a key per element): +1 fast, -1 exact division, 0 undecided -- the row
// holds an exact zero, which hides whether it also holds a non-zero value below 2^-60, and the
// caller looks again with range_key.
MCC_HD int fast_division_from_min_abs(float dn, float row_sum_sq, float row_min_abs) {
    if (!(dn >= 0x1p-40f && dn <= 0x1p40f && row_sum_sq < 0x1p100f)) return -1;
    if (row_min_abs >= 0x1p-60f) return 1;
    return row_min_abs == 0.0f ? 0 : -1;
}

template <bool FAST>
MCC_HD float div_by_row(float gw, float dn, double rd) {
    if (!FAST) return gw / dn;
    return (float)((double)gw * rd);
}

// rd need not be the correctly rounded reciprocal: with a relative error e_rd the double product is
// q* (1 + e), |e| <= e_rd + 2^-53, and the argument above goes through for e_rd <= 2^-49.1.  The
// device takes the hardware's approximate reciprocal through two Newton steps (a few 2^-53; five
// instructions instead of the twenty-five of a correctly rounded division); dn is in
// [2^-40, 2^40] wherever rd is used, so nothing needs scaling.
MCC_HD double row_reciprocal(float dn) {
#if defined(__HIP_DEVICE_COMPILE__)
    const double d = (double)dn;
    double r = __builtin_amdgcn_rcp(d);
    r = __builtin_fma(r, __builtin_fma(-d, r, 1.0), r);
    r = __builtin_fma(r, __builtin_fma(-d, r, 1.0), r);
    return r;
#else
    return 1.0 / (double)dn;
#endif
}

MCC_HD float clamp_f(float x, float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_fmed3f(x, lo, hi);
#else
    return fminf(fmaxf(x, lo), hi);
#endif
}

// Per-row constants of the tick (kernels/compact_counter.cl:118,123).
struct TickConsts {
    float dn;         // denom[row]
    double rd;        // row_reciprocal(denom[row])
    float k;          // Cf / s_new
    float neg_lr;     // -lr
    float neg_lim_neg, lim_pos;  // clamp of floor(val), as floats
    float two_m24;               // 2^-24 (kept in a register: see the kernel)
    uint32_t seed_mix;           // seed_mix(seed)
};

// One stochastic-rounding tick (kernels/compact_counter.cl:120-136).
//   code : current 6-bit code           gw   : weight gradient of this element
//   elem_x : hash_first(row*in + i), the RNG index after the first xor-shift
//   c_reb, q_off : the decode tables above;  fin : the (q, total) -> code table
// Returns the new 6-bit code.
//   first_product : hash_first(row*in + i) * kHashMul1 (see hash_delta)
template <bool FAST_DIV, typename CReb, typename QOff, typename Fin>
MCC_HD uint32_t tick_code_from_product(uint32_t code, float gw, const TickConsts& tc, uint32_t first_product,
                                       CReb c_reb, QOff q_off, Fin fin) {
    const float tick = (tc.neg_lr * div_by_row<FAST_DIV>(gw, tc.dn, tc.rd)) * tc.k;
    const float val = c_reb[code] + tick;
    const float f = floorf(val);
    const float frac = val - f;
    const uint32_t h = draw_hash_from_product(tc.seed_mix, first_product);
    const float rnd = (float)(h & 0x00ffffffu) * tc.two_m24;
    // q_off + floor + [rnd < frac]: one add-with-carry on the GPU
    const int idx = q_off[code] + (int)clamp_f(f, tc.neg_lim_neg, tc.lim_pos) + (rnd < frac ? 1 : 0);
    return fin[idx];
}

template <bool FAST_DIV, typename CReb, typename QOff, typename Fin>
MCC_HD uint32_t tick_code(uint32_t code, float gw, const TickConsts& tc, uint32_t elem_x,
                          CReb c_reb, QOff q_off, Fin fin) {
    return tick_code_from_product<FAST_DIV>(code, gw, tc, elem_x * kHashMul1, c_reb, q_off, fin);
}

// Row statistics epilogue (kernels/compact_counter.cl:92-99), given the tree
// totals sum_sq = sum g^2 and sum_gt = sum g*t of one row.
struct RowStats {
    float v_new, denom, scale_new;
};

MCC_HD RowStats finish_row_stats(float sum_sq, float sum_gt, float v_old, float scale_old,
                                 int in_features, float lr_scale, float rms_beta, float rms_eps) {
    // a power of two divides exactly like its reciprocal multiplies (one rounding of the same real
    // number either way), and the reciprocal's bits are its exponent: no division
    float gsq;
    if ((in_features & (in_features - 1)) == 0) {
        int log2_in = 0;
        while ((1 << log2_in) < in_features) ++log2_in;  // a kernel argument: scalar, a handful of instructions
        const uint32_t inv_bits = (uint32_t)(127 - log2_in) << 23;
        float inv;
        __builtin_memcpy(&inv, &inv_bits, 4);
        gsq = sum_sq * inv;
    } else {
        gsq = sum_sq / (float)in_features;
    }
    // lr_scale == 0: the product below is +-0 for every finite gs and the scale stays as it is
    // (up to its clamp), so the square root and the division are skipped
    const float gs = lr_scale != 0.0f ? sum_gt / sqrtf((float)in_features) : 0.0f;
    const float a = rms_beta * v_old;
    const float b = (1.0f - rms_beta) * gsq;
    RowStats r;
    r.v_new = a + b;
    r.denom = fmaxf(sqrtf(r.v_new), rms_eps);
    const float sn = scale_old - lr_scale * gs;
    r.scale_new = fminf(fmaxf(sn, 1e-5f), 10.0f);
    return r;
}

}  // namespace mcc
