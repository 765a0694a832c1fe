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

namespace mcc {

// lowbias32 (kernels/compact_counter.cl:17-21)
MCC_HD uint32_t hash_u32(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

// 24-bit word of one packed group -> code k (kernels/compact_counter.cl:25-31)
MCC_HD uint32_t code_of(uint32_t word, int k) { return (word >> (6 * k)) & 0x3fu; }

// Per-row constants of the tick (kernels/compact_counter.cl:118,123-124): the
// reference evaluates them per element from the same per-row operands, so
// hoisting them changes no bit.
struct RowConsts {
    float dn;      // denom[row]
    float k;       // Cf / s_new
    float ratio;   // s_old / s_new
    float neg_lr;  // -lr
};

// Constants of the state encoding for one counter depth C (lv = 2C-1 levels per
// ternary value).  (code * magic) >> 16 == code / lv for every code < 64.
struct Codec {
    int C, lv;
    uint32_t magic;
    float Cf, inv_c;
};

MCC_HD Codec make_codec(int C) {
    Codec cd;
    cd.C = C;
    cd.lv = 2 * C - 1;
    cd.magic = 65536u / (uint32_t)cd.lv + 1u;
    cd.Cf = (float)C;
    cd.inv_c = 1.0f / (float)C;
    return cd;
}

// t + 1 = code / lv  (kernels/compact_counter.cl:10)
MCC_HD int code_q(uint32_t code, const Codec& cd) { return (int)((code * cd.magic) >> 16); }

// Largest |floor(val)| that can still matter.  With t = code/lv - 1 in
// [-1, 63/lv - 1] the ternary value saturates whenever |total| >= (63/lv + 1)*C,
// which is <= 64 for every C with 3*(2C-1) <= 64; totals beyond that all give
// the same saturated code, so floor(val) is clamped to +-kTotalClamp first.
constexpr float kTotalClamp = 128.0f;

// One stochastic-rounding tick (kernels/compact_counter.cl:120-136).
//   code  : current 6-bit code          gw   : weight gradient of this element
//   elem  : row*in + i (the RNG index)  seed : update seed
// Returns the new 6-bit code.
//
// Differences in form (not in value) from the kernel text, valid for finite
// inputs with |val| < 2^31:
//  * floor(val) is clamped to +-kTotalClamp (see above);
//  * carry = trunc(ccv / Cf) is evaluated as trunc((ccv +- 0.5) * (1/Cf)):
//    ccv is an integer with |ccv| <= 129, so (|ccv| + 0.5)/C has a fractional
//    part in [0.5/C, 1 - 0.5/C], at least 0.045 away from an integer, far more
//    than the 2^-16 rounding error of the product;
//  * rem = ccv - carry*Cf is one fma: both steps are exact on small integers.
MCC_HD uint32_t tick_code(uint32_t code, float gw, const RowConsts& rc, uint32_t seed,
                          uint32_t elem, const Codec& cd) {
    const int C = cd.C, lv = cd.lv;
    const float Cf = cd.Cf, inv_c = cd.inv_c;
    const int q = code_q(code, cd);               // t + 1
    const int c = (int)code - q * lv - (C - 1);
    const float tick = (rc.neg_lr * (gw / rc.dn)) * rc.k;
    const float c_reb = (float)c * rc.ratio;
    const float val = c_reb + tick;
    const float f = floorf(val);
    const float frac = val - f;
    const uint32_t h = hash_u32(seed ^ hash_u32(elem));
    const float rnd = (float)(h & 0x00ffffffu) * (1.0f / 16777216.0f);
    const float fc = fminf(fmaxf(f, -kTotalClamp), kTotalClamp);
    const float ccv = fc + (rnd < frac ? 1.0f : 0.0f);
    const float carry = truncf((ccv + copysignf(0.5f, ccv)) * inv_c);
    float rem = fmaf(-carry, Cf, ccv);
    const int nt = (q - 1) + (int)carry;
    const int ct = nt < -1 ? -1 : (nt > 1 ? 1 : nt);
    if (ct != nt) rem = fminf(fmaxf(ccv, -1.0f), 1.0f) * (Cf - 1.0f);
    const int ri = (int)rem;
    return (uint32_t)((ct + 1) * lv + ri + (C - 1));
}

// Row statistics epilogue (kernels/compact_counter.cl:92-99), given the tree
// totals sum_sq = sum g^2 and sum_gt = sum g*t of one row.
struct RowStats {
    float v_new, denom, scale_new;
};

MCC_HD RowStats finish_row_stats(float sum_sq, float sum_gt, float v_old, float scale_old,
                                 int in_features, float lr_scale, float rms_beta, float rms_eps) {
    const float gsq = sum_sq / (float)in_features;
    const float gs = sum_gt / sqrtf((float)in_features);
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
