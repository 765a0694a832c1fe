// CPU build of the kernels' tick arithmetic (motifcl_amd/csrc/counter_math.hpp) checked
// against the oracle's literal restatement (oracle/counter_oracle.c) on millions of
// inputs, including every code, every C, integral / near-integral / huge / tiny values.
// Build: g++ -O2 -ffp-contract=off -fopenmp check_tick_math.cpp ../../oracle/counter_oracle.c-as-lib
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>
#include <vector>

#include "../../motifcl_amd/csrc/counter_math.hpp"

extern "C" int oracle_tick_code(int code, float gw, float s_old, float s_new, float dn, int C,
                                float lr, uint32_t seed, uint32_t elem);

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint64_t next_u64() {
    rng_state ^= rng_state << 13; rng_state ^= rng_state >> 7; rng_state ^= rng_state << 17;
    return rng_state;
}
static double uni() { return (next_u64() >> 11) * (1.0 / 9007199254740992.0); }
static float log_uniform(double lo, double hi) { return (float)std::exp(std::log(lo) + uni() * (std::log(hi) - std::log(lo))); }

int main(int argc, char** argv) {
    const long per_c = argc > 1 ? std::atol(argv[1]) : 2000000;
    long mismatches = 0, checked = 0, n_fast = 0;
    for (int C = 1; C <= 11; ++C) {
        const mcc::Codec cd = mcc::make_codec(C);
        const mcc::LutGeom g = mcc::lut_geom(cd);
        if (mcc::fin_size(g) > mcc::kLutFinMaxBytes) { std::printf("LUT too large for C=%d\n", C); return 2; }
        std::vector<uint8_t> fin(mcc::fin_size(g));
        std::vector<int> q_off(64);
        std::vector<float> c_reb(64);
        for (uint32_t code = 0; code < 64; ++code) q_off[code] = mcc::q_off_entry(code, cd, g);
        for (int i = 0; i < mcc::fin_size(g); ++i) mcc::fill_fin_entry(i, cd, g, fin.data());
        // the table build's divisions by C and by the table width
        for (int n = 0; n < 5000; ++n)
            if ((int)(((uint32_t)n * cd.c_magic) >> 16) != n / C) { std::printf("division by C fails C=%d n=%d\n", C, n); return 2; }
        for (int i = 0; i < mcc::fin_size(g); ++i)
            if ((int)(((uint32_t)i * g.width_magic) >> 20) != i / g.width) { std::printf("division by the width fails C=%d i=%d\n", C, i); return 2; }
        // (code * magic) >> 16 == code / lv
        for (uint32_t code = 0; code < 64; ++code)
            if (mcc::code_q(code, cd) != (int)code / cd.lv) { std::printf("magic division fails C=%d code=%u\n", C, code); return 2; }
        auto make_tc = [&](float dn, float s_old, float s_new, float lr, uint32_t seed) {
            mcc::TickConsts tc;
            tc.dn = dn; tc.rd = mcc::row_reciprocal(dn); tc.k = cd.Cf / s_new; tc.neg_lr = -lr;
            tc.neg_lim_neg = -(float)g.lim_neg; tc.lim_pos = (float)g.lim_pos;
            tc.seed_mix = mcc::seed_mix(seed); tc.two_m24 = 1.0f / 16777216.0f;
            for (uint32_t code = 0; code < 64; ++code) c_reb[code] = mcc::c_reb_entry(code, cd, s_old / s_new);
            return tc;
        };
        const float lrs[] = {3e-3f, 0.05f, 1.0f, 16.0f, 100.0f, 0.0f};
        for (long it = 0; it < per_c; ++it) {
            const int code = (int)(next_u64() % 64);
            const int mode = (int)(next_u64() % 8);
            float lr = lrs[next_u64() % 6];
            float dn = (next_u64() & 15) ? log_uniform(1e-8, 1e3) : log_uniform(1e-30, 1e30), s_old = log_uniform(1e-5, 10.0), s_new = log_uniform(1e-5, 10.0);
            float gw;
            if (mode == 0) { s_new = s_old; }                       // lr_scale = 0: ratio is exactly 1
            if (mode == 1) gw = 0.0f;
            else if (mode == 2) gw = (uni() < 0.5 ? -1.f : 1.f) * log_uniform(1e-44, 1e-6);
            else if (mode == 3) gw = (uni() < 0.5 ? -1.f : 1.f) * log_uniform(1e3, 1e12);
            else gw = (float)((uni() - 0.5) * 2.0) * log_uniform(1e-6, 10.0);
            if (mode == 4 || mode == 5) {
                // integral or near-integral val: tick = -gw exactly (dn = 64, lr = 16, C/s_new = 4)
                dn = 64.0f; lr = 16.0f; s_new = (float)C / 4.0f; s_old = s_new;
                gw = (float)((long)(next_u64() % 401) - 200);
                if (mode == 5) gw = std::nextafterf(gw, uni() < 0.5 ? -1e9f : 1e9f);
            }
            // the reference's conversions are undefined from |val| = 2^31 on: stay inside the contract
            const float bound = std::fabs((lr * (gw / dn)) * ((float)C / s_new)) + 64.0f * (s_old / s_new);
            if (!(bound < 2.0e9f)) continue;
            const uint32_t seed = (uint32_t)next_u64(), elem = (uint32_t)next_u64();
            const mcc::TickConsts tc = make_tc(dn, s_old, s_new, lr, seed);
            // the kernel decides per row from the row's sum of squares and smallest non-zero
            // magnitude; a one-element "row" exercises both branches of that decision
            const bool fast = mcc::row_takes_fast_division(dn, (next_u64() & 7) ? gw * gw * 64.0f : 0x1p110f,
                                                           mcc::range_key(gw));
            n_fast += fast;
            const uint32_t got = fast
                ? mcc::tick_code<true>((uint32_t)code, gw, tc, mcc::hash_first(elem), c_reb.data(), q_off.data(), fin.data())
                : mcc::tick_code<false>((uint32_t)code, gw, tc, mcc::hash_first(elem), c_reb.data(), q_off.data(), fin.data());
            const int exp = oracle_tick_code(code, gw, s_old, s_new, dn, C, lr, seed, elem);
            ++checked;
            if ((int)got != exp) {
                if (mismatches < 10)
                    std::printf("MISMATCH C=%d code=%d gw=%a dn=%a s_old=%a s_new=%a lr=%a seed=%u elem=%u got=%u exp=%d\n",
                                C, code, gw, dn, s_old, s_new, lr, seed, elem, got, exp);
                ++mismatches;
            }
        }
        // every (q, total) pair of the table against the oracle through exact integer ticks
        for (int code = 0; code < 64; ++code)
            for (int gi = -4 * 64; gi <= 4 * 64; ++gi) {
                const float s = (float)C / 4.0f;
                const mcc::TickConsts tc = make_tc(64.0f, s, s, 16.0f, 1u);
                const uint32_t got = mcc::tick_code<true>((uint32_t)code, (float)gi, tc, mcc::hash_first(2u), c_reb.data(), q_off.data(), fin.data());
                const int exp = oracle_tick_code(code, (float)gi, s, s, 64.0f, C, 16.0f, 1u, 2u);
                ++checked;
                if ((int)got != exp) { if (mismatches < 10) std::printf("TABLE MISMATCH C=%d code=%d g=%d got=%u exp=%d\n", C, code, gi, got, exp); ++mismatches; }
            }
    }
    // the reciprocal product tolerates a reciprocal that is off by a few units in the last place
    // (the device refines the hardware's approximation instead of dividing)
    for (long it = 0; it < 4000000; ++it) {
        const float dn = log_uniform(1e-12, 1e12);
        const float gw = (uni() < 0.5 ? -1.f : 1.f) * log_uniform(1e-18, 1e15);
        double rd = 1.0 / (double)dn;
        const int ulps = (int)(next_u64() % 9) - 4;
        for (int u = 0; u < (ulps < 0 ? -ulps : ulps); ++u) rd = std::nextafter(rd, ulps < 0 ? 0.0 : 1e300);
        if ((float)((double)gw * rd) != gw / dn) { std::printf("reciprocal product fails gw=%a dn=%a ulps=%d\n", gw, dn, ulps); return 2; }
    }
    // division by a power of two as a product with its reciprocal (finish_row_stats)
    for (long it = 0; it < 2000000; ++it) {
        const float x = (next_u64() & 7) ? log_uniform(1e-44, 1e38) : log_uniform(1e-45, 1e-36);
        const int k = (int)(next_u64() % 21);
        const mcc::RowStats a = mcc::finish_row_stats(x, 0.f, 0.f, 1.f, 1 << k, 0.f, 0.f, 0.f);
        if (a.v_new != x / (float)(1 << k)) { std::printf("power-of-two division fails x=%a k=%d\n", x, k); return 2; }
    }
    // collapsed seed xor: hash(seed ^ hash(elem)) == hash_rest(seed_mix(seed) ^ hash_open(hash_first(elem)))
    for (int i = 0; i < 4000000; ++i) {
        const uint32_t seed = (uint32_t)next_u64(), elem = (uint32_t)next_u64();
        if (mcc::draw_hash(mcc::seed_mix(seed), mcc::hash_first(elem)) != mcc::hash_u32(seed ^ mcc::hash_u32(elem))) {
            std::printf("draw_hash differs at seed=%u elem=%u\n", seed, elem);
            return 2;
        }
    }
    // first products by addition: (x ^ k) * M1 == x * M1 + hash_delta(x & 3, k)
    for (long it = 0; it < 4000000; ++it) {
        const uint32_t x = (uint32_t)next_u64();
        for (uint32_t k = 0; k < 4; ++k)
            if ((x ^ k) * mcc::kHashMul1 != x * mcc::kHashMul1 + mcc::hash_delta(x & 3u, k)) {
                std::printf("hash_delta fails at %u^%u\n", x, k);
                return 2;
            }
    }
    // the per-row decision from the smallest magnitude agrees with the one from the key whenever it decides
    for (long it = 0; it < 2000000; ++it) {
        const float dn = log_uniform(1e-14, 1e14), ss = log_uniform(1e-30, 1e35);
        float g = (next_u64() & 3) ? log_uniform(1e-45, 1e3) : 0.0f;
        const int d = mcc::fast_division_from_min_abs(dn, ss, g);
        const bool ref = mcc::row_takes_fast_division(dn, ss, mcc::range_key(g));
        if ((d == 1 && !ref) || (d == -1 && ref && g != 0.0f) || (d == 0 && g != 0.0f)) {
            std::printf("fast_division_from_min_abs disagrees dn=%a ss=%a g=%a\n", dn, ss, g);
            return 2;
        }
    }
    // shared first hash step: (e + k) ^ ((e + k) >> 16) == (e ^ (e >> 16)) ^ k for e % 4 == 0
    for (long it = 0; it < 4000000; ++it) {
        const uint32_t e = (uint32_t)next_u64() & ~3u;
        for (uint32_t k = 0; k < 4; ++k)
            if (mcc::hash_first(e + k) != (mcc::hash_first(e) ^ k)) { std::printf("hash_first sharing fails at %u+%u\n", e, k); return 2; }
    }
    for (uint32_t e : {0xfffcu, 0x1fffcu, 0xfffffffcu, 0x7ffffffcu, 0u})
        for (uint32_t k = 0; k < 4; ++k)
            if (mcc::hash_first(e + k) != (mcc::hash_first(e) ^ k)) { std::printf("hash_first sharing fails at %u+%u\n", e, k); return 2; }
    std::printf("checked %ld ticks (%ld through the reciprocal division), %ld mismatches\n", checked, n_fast, mismatches);
    return mismatches == 0 ? 0 : 1;
}
