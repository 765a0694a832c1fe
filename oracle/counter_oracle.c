/*
 * counter_oracle.c -- CPU restatement of MotifCL's compact-counter update path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It exists to check the HIP
 * kernels.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may load it; nothing under motifcl_amd/ may include, link or call it.
 *
 * Each function restates one piece of the reference, cited as file:line
 * relative to the MotifCL source tree.  Every float operation is one IEEE-754
 * binary32 round-to-nearest-even operation: build with -ffp-contract=off and
 * without -ffast-math (x86-64 SSE has no excess precision; sqrtf and '/' are
 * correctly rounded).  The reference's own float semantics are implementation
 * defined (OpenCL C allows contraction); this file fixes them.
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   codec / packing  : reference known-answer vectors
 *                      (tests/test_vulkan_runtime_standalone.cpp:579-616,
 *                       tests/test_vulkan_backend.cpp:582-592), exhaustive
 *                      round trips.
 *   hash             : algebraic inverse built from modular inverses; the
 *                      constants are compared with the reference text when it
 *                      is present.
 *   decode / grad_x  : reference closed-form vectors
 *                      (tests/test_vulkan_runtime_standalone.cpp:1134-1160).
 *   row stats        : double-precision brute force + an independent numpy
 *                      lane/tree emulation.
 *   tick             : closed-form integer-tick cases, G == 0 fixed point,
 *                      saturation, invariants, unbiasedness.
 *   SR draw stream   : PARITY UNPINNED.  Which 24 bits decide a fractional
 *                      tick (seed ^ hash(elem), hashed again) is fixed only by
 *                      reading kernels/compact_counter.cl:127 and its GLSL twin
 *                      kernels/vulkan/counter_apply_update_fused_f32.comp:104;
 *                      the reference holds no executed vector for it.
 *
 * Conversions float->int that C leaves undefined are made explicit and
 * saturating (NaN -> 0); the reference leaves them undefined
 * (kernels/compact_counter.cl:131,134), so inputs that reach them
 * (|val| >= 2^31) are outside the parity contract.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_LANES 64 /* CC_RS_LSIZE, kernels/compact_counter.cl:58 */

/* ---- codec: kernels/compact_counter.cl:7-16 ------------------------------ */
void oracle_decode(int code, int C, int *t, int *c) {
    int lv = 2 * C - 1;
    *t = code / lv - 1;
    *c = code % lv - (C - 1);
}

int oracle_encode(int t, int c, int C) {
    int lv = 2 * C - 1;
    return (int)(uint8_t)((t + 1) * lv + (c + (C - 1)));
}

/* ---- hash RNG: kernels/compact_counter.cl:17-24 -------------------------- */
uint32_t oracle_hash_u32(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

float oracle_uniform01(uint32_t x) {
    return (float)(oracle_hash_u32(x) & 0x00ffffffu) * (1.0f / 16777216.0f);
}

/* ---- packing: kernels/compact_counter.cl:25-36 --------------------------- */
void oracle_unpack4(const uint8_t *p, int cc[4]) {
    int b0 = p[0], b1 = p[1], b2 = p[2];
    cc[0] = b0 & 0x3F;
    cc[1] = ((b0 >> 6) | (b1 << 2)) & 0x3F;
    cc[2] = ((b1 >> 4) | (b2 << 4)) & 0x3F;
    cc[3] = (b2 >> 2) & 0x3F;
}

void oracle_pack4(uint8_t *p, const int cc[4]) {
    p[0] = (uint8_t)((cc[0] & 0x3F) | ((cc[1] & 0x03) << 6));
    p[1] = (uint8_t)(((cc[1] >> 2) & 0x0F) | ((cc[2] & 0x0F) << 4));
    p[2] = (uint8_t)(((cc[2] >> 4) & 0x03) | ((cc[3] & 0x3F) << 2));
}

/* pack/unpack whole code arrays (helpers for tests and benches) */
void oracle_pack_codes(const uint8_t *codes, size_t n_codes, uint8_t *state) {
    for (size_t g = 0; g < n_codes / 4; ++g) {
        int cc[4] = {codes[4 * g], codes[4 * g + 1], codes[4 * g + 2], codes[4 * g + 3]};
        oracle_pack4(state + 3 * g, cc);
    }
}

void oracle_unpack_codes(const uint8_t *state, size_t n_codes, uint8_t *codes) {
    for (size_t g = 0; g < n_codes / 4; ++g) {
        int cc[4];
        oracle_unpack4(state + 3 * g, cc);
        for (int k = 0; k < 4; ++k) codes[4 * g + k] = (uint8_t)cc[k];
    }
}

/* ---- decode weight: kernels/compact_counter.cl:39-55 ---------------------- */
void oracle_decode_weight(const uint8_t *state, const float *scale, float *w,
                          int C, int in_features, int out_features) {
    int gpr = in_features / 4;
    for (int row = 0; row < out_features; ++row)
        for (int g = 0; g < gpr; ++g) {
            int cc[4];
            oracle_unpack4(state + ((size_t)row * gpr + g) * 3, cc);
            float s = scale[row];
            for (int k = 0; k < 4; ++k) {
                int t, c;
                oracle_decode(cc[k], C, &t, &c);
                w[(size_t)row * in_features + g * 4 + k] = s * (float)t;
            }
        }
}

/* ---- row stats, dense G: kernels/compact_counter.cl:59-100 ---------------- */
/* One row.  64 virtual lanes walk groups lid, lid+64, ...; then the binary
 * tree lg[lid] += lg[lid+s] for s = 32..1; lane 0 finishes.                  */
static void row_stats_one(const uint8_t *state_row, float scale_row, float *v_row,
                          const float *g_row, float *scale_new, float *denom,
                          int C, int in_features,
                          float lr_scale, float rms_beta, float rms_eps) {
    int gpr = in_features / 4;
    float lg[ORACLE_LANES], lgs[ORACLE_LANES];
    for (int lid = 0; lid < ORACLE_LANES; ++lid) {
        float g_sq = 0.0f, grad_s = 0.0f;
        for (int g = lid; g < gpr; g += ORACLE_LANES) {
            int cc[4];
            oracle_unpack4(state_row + (size_t)g * 3, cc);
            for (int k = 0; k < 4; ++k) {
                float gw = g_row[g * 4 + k];
                float sq = gw * gw;
                g_sq = g_sq + sq;
                int t, c;
                oracle_decode(cc[k], C, &t, &c);
                float gt = gw * (float)t;
                grad_s = grad_s + gt;
            }
        }
        lg[lid] = g_sq;
        lgs[lid] = grad_s;
    }
    for (int s = ORACLE_LANES / 2; s > 0; s >>= 1)
        for (int lid = 0; lid < s; ++lid) {
            lg[lid] = lg[lid] + lg[lid + s];
            lgs[lid] = lgs[lid] + lgs[lid + s];
        }
    float gsq = lg[0] / (float)in_features;
    float gs = lgs[0] / sqrtf((float)in_features);
    float a = rms_beta * *v_row;
    float b = (1.0f - rms_beta) * gsq;
    float vv = a + b;
    *v_row = vv;
    *denom = fmaxf(sqrtf(vv), rms_eps);
    float sn = scale_row - lr_scale * gs;
    /* clamp(x, 1e-5f, 10.0f) = fmin(fmax(x, lo), hi) (OpenCL C 6.12.4) */
    *scale_new = fminf(fmaxf(sn, 1e-5f), 10.0f);
}

void oracle_row_stats(const uint8_t *state, const float *scale, float *v,
                      const float *grad_w, float *scale_new, float *denom,
                      int C, int in_features, int out_features,
                      float lr_scale, float rms_beta, float rms_eps) {
    size_t row_bytes = (size_t)(in_features / 4) * 3;
#pragma omp parallel for schedule(static)
    for (int row = 0; row < out_features; ++row)
        row_stats_one(state + row * row_bytes, scale[row], &v[row],
                      grad_w + (size_t)row * in_features, &scale_new[row], &denom[row],
                      C, in_features, lr_scale, rms_beta, rms_eps);
}

/* saturating float -> int32, NaN -> 0 (the reference leaves this undefined) */
static int sat_i32(float x) {
    if (x != x) return 0;
    if (x >= 2147483648.0f) return INT32_MAX;
    if (x <= -2147483648.0f) return INT32_MIN;
    return (int)x;
}

/* ---- one SR tick: kernels/compact_counter.cl:118-136 ---------------------- */
int oracle_tick_code(int code, float gw, float s_old, float s_new, float dn,
                     int C, float lr, uint32_t seed, uint32_t elem) {
    float Cf = (float)C;
    int t, c;
    oracle_decode(code, C, &t, &c);
    float q = gw / dn;
    float k = Cf / s_new;
    float m = -lr * q;
    float tick = m * k;
    float ratio = s_old / s_new;
    float c_reb = (float)c * ratio;
    float val = c_reb + tick;
    float f = floorf(val);
    float rnd = oracle_uniform01(seed ^ oracle_hash_u32(elem));
    float frac = val - f;
    float ccv = f + (rnd < frac ? 1.0f : 0.0f);
    float carry = truncf(ccv / Cf);
    float cm = carry * Cf;
    float rem = ccv - cm;
    int64_t nt = (int64_t)t + (int64_t)sat_i32(carry);
    int ct = nt < -1 ? -1 : (nt > 1 ? 1 : (int)nt);
    if ((int64_t)ct != nt)
        rem = (ccv > 0.0f ? 1.0f : (ccv < 0.0f ? -1.0f : 0.0f)) * (Cf - 1.0f);
    int ri = sat_i32(rem);
    ri = ri < -(C - 1) ? -(C - 1) : (ri > C - 1 ? C - 1 : ri);
    return oracle_encode(ct, ri, C);
}

/* ---- apply, dense G: kernels/compact_counter.cl:104-139 ------------------- */
void oracle_apply_update(uint8_t *state, const float *scale, const float *scale_new,
                         const float *denom, const float *grad_w,
                         int C, int in_features, int out_features,
                         float lr, uint32_t seed) {
    int gpr = in_features / 4;
#pragma omp parallel for schedule(static)
    for (int row = 0; row < out_features; ++row)
        for (int g = 0; g < gpr; ++g) {
            uint8_t *p = state + ((size_t)row * gpr + g) * 3;
            int cc[4], nc[4];
            oracle_unpack4(p, cc);
            for (int k = 0; k < 4; ++k) {
                /* elem = row*in + g*4 + k as a 32-bit int, then (uint) */
                uint32_t elem = (uint32_t)row * (uint32_t)in_features + (uint32_t)(g * 4 + k);
                nc[k] = oracle_tick_code(cc[k], grad_w[(size_t)row * in_features + g * 4 + k],
                                         scale[row], scale_new[row], denom[row],
                                         C, lr, seed, elem);
            }
            oracle_pack4(p, nc);
        }
}

/* ---- host orchestration, dense G: src/nn/compact_counter.cpp:113-156 ------ */
/* pass 1 (stats) -> pass 2 (apply, old scale + new scale) -> commit scale.   */
int oracle_update_dense(uint8_t *state, float *scale, float *v, const float *grad_w,
                        int C, int in_features, int out_features,
                        float lr, float lr_scale, float rms_beta, float rms_eps,
                        uint32_t seed) {
    float *scale_new = (float *)malloc(sizeof(float) * (size_t)out_features);
    float *denom = (float *)malloc(sizeof(float) * (size_t)out_features);
    if (!scale_new || !denom) { free(scale_new); free(denom); return -1; }
    oracle_row_stats(state, scale, v, grad_w, scale_new, denom, C, in_features, out_features,
                     lr_scale, rms_beta, rms_eps);
    oracle_apply_update(state, scale, scale_new, denom, grad_w, C, in_features, out_features,
                        lr, seed);
    memcpy(scale, scale_new, sizeof(float) * (size_t)out_features); /* copy_f32, kernels/basic.cl:6-9 */
    free(scale_new);
    free(denom);
    return 0;
}

/* ---- weight gradient, sequential in r: kernels/compact_counter.cl:174-175 - */
/* gw[o,i] = (((0 + dY[0,o]*X[0,i]) + dY[1,o]*X[1,i]) + ...), fp32.  The loop
 * nest blocks rows and columns so that X streams through cache once per block
 * of 8 rows; every element still accumulates r = 0..N-1 in order.            */
void oracle_grad_w_seq(const float *grad_out, const float *x, float *grad_w,
                       int in_features, int out_features, int N) {
    enum { OB = 8, IB = 1024 }; /* rows and columns per block: 32 KiB of accumulators */
    int n_ob = (out_features + OB - 1) / OB;
    int n_ib = (in_features + IB - 1) / IB;
#pragma omp parallel for collapse(2) schedule(static)
    for (int ob = 0; ob < n_ob; ++ob)
        for (int ib = 0; ib < n_ib; ++ib) {
            int o0 = ob * OB, o1 = o0 + OB < out_features ? o0 + OB : out_features;
            int i0 = ib * IB, i1 = i0 + IB < in_features ? i0 + IB : in_features;
            for (int o = o0; o < o1; ++o)
                for (int i = i0; i < i1; ++i) grad_w[(size_t)o * in_features + i] = 0.0f;
            for (int r = 0; r < N; ++r) {
                const float *x_row = x + (size_t)r * in_features;
                for (int o = o0; o < o1; ++o) {
                    float go = grad_out[(size_t)r * out_features + o];
                    float *g_row = grad_w + (size_t)o * in_features;
                    for (int i = i0; i < i1; ++i) {
                        float p = go * x_row[i];
                        g_row[i] = g_row[i] + p;
                    }
                }
            }
        }
}

/* ---- fused update: src/nn/compact_counter.cpp:158-231 --------------------- */
/* The reference recomputes gw in both passes (kernels/compact_counter.cl:152-239);
 * both recomputations give the same fp32 value, so computing it once into a
 * caller-supplied buffer and running the dense passes is the same function.  */
int oracle_update_fused(uint8_t *state, float *scale, float *v,
                        const float *grad_out, const float *x, float *grad_w_tmp,
                        int C, int in_features, int out_features, int N,
                        float lr, float lr_scale, float rms_beta, float rms_eps,
                        uint32_t seed) {
    oracle_grad_w_seq(grad_out, x, grad_w_tmp, in_features, out_features, N);
    return oracle_update_dense(state, scale, v, grad_w_tmp, C, in_features, out_features,
                               lr, lr_scale, rms_beta, rms_eps, seed);
}

/* ---- forward: src/nn/compact_counter.cpp:287-293 (decode + x @ w^T) ------- */
void oracle_forward(const float *x, const uint8_t *state, const float *scale, float *y,
                    int C, int in_features, int out_features, int N) {
    float *w = (float *)malloc(sizeof(float) * (size_t)in_features * out_features);
    oracle_decode_weight(state, scale, w, C, in_features, out_features);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < N; ++r)
        for (int o = 0; o < out_features; ++o) {
            float acc = 0.0f;
            for (int i = 0; i < in_features; ++i) {
                float p = x[(size_t)r * in_features + i] * w[(size_t)o * in_features + i];
                acc = acc + p;
            }
            y[(size_t)r * out_features + o] = acc;
        }
    free(w);
}

/* ---- grad_x: kernels/compact_counter.cl:248-269 --------------------------- */
void oracle_backward_input(const float *grad_out, const uint8_t *state, const float *scale,
                           float *grad_x, int C, int in_features, int out_features, int N) {
    int gpr = in_features / 4;
    int lv = 2 * C - 1;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < N; ++r)
        for (int i = 0; i < in_features; ++i) {
            int g = i >> 2, k = i & 3;
            float acc = 0.0f;
            for (int o = 0; o < out_features; ++o) {
                int cc[4];
                oracle_unpack4(state + ((size_t)o * gpr + g) * 3, cc);
                int t = cc[k] / lv - 1;
                float a = grad_out[(size_t)r * out_features + o] * scale[o];
                float p = a * (float)t;
                acc = acc + p;
            }
            grad_x[(size_t)r * in_features + i] = acc;
        }
}

/* ---- layer init packing: src/nn/compact_counter.cpp:64-84 ----------------- */
/* Packs caller-supplied ternary values with c = 0; the reference draws them
 * from std::uniform_int_distribution, which the C++ standard does not pin.   */
void oracle_init_state(const int8_t *tern, uint8_t *state, float *scale, float *v,
                       int C, int in_features, int out_features, float init_gain) {
    int gpr = in_features / 4;
    for (int row = 0; row < out_features; ++row)
        for (int g = 0; g < gpr; ++g) {
            int code[4];
            for (int k = 0; k < 4; ++k)
                code[k] = oracle_encode(tern[(size_t)row * in_features + g * 4 + k], 0, C);
            oracle_pack4(state + ((size_t)row * gpr + g) * 3, code);
        }
    float s0 = init_gain * sqrtf(3.0f / (2.0f * (float)in_features));
    for (int row = 0; row < out_features; ++row) { scale[row] = s0; v[row] = 0.0f; }
}

/* ---- FP32 side optimizers: kernels/optim.cl:1-7 and :31-53, host part
 *      src/ops/optim.cpp:65-86 (bias corrections in binary32) ------------------ */
void oracle_sgd_update(float *param, const float *grad, size_t n, float lr) {
    for (size_t i = 0; i < n; ++i) {
        float d = lr * grad[i];
        param[i] = param[i] - d;
    }
}

void oracle_adam_update(float *param, const float *grad, float *m, float *v, size_t n,
                        float lr, float beta1, float beta2, float eps, int step,
                        float weight_decay) {
    float inv_bias1 = 1.0f / (1.0f - powf(beta1, (float)step));
    float inv_bias2 = 1.0f / (1.0f - powf(beta2, (float)step));
    for (size_t i = 0; i < n; ++i) {
        float g = grad[i];
        float a = beta1 * m[i];
        float b = (1.0f - beta1) * g;
        float mt = a + b;
        float c = beta2 * v[i];
        float d = (1.0f - beta2) * g;
        float e = d * g;
        float vt = c + e;
        m[i] = mt;
        v[i] = vt;
        float p = param[i];
        float num = mt * inv_bias1;
        float den = sqrtf(vt * inv_bias2) + eps;
        float update = num / den;
        float s1 = lr * update;
        float s2 = (lr * weight_decay) * p;
        float q = p - s1;
        param[i] = q - s2;
    }
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}
