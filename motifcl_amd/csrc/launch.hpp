// Internal launch functions behind the C ABI.  Arguments arrive validated.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <string>

namespace mcc {

// Failure reporting of the C ABI (capi.hip): stores the message mcc_last_error() returns.
int report_failure(int code, const std::string& message);
int report_hip_failure(hipError_t e, const char* what);

// The fused step behind mcc_compact_counter_apply_update_fused (capi.hip): validates, then
// enqueues; `workspace_nbytes` selects the two-kernel or the strip path.
int fused_update(void* stream, uint8_t* state, size_t state_nbytes, float* scale, size_t scale_nbytes, float* v,
                 size_t v_nbytes, const float* grad_out, size_t grad_out_nbytes, const float* x, size_t x_nbytes,
                 void* workspace, size_t workspace_nbytes, size_t C, size_t in_features, size_t out_features,
                 size_t batch, float lr, float lr_scale, float rms_beta, float rms_eps, uint32_t seed);

// One counter tensor of an update-only batch (device pointers).
struct UpdateTensor {
    uint8_t* state;
    float* scale;
    float* v;
    const float* grad_w;
    int in_features, out_features;
    int row_start;  // first row of this tensor in the launch's concatenated row space
    uint32_t seed;
    float lr;
    int first_row;  // rows 0.. of this descriptor are rows first_row.. of the tensor they belong to
                    // (a row band updated on its own): the draw hashes the tensor's element index
};
constexpr int kMaxUpdateBatch = 64;  // tensors per launch: the descriptors travel as kernel arguments

hipError_t launch_update_batch(hipStream_t stream, const UpdateTensor* tensors, size_t n, int C,
                               float lr_scale, float rms_beta, float rms_eps);

// state, scale, v and grad_w start at row `first_row` of the tensor (0: the whole tensor)
hipError_t launch_update_dense(hipStream_t stream, uint8_t* state, float* scale, float* v,
                               const float* grad_w, int C, int in_features, int out_features,
                               float lr, float lr_scale, float rms_beta, float rms_eps,
                               uint32_t seed, int first_row = 0);

// c[m,n] = a[k,m]^T . b[k,n].  Small outputs split the k range into plan.splits chunks whose
// partial products go to `slices` (plan.splits * m * n floats, may start at c) and are then summed
// in chunk order into c; gemm_tn_slices tells how many slices a shape needs (1: none).
struct GemmTnPlan {
    int tile;    // 128 or 64
    int splits;  // chunks of the k range
    int chunk;   // tokens per chunk, a multiple of 16
};
GemmTnPlan plan_gemm_tn(int k, int m, int n);
size_t gemm_tn_slices(int k, int m, int n);
// Bytes of hand-off words a contraction of this shape can use beyond its slices (0: none): shapes
// of more than two rounds of 256 x 256 tiles that are not whole rounds run as one launch of equal
// spans (gemm_tn_f32_wide.hip) when the caller lends them.
size_t gemm_tn_sync_nbytes(int k, int m, int n);
// mode: 0 = fp32 matrix instruction; 1 = both operands split into three bf16 terms, six bf16
// passes (gemm_tn_bf16x6.hip), where the shape allows it
// lda: floats between rows of a (0 = m); a wider lda contracts a column band of a [k, lda] matrix,
// cut up as `band_plan` says (the caller sized `slices` for it) instead of by the band's own shape
// sync_words: gemm_tn_sync_nbytes bytes of device memory, or null (the result is the same bits)
hipError_t launch_gemm_tn_f32(hipStream_t stream, const float* a, const float* b, float* c,
                              int k, int m, int n, float* slices, int mode = 0, int lda = 0,
                              const GemmTnPlan* band_plan = nullptr, int* sync_words = nullptr);
// 256 x 256-tile form of the contraction for whole tiles (gemm_tn_f32_wide.hip)
bool gemm_tn_wide_supports(const float* a, const float* b, int k, int m, int n, int chunk);
hipError_t launch_gemm_tn_wide(hipStream_t stream, const float* a, const float* b, float* out, int k, int m, int n,
                               int tiles_x, int tiles_y, int chunk, int splits);
// The whole contraction as one launch of at most kWideSpanWorkgroups workgroups with equal spans of
// the (tile, slab) sequence; `words` holds kWideSpanWorkgroups ints (cleared by the launch).
constexpr int kWideSpanWorkgroups = 256;
bool gemm_tn_wide_spans_apply(int k, int m, int n);
hipError_t launch_gemm_tn_wide_spans(hipStream_t stream, const float* a, const float* b, float* out, int k, int m,
                                     int n, int* words);
// Test aid (motifcl_amd_diag.h): polls a workgroup spends on a parked tile before it computes the
// tile alone (0xffffffff restores the default), and whether workgroups take up the tile begun by
// their neighbour before instead of after their own tiles, so that every wait runs out.
void set_gemm_tn_wide_spans_test_mode(unsigned polls, int start_first);

// One contraction of a grouped launch: out holds gemm_tn_slices(k, m, n) matrices of m*n floats,
// the result ends up in the first.
struct GemmTnJob {
    const float* a;  // [k, m]
    const float* b;  // [k, n]
    float* out;
    int k, m, n;
    int* sync_words = nullptr;  // as for launch_gemm_tn_f32
};
hipError_t launch_gemm_tn_group(hipStream_t stream, const GemmTnJob* jobs, size_t n);
// A list whose jobs all sit on whole 256 x 256 tiles and together hold at least two tiles per CU
// runs as ONE launch of equal spans of the list's (tile, slab) sequence: no token chunks, no slices
// (every out is m * n floats, the unchunked token-order sum).  `words` holds kWideSpanWorkgroups
// ints.  a, b and out must be 16-byte aligned.  ..._applies is a function of the shapes alone.
bool gemm_tn_spans_group_applies(const GemmTnJob* jobs, size_t n);
hipError_t launch_gemm_tn_wide_spans_group(hipStream_t stream, const GemmTnJob* jobs, size_t n, int* words);

bool gemm_tn_bf16x6_supports(const float* a, const float* b, int k, int m, int n, const GemmTnPlan& plan);
hipError_t launch_gemm_tn_bf16x6(hipStream_t stream, const float* a, const float* b, float* out,
                                 int k, int m, int n, const GemmTnPlan& plan);

// Fused step that keeps G in the contraction's accumulators (counter_fused_strip.hip).
// Shapes: in_features and out_features multiples of 128.  Large layers whose sides are multiples of
// 256 run on 256 x 256 tiles (same workspace, same bytes).
bool fused_strip_supports(size_t in_features, size_t out_features, size_t batch);
size_t fused_strip_workspace_nbytes(size_t in_features, size_t out_features, size_t batch);
// Polls one device-side wait of the strip step may spend before it gives up (0 restores the
// default, about four seconds; a test aid declared in motifcl_amd_diag.h).
unsigned fused_strip_spin_limit();
void set_fused_strip_spin_limit(unsigned spins);
// Tiles of the strip step: 0 chosen by shape (256 x 256 where their rounds keep the device busy,
// else 128 x 128), 1 wide whenever the shape allows, 2 never wide.  The result is the same bytes.
// grid_cap > 0 (a test aid) holds the wide kernel's grid to that many workgroups, which then park
// tiles on small layers too: such a launch needs fused_strip_workspace_nbytes_for_grid bytes.
// Both settings, like the spin limit, belong to the calling thread.
void set_fused_strip_wide_mode(int mode, int grid_cap);
size_t fused_strip_workspace_nbytes_for_grid(size_t in_features, size_t out_features, size_t batch, int grid_cap);
// A launch on another stream than the previous strip launch of this GPU is ordered behind it on
// the device (the two would compete for resident workgroups).  Strip launches that give up a wait
// raise a per-device count that fused_strip_take_failures reads and clears (the stream must have
// been synchronised).  workspace_nbytes: what the caller lent (checked against the parking slots
// the launch needs).
hipError_t launch_fused_strip(hipStream_t stream, uint8_t* state, float* scale, float* v,
                              const float* grad_out, const float* x, void* workspace, int C,
                              int in_features, int out_features, int tokens, float lr, float lr_scale,
                              float rms_beta, float rms_eps, uint32_t seed, unsigned spin_limit,
                              size_t workspace_nbytes);
hipError_t fused_strip_take_failures(int* count);

hipError_t launch_decode_weight(hipStream_t stream, const uint8_t* state, const float* scale,
                                float* weight, int C, int in_features, int out_features);

// y[batch,out] = x[batch,in] . W(state)^T
hipError_t launch_forward(hipStream_t stream, const float* x, const uint8_t* state,
                          const float* scale, float* y, int C, int batch, int in_features,
                          int out_features);

// grad_x[batch,in] = grad_out[batch,out] . W(state)
hipError_t launch_backward_input(hipStream_t stream, const float* grad_out, const uint8_t* state,
                                 const float* scale, float* grad_x, int C, int batch,
                                 int in_features, int out_features);

// param -= lr * grad; Adam with precomputed bias corrections (side_optim.hip)
hipError_t launch_sgd_update(hipStream_t stream, float* param, const float* grad, size_t n, float lr);
hipError_t launch_adam_update(hipStream_t stream, float* param, const float* grad, float* m, float* v,
                              size_t n, float lr, float beta1, float beta2, float eps, float inv_bias1,
                              float inv_bias2, float weight_decay);

}  // namespace mcc
