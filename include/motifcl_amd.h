/*
 * motifcl_amd.h -- C ABI of the MI355X (gfx950) compact-counter update library.
 *
 * Every entry point takes plain device pointers with their byte sizes, scalar
 * arguments and a HIP stream (hipStream_t passed as void*, NULL = the default
 * stream).  Work is enqueued on that stream and the call returns without
 * waiting.  Return value: 0 (MCC_OK) on success, a negative MCC_E_* code on
 * failure; mcc_last_error() then returns the message for the calling thread.
 * Validation failures never enqueue work and never throw -- the convention of
 * the reference's VulkanOpResult{success,error}
 * (include/motifcl/runtime/vulkan_backend.hpp:80-84).
 *
 * Data layout (kernels/compact_counter.cl:1-5):
 *   state  u8  [out, in/4, 3]  four 6-bit codes per 3 bytes, little-endian
 *                              24-bit word c0 | c1<<6 | c2<<12 | c3<<18
 *   scale  f32 [out]           per-row weight scale
 *   v      f32 [out]           per-row RMS second moment
 *   grad_w f32 [out, in]       dense weight gradient, row-major
 *   x      f32 [batch, in]     layer input, row-major
 *   grad_out f32 [batch, out]  upstream gradient, row-major
 */
#ifndef MOTIFCL_AMD_H
#define MOTIFCL_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MCC_OK 0
#define MCC_E_INVALID (-1) /* argument validation failed; nothing was enqueued */
#define MCC_E_RUNTIME (-2) /* a HIP call failed */

/* Message of the last failure on this thread ("" if none). */
const char* mcc_last_error(void);

/* Name and architecture of the current HIP device, e.g. "AMD Instinct MI355X (gfx950)".
 * Replaces VulkanOpResult::device_name. */
const char* mcc_device_name(void);

/*
 * Update-only step: the optimizer step for a supplied dense weight gradient.
 * Replaces CounterStateLinear::apply_update_seed
 * (src/nn/compact_counter.cpp:113-156: counter_row_stats_f32 ->
 * counter_apply_update_f32 -> copy_f32; kernels/compact_counter.cl:59-139).
 * Mutates state, scale and v in place.  Results are bit-identical to the
 * reference arithmetic evaluated in IEEE-754 binary32 without contraction.
 */
int mcc_compact_counter_apply_update_dense(
    void* stream,
    uint8_t* state, size_t state_nbytes,
    float* scale, size_t scale_nbytes,
    float* v, size_t v_nbytes,
    const float* grad_w, size_t grad_w_nbytes,
    size_t C, size_t in_features, size_t out_features,
    float lr, float lr_scale, float rms_beta, float rms_eps, uint32_t seed);

/*
 * Update-only step for a list of counter tensors in one call -- the optimizer step of a
 * whole model when every dense weight gradient is already in memory.  Each tensor gets
 * exactly the result of mcc_compact_counter_apply_update_dense with its own lr and seed;
 * C, lr_scale, rms_beta and rms_eps are shared.  The reference applies the update layer by
 * layer from the host (CounterStateLinear::apply_update_seed,
 * src/nn/compact_counter.cpp:113-156, once per module; the layer lists it walks are e.g.
 * tools/train_ternary15m.cpp:313-318); one launch over the rows of many tensors keeps the
 * memory system and the ALUs busy together, which a single small tensor cannot.
 * `tensors` is a host array; tensors must not alias each other.
 */
typedef struct mcc_counter_tensor {
    uint8_t* state;      size_t state_nbytes;
    float* scale;        size_t scale_nbytes;
    float* v;            size_t v_nbytes;
    const float* grad_w; size_t grad_w_nbytes;
    size_t in_features, out_features;
    float lr;
    uint32_t seed;
} mcc_counter_tensor;

int mcc_compact_counter_apply_update_dense_batched(
    void* stream, const mcc_counter_tensor* tensors, size_t n_tensors,
    size_t C, float lr_scale, float rms_beta, float rms_eps);

/*
 * Bytes of transient workspace mcc_compact_counter_apply_update_fused needs
 * for the given shape (0 on invalid dimensions): out*in*4 times the number of
 * token chunks the contraction is split into, plus 1 KiB of hand-off words
 * for large shapes that are not a whole number of rounds of 256 x 256 tiles
 * (their contraction then runs as one launch of equal spans; a workspace of
 * out*in*4 bytes without the words is accepted and gives the same bytes).
 * Layers with fewer than about 1024 output tiles split their tokens so that
 * the whole GPU works on them; the size depends on (in, out, batch) only.
 */
size_t mcc_compact_counter_fused_workspace_nbytes(size_t in_features, size_t out_features,
                                                  size_t batch);

/*
 * Bytes of the small workspace with which mcc_compact_counter_apply_update_fused
 * runs without a buffer of the size of the weight gradient, or 0 when the shape
 * has no way smaller than the full workspace (tiny layers).  Layers whose in and
 * out are multiples of 128 with in >= 768 take the accumulator-resident strip
 * path: 512 bytes of partial row sums per output row plus a few control words,
 * and, for layers of more than 256 tiles of 256 x 256, room to park 2 (in/256 - 1)
 * such tiles between the passes of the kernel's grid (24 MB for the largest layer
 * of a 7B model instead of 180 MB).  Every other shape
 * is updated band by band of an eighth of its output rows: the workspace holds
 * one band's gradient.  No counterpart in the reference, whose fused kernels
 * recompute the gradient instead of holding it.
 */
size_t mcc_compact_counter_fused_strip_workspace_nbytes(size_t in_features, size_t out_features,
                                                        size_t batch);

/*
 * Waits for `stream` and reports whether every strip-path step of this process
 * on the current GPU since the last call completed: MCC_OK, or MCC_E_RUNTIME
 * when a step gave up a wait between tiles.  Such a step leaves whole strips
 * (128 or 256 rows) of its tensor without their update -- state, scale and v of those rows
 * are untouched, no strip is half-updated -- and the report clears the count.
 * The count lives in the library, per GPU, so it survives other layers' steps
 * through the same workspace; the workspace and shape arguments are not looked
 * at (kept for callers written against the first form of this call).  Always
 * MCC_OK for steps on the full workspace or band by band.  No counterpart in
 * the reference.
 */
int mcc_compact_counter_fused_check(void* stream, const void* workspace, size_t workspace_nbytes,
                                    size_t in_features, size_t out_features, size_t batch);

/*
 * Fused step: weight-gradient contraction grad_w = grad_out^T . x on the fp32
 * matrix cores followed by the counter update.
 * Replaces run_vulkan_compact_counter_apply_update_fused
 * (include/motifcl/runtime/vulkan_backend.hpp:733-749,
 *  src/runtime/vulkan_backend.cpp:8475-8578) and the OpenCL twin in
 * CounterStateLinear::apply_update_backward (src/nn/compact_counter.cpp:158-231).
 * The reference's scale_new/denom scratch buffers are not needed; instead the
 * caller lends `workspace`, whose size selects how the step runs:
 *   - >= mcc_compact_counter_fused_workspace_nbytes (one f32[out,in] slice
 *     per token chunk of the contraction; large layers have one chunk):
 *     contraction into the workspace, then the update kernel.  After the call
 *     the first out*in floats of the workspace hold grad_w.  The fastest way.
 *   - >= mcc_compact_counter_fused_strip_workspace_nbytes but smaller than
 *     the above: no weight-sized buffer exists at any time, which is the
 *     property tests/test_memory_truth_gate.cpp:109-113 of the reference asks
 *     for.  Any lr_scale.  On the strip path (see the size query) the update is
 *     applied from the contraction's accumulators; x must be 16-byte aligned;
 *     tiles of one row strip wait for each other on the device, so two such
 *     steps must not run side by side on one GPU: a call on another stream than
 *     the previous strip call is ordered behind it on the device (the stream
 *     waits for an event recorded after that call; the host does not wait),
 *     every wait is bounded, and mcc_compact_counter_fused_check reports a
 *     wait that was given up.  On a stream under graph capture no such order
 *     is added: do not replay two such graphs side by side.
 * The ways produce identical bytes whenever none of them splits the tokens into
 * chunks, i.e. for fewer than 512 tokens or layers of at least 1024 tiles of
 * 128 x 128 (mcc_compact_counter_fused_workspace_nbytes == out*in*4); where
 * one does, its gradient is the sum of chunk sums and they differ by that
 * rounding (a few counters in 10^5 flip differently).
 * grad_w differs from the reference's
 * sequential fp32 sum only by summation order (relative error <= 1e-4 of the
 * row norm); given that grad_w the counter arithmetic is the same as in the
 * dense entry point.
 */
int mcc_compact_counter_apply_update_fused(
    void* stream,
    uint8_t* state, size_t state_nbytes,
    float* scale, size_t scale_nbytes,
    float* v, size_t v_nbytes,
    const float* grad_out, size_t grad_out_nbytes,
    const float* x, size_t x_nbytes,
    void* workspace, size_t workspace_nbytes,
    size_t C, size_t in_features, size_t out_features, size_t batch,
    float lr, float lr_scale, float rms_beta, float rms_eps, uint32_t seed);

/*
 * The fused step with the workspace inside the library: the same step as
 * mcc_compact_counter_apply_update_fused, for callers that cannot allocate device
 * memory -- code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  The workspace is a
 * static device array of MCC_NOALLOC_WORKSPACE_NBYTES bytes that every GPU the
 * library runs on holds from its first use there until the process ends; the
 * call itself allocates nothing (no hipMalloc / hipFree, no stream-ordered
 * allocation; with mcc_profiler_enable(1) the profiler may still create events).
 * The step runs as mcc_compact_counter_apply_update_fused would with
 *   - mcc_compact_counter_fused_workspace_nbytes(in, out, batch) bytes when that
 *     fits the array (identical bytes to that call), else
 *   - mcc_compact_counter_fused_strip_workspace_nbytes(in, out, batch) bytes when
 *     that fits, else
 *   - it fails with MCC_E_INVALID and a message that names both sizes.
 * All calls on one GPU share that GPU's array, which keeps the last call's
 * contents: two calls that overlap in time on one GPU (different streams) race.
 * The first call on a GPU looks up the array's address there (and, for a shape
 * on the strip path, creates the event that orders strip steps of different
 * streams): make that first call outside graph capture; later calls may be
 * captured and replayed.  A step that took the strip path reports a given-up
 * wait through mcc_compact_counter_fused_check, like the lent-workspace call
 * (its workspace arguments are not looked at: pass a null pointer and 0).
 * Arguments and validation are those of mcc_compact_counter_apply_update_fused
 * without the workspace.
 */
#define MCC_NOALLOC_WORKSPACE_NBYTES ((size_t)32 << 20)
int mcc_compact_counter_apply_update_fused_static(
    void* stream,
    uint8_t* state, size_t state_nbytes,
    float* scale, size_t scale_nbytes,
    float* v, size_t v_nbytes,
    const float* grad_out, size_t grad_out_nbytes,
    const float* x, size_t x_nbytes,
    size_t C, size_t in_features, size_t out_features, size_t batch,
    float lr, float lr_scale, float rms_beta, float rms_eps, uint32_t seed);

/*
 * The fused step for a list of tensors in a handful of launches: one grouped
 * contraction per tile size, one launch that adds the token-chunk slices, and
 * the batched update.  For models made of small layers (the 288- and 768-wide
 * linears of the 15M-parameter model) the per-tensor entry point is bound by
 * its three launches per tensor; this one costs about five launches for all of
 * them.  It has no single counterpart in the reference: it stands for the
 * per-layer calls of apply_update_backward (src/nn/compact_counter.cpp:158-231)
 * of a caller that keeps every layer's grad_out and x alive until the end of
 * its backward pass, which is equivalent because no layer's update reads
 * another layer's state.  state, scale and v come out bit-identical to calling
 * mcc_compact_counter_apply_update_fused per tensor with a full workspace --
 * except for a list that runs as equal spans: when every layer's sides are
 * multiples of 256, every token count a multiple of 16 and the list holds at
 * least 512 tiles of 256 x 256 (the 110M-shaped model: 1296), the contractions
 * of the whole list are one launch in which every workgroup gets an equal share
 * of the list's tiles and tokens, with no token chunks: each gradient is then
 * the unchunked token-order sum (the reference's order up to pairing), state,
 * scale and v are exact for that gradient, and they equal the per-tensor call's
 * wherever that call does not split the tokens into chunks and differ from it
 * by the rounding of its chunk sums elsewhere (counter-flip fraction ~1e-6).
 * Such a list needs 16-byte aligned grad_out and x.
 * Likewise a list of small layers whose tiles together number 512 or more (the
 * 15M-shaped model: 42 layers) is cut into token chunks per list, fewer than a
 * layer's own call would use: its gradients are the sums over those chunks,
 * state, scale and v exact for them, with the same relation to the per-tensor
 * call.
 * `workspace` (256-byte aligned) holds
 * mcc_compact_counter_fused_batched_workspace_nbytes(tensors, n) bytes: the
 * per-tensor workspaces, each rounded up to 256 bytes, one after the other (as
 * equal spans: out * in floats per tensor plus 1 KiB; the size depends on the
 * calling thread's contraction mode, so query it in the mode the call runs in).
 * Under MCC_CONTRACTION_BF16X6 the tensors are processed one by one.
 */
typedef struct mcc_fused_tensor {
    uint8_t* state;        size_t state_nbytes;
    float* scale;          size_t scale_nbytes;
    float* v;              size_t v_nbytes;
    const float* grad_out; size_t grad_out_nbytes;  /* [batch, out_features] */
    const float* x;        size_t x_nbytes;         /* [batch, in_features] */
    size_t in_features, out_features, batch;
    float lr;
    uint32_t seed;
} mcc_fused_tensor;
size_t mcc_compact_counter_fused_batched_workspace_nbytes(const mcc_fused_tensor* tensors, size_t n_tensors);
int mcc_compact_counter_apply_update_fused_batched(
    void* stream, const mcc_fused_tensor* tensors, size_t n_tensors,
    void* workspace, size_t workspace_nbytes,
    size_t C, float lr_scale, float rms_beta, float rms_eps);

/*
 * How the weight-gradient contraction (inside the two-kernel fused step and in
 * mcc_matmul_transpose_a_f32) multiplies.  A setting of the calling thread: it
 * governs the calls that thread makes afterwards and no other thread's.  No
 * counterpart in the reference.
 *   MCC_CONTRACTION_FP32    the fp32 matrix instruction (default)
 *   MCC_CONTRACTION_BF16X6  both operands split into three bf16 terms, six bf16
 *                           matrix passes per product: per-product error of one
 *                           binary32 rounding, as the fp32 instruction, at about
 *                           1.2 x its speed on 7B-sized layers (72 against 88 ms
 *                           for a seven-tensor layer step at 32768 tokens).  Used
 *                           for whole 128 x 128 tiles and
 *                           token counts that are multiples of 32; other shapes
 *                           silently use the fp32 instruction.  The two modes give
 *                           gradients that differ in the last bits, so counters
 *                           whose tick lands within that distance of a rounding
 *                           boundary may come out differently.
 */
#define MCC_CONTRACTION_FP32 0
#define MCC_CONTRACTION_BF16X6 1
int mcc_set_contraction_mode(int mode);
int mcc_get_contraction_mode(void);

/*
 * c[m,n] = a[k,m]^T . b[k,n], fp32, row-major.
 * Replaces matmul_transpose_a (include/motifcl/ops/matmul.hpp:8,
 * src/ops/matmul.cpp:1416-1418), the producer of the dense weight gradient
 * (grad_w = matmul_transpose_a(grad_out, x), tests/test_memory_truth_gate.cpp:49).
 */
int mcc_matmul_transpose_a_f32(
    void* stream,
    const float* a, size_t a_nbytes,
    const float* b, size_t b_nbytes,
    float* c, size_t c_nbytes,
    size_t k, size_t m, size_t n);

/*
 * weight[out,in] = scale[row] * t(state).
 * Replaces run_vulkan_compact_counter_decode_weight
 * (include/motifcl/runtime/vulkan_backend.hpp:713-719,
 *  src/runtime/vulkan_backend.cpp:8603-8660; kernels/compact_counter.cl:39-55).
 */
int mcc_compact_counter_decode_weight(
    void* stream,
    const uint8_t* state, size_t state_nbytes,
    const float* scale, size_t scale_nbytes,
    float* weight, size_t weight_nbytes,
    size_t in_features, size_t out_features, size_t C);

/*
 * out[batch,out] = x[batch,in] . W(state)^T with the ternary weights decoded
 * from the packed state inside the contraction (no dense weight buffer).
 * Runs on the bf16 matrix cores with every product exact: the ternary weight
 * is exact in bf16 and each activation is split into three bf16 terms whose sum
 * is the activation, so the result has fp32 accuracy (the terms of an fp32
 * contraction, summed in another order).  Activations must be finite and
 * below 3.38e38 in magnitude (the largest bf16); terms below 2^-110 lose
 * their low bits.
 * Replaces run_vulkan_compact_counter_forward_u8
 * (include/motifcl/runtime/vulkan_backend.hpp:722-730,
 *  src/runtime/vulkan_backend.cpp:8662-8725).
 */
int mcc_compact_counter_forward_u8(
    void* stream,
    const float* x, size_t x_nbytes,
    const uint8_t* state, size_t state_nbytes,
    const float* scale, size_t scale_nbytes,
    float* out, size_t out_nbytes,
    size_t batch, size_t in_features, size_t out_features, size_t C);

/*
 * grad_x[batch,in] = grad_out[batch,out] . W(state), decoded in-kernel; grad_out
 * is multiplied by the row scale first, as the reference does, then split as in
 * the forward product (same accuracy, same requirement of finite inputs).
 * Replaces run_vulkan_compact_counter_backward_input_u8
 * (include/motifcl/runtime/vulkan_backend.hpp:750-758,
 *  src/runtime/vulkan_backend.cpp:8727-8803; kernels/compact_counter.cl:248-269).
 */
int mcc_compact_counter_backward_input_u8(
    void* stream,
    const uint8_t* state, size_t state_nbytes,
    const float* scale, size_t scale_nbytes,
    const float* grad_out, size_t grad_out_nbytes,
    float* grad_x, size_t grad_x_nbytes,
    size_t batch, size_t in_features, size_t out_features, size_t C);

/*
 * FP32 side optimizers for the non-counter tensors of a counter model
 * (embedding, norm gains).  Replace sgd_update and adam_update_fast
 * (include/motifcl/ops/optim.hpp, src/ops/optim.cpp:17-86; kernels
 * kernels/optim.cl:1-7,31-53).  `n` counts elements; all buffers hold n floats.
 * Adam: step >= 1; the bias corrections 1/(1 - beta^step) are computed on the
 * host in binary32 as the reference does (src/ops/optim.cpp:70-71).
 */
int mcc_sgd_update_f32(void* stream, float* param, size_t param_nbytes, const float* grad,
                       size_t grad_nbytes, size_t n, float lr);
int mcc_adam_update_f32(void* stream, float* param, size_t param_nbytes, const float* grad,
                        size_t grad_nbytes, float* m, size_t m_nbytes, float* v, size_t v_nbytes,
                        size_t n, float lr, float beta1, float beta2, float eps, int step,
                        float weight_decay);

/*
 * Device-resident storage.  Replaces the pooled VulkanRuntime::create_buffer /
 * Storage allocator (src/runtime/vulkan_backend.cpp:4663-4719,6462-6510;
 * src/tensor/storage.cpp:35-79): freed blocks are kept in power-of-two buckets
 * and reused; mcc_device_pool_clear returns them to the driver.  The byte
 * counters mirror device_bytes_current/peak (src/runtime/buffer.cpp:16-30).
 */
int mcc_device_alloc(void** ptr, size_t nbytes);
int mcc_device_free(void* ptr);
int mcc_device_pool_clear(void);
size_t mcc_device_bytes_current(void);
size_t mcc_device_bytes_peak(void);
void mcc_device_bytes_reset_peak(void);
int mcc_memcpy_h2d(void* stream, void* dst, const void* src, size_t nbytes);
int mcc_memcpy_d2h(void* stream, void* dst, const void* src, size_t nbytes);
int mcc_memset_zero(void* stream, void* dst, size_t nbytes);
/* Waits for everything enqueued on `stream` (Backend::finish,
 * src/runtime/backend.cpp:328-331). */
int mcc_stream_synchronize(void* stream);

/*
 * Per-kernel GPU timing.  While enabled, each kernel launched through this ABI is
 * bracketed by HIP events on its launch stream; mcc_profiler_query waits for them and
 * returns the summed duration and launch count of one kernel family:
 * "gemm_tn_f32", "counter_update", "counter_decode_weight", "counter_forward",
 * "counter_backward_input".  Replaces Profiler (src/runtime/profiler.cpp) and
 * VulkanRuntime::set_gpu_timing_enabled / last_gpu_time_us
 * (include/motifcl/runtime/vulkan_backend.hpp:181-185).
 */
void mcc_profiler_enable(int on);
void mcc_profiler_reset(void);
int mcc_profiler_query(const char* kernel_name, double* total_ms, uint64_t* launches);

#ifdef __cplusplus
}
#endif

#endif /* MOTIFCL_AMD_H */
