// C ABI of the library: argument validation, error reporting and device
// storage.  Validation mirrors the reference's Vulkan host wrappers
// (src/runtime/vulkan_backend.cpp:8497-8521, 8603-8650, 8662-8712, 8727-8786):
// failures are reported, never thrown, and enqueue nothing.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <limits>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/motifcl_amd.h"
#include "launch.hpp"

namespace {
thread_local std::string g_error;
}  // namespace

namespace mcc {

// Records the calling thread's failure message and returns `code` (shared with diag.hip).
int report_failure(int code, const std::string& message) {
    g_error = message;
    return code;
}

int report_hip_failure(hipError_t e, const char* what) {
    return report_failure(MCC_E_RUNTIME, std::string(what) + ": " + hipGetErrorString(e));
}

}  // namespace mcc

namespace {

int fail(int code, const std::string& message) { return mcc::report_failure(code, message); }

int hip_fail(hipError_t e, const char* what) { return mcc::report_hip_failure(e, what); }

constexpr size_t kIntMax = static_cast<size_t>(std::numeric_limits<int>::max());

// 0: weight-gradient contraction on the fp32 matrix instruction; 1: split-bf16 form where the
// shape allows it
// the calling thread's setting: other threads' calls are not affected and no call sees it change
thread_local int g_contraction_mode = 0;

// Shared shape/codec checks.  `what` names the operation in messages.
bool check_codec(const char* what, size_t C, size_t in_features, size_t out_features) {
    if (in_features == 0 || out_features == 0) {
        g_error = std::string(what) + " requires non-zero dimensions";
        return false;
    }
    if (in_features % 4 != 0) {
        g_error = std::string(what) + " requires in_features divisible by 4";
        return false;
    }
    if (C == 0 || 3 * (2 * C - 1) > 64) {
        g_error = std::string(what) + " C is out of 6-bit range";
        return false;
    }
    if (in_features > kIntMax || out_features > kIntMax ||
        out_features > kIntMax / in_features) {
        g_error = std::string(what) + " dimensions exceed the 32-bit element index of the state encoding";
        return false;
    }
    return true;
}

// True when two entries of `states` are the same pointer: descriptors that share a state would be
// updated by several workgroups of one launch at once.
bool has_duplicate(std::vector<const void*> states) {
    std::sort(states.begin(), states.end());
    return std::adjacent_find(states.begin(), states.end()) != states.end();
}

// ---- pooled device storage -------------------------------------------------
struct Pool {
    std::mutex mu;
    std::map<size_t, std::vector<void*>> free_blocks;   // bucket bytes -> cached blocks
    std::unordered_map<void*, size_t> live;             // block -> bucket bytes
    size_t cached_bytes = 0;
};
Pool& pool() {
    static Pool p;
    return p;
}
std::atomic<size_t> g_bytes_current{0};
std::atomic<size_t> g_bytes_peak{0};
constexpr size_t kPoolMaxCachedBytes = size_t(2) << 30;  // cap as in vulkan_backend.cpp:6462-6510

size_t bucket_of(size_t nbytes) {
    size_t b = 256;
    while (b < nbytes) b <<= 1;
    return b;
}

__global__ void fill_zero_kernel(uint8_t* dst, size_t nbytes) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nbytes; i += stride) dst[i] = 0;
}

void track_alloc(size_t n) {
    const size_t cur = g_bytes_current.fetch_add(n) + n;
    size_t prev = g_bytes_peak.load();
    while (cur > prev && !g_bytes_peak.compare_exchange_weak(prev, cur)) {
    }
}

// ---- per-kernel GPU timing ---------------------------------------------------
// When enabled, every kernel launch made through this ABI is bracketed by two HIP
// events on the launch stream (the reference's counterpart: Profiler /
// VulkanRuntime::set_gpu_timing_enabled, include/motifcl/runtime/vulkan_backend.hpp:181-185).
struct TimedLaunch {
    const char* name;
    hipEvent_t start, stop;
};
struct Profiler {
    std::mutex mu;
    bool enabled = false;
    std::vector<TimedLaunch> records;
    std::vector<hipEvent_t> spare;
    hipEvent_t take() {
        if (!spare.empty()) {
            hipEvent_t e = spare.back();
            spare.pop_back();
            return e;
        }
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess) return nullptr;
        return e;
    }
};
Profiler& profiler() {
    static Profiler p;
    return p;
}

class ScopedKernelTimer {
public:
    ScopedKernelTimer(const char* name, hipStream_t stream) : stream_(stream) {
        Profiler& p = profiler();
        std::lock_guard<std::mutex> lock(p.mu);
        if (!p.enabled) return;
        rec_.name = name;
        rec_.start = p.take();
        rec_.stop = p.take();
        active_ = rec_.start && rec_.stop;
        if (active_) (void)hipEventRecord(rec_.start, stream_);
    }
    ~ScopedKernelTimer() {
        if (!active_) return;
        (void)hipEventRecord(rec_.stop, stream_);
        Profiler& p = profiler();
        std::lock_guard<std::mutex> lock(p.mu);
        p.records.push_back(rec_);
    }
private:
    hipStream_t stream_;
    TimedLaunch rec_{};
    bool active_ = false;
};

}  // namespace

extern "C" {

const char* mcc_last_error(void) { return g_error.c_str(); }

const char* mcc_device_name(void) {
    static thread_local std::string name;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        name = "";
        return name.c_str();
    }
    name = std::string(prop.name) + " (" + prop.gcnArchName + ")";
    return name.c_str();
}

// Validation shared by the single and the batched update-only entry points; fills `out`.
static int check_update_tensor(const mcc_counter_tensor& t, size_t C, float lr_scale, float rms_beta,
                               float rms_eps, mcc::UpdateTensor* out) {
    const char* what = "compact-counter update";
    if (!check_codec(what, C, t.in_features, t.out_features)) return MCC_E_INVALID;
    if (!std::isfinite(t.lr)) return fail(MCC_E_INVALID, "compact-counter update requires finite lr");
    if (!std::isfinite(lr_scale)) return fail(MCC_E_INVALID, "compact-counter update requires finite lr_scale");
    if (!std::isfinite(rms_beta)) return fail(MCC_E_INVALID, "compact-counter update requires finite rms_beta");
    if (!std::isfinite(rms_eps) || rms_eps < 0.0f)
        return fail(MCC_E_INVALID, "compact-counter update requires non-negative finite rms_eps");
    if (!t.state || !t.scale || !t.v || !t.grad_w)
        return fail(MCC_E_INVALID, "compact-counter update received a null buffer");
    const size_t n_groups = t.out_features * (t.in_features / 4);
    if (t.state_nbytes < n_groups * 3) return fail(MCC_E_INVALID, "compact-counter update state buffer is too small");
    if (t.scale_nbytes < t.out_features * sizeof(float) || t.v_nbytes < t.out_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter update per-row buffer is too small");
    if (t.grad_w_nbytes < t.out_features * t.in_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter update gradient buffer is too small");
    if (reinterpret_cast<uintptr_t>(t.grad_w) % alignof(float) || reinterpret_cast<uintptr_t>(t.scale) % alignof(float) ||
        reinterpret_cast<uintptr_t>(t.v) % alignof(float))
        return fail(MCC_E_INVALID, "compact-counter update float buffers must be 4-byte aligned");
    out->state = t.state; out->scale = t.scale; out->v = t.v; out->grad_w = t.grad_w;
    out->in_features = (int)t.in_features; out->out_features = (int)t.out_features;
    out->row_start = 0; out->seed = t.seed; out->lr = t.lr; out->first_row = 0;
    return MCC_OK;
}

int mcc_compact_counter_apply_update_dense(void* stream, uint8_t* state, size_t state_nbytes,
                                           float* scale, size_t scale_nbytes, float* v,
                                           size_t v_nbytes, const float* grad_w,
                                           size_t grad_w_nbytes, size_t C, size_t in_features,
                                           size_t out_features, float lr, float lr_scale,
                                           float rms_beta, float rms_eps, uint32_t seed) {
    const mcc_counter_tensor t = {state, state_nbytes, scale, scale_nbytes, v, v_nbytes, grad_w, grad_w_nbytes,
                                  in_features, out_features, lr, seed};
    return mcc_compact_counter_apply_update_dense_batched(stream, &t, 1, C, lr_scale, rms_beta, rms_eps);
}

int mcc_compact_counter_apply_update_dense_batched(void* stream, const mcc_counter_tensor* tensors,
                                                   size_t n_tensors, size_t C, float lr_scale,
                                                   float rms_beta, float rms_eps) {
    if (n_tensors == 0) return MCC_OK;
    if (!tensors) return fail(MCC_E_INVALID, "compact-counter update received a null tensor list");
    std::vector<mcc::UpdateTensor> dev(n_tensors);
    for (size_t i = 0; i < n_tensors; ++i) {
        const int rc = check_update_tensor(tensors[i], C, lr_scale, rms_beta, rms_eps, &dev[i]);
        if (rc != MCC_OK) {
            if (n_tensors > 1) g_error = "tensor " + std::to_string(i) + ": " + g_error;
            return rc;
        }
    }
    if (n_tensors > 1) {
        std::vector<const void*> states(n_tensors);
        for (size_t i = 0; i < n_tensors; ++i) states[i] = tensors[i].state;
        if (has_duplicate(std::move(states)))
            return fail(MCC_E_INVALID, "compact-counter update received the same state twice in one list");
    }
    hipError_t e;
    {
        ScopedKernelTimer timer("counter_update", static_cast<hipStream_t>(stream));
        e = mcc::launch_update_batch(static_cast<hipStream_t>(stream), dev.data(), n_tensors, (int)C, lr_scale,
                                     rms_beta, rms_eps);
    }
    if (e != hipSuccess) return hip_fail(e, "compact-counter update launch failed");
    return MCC_OK;
}

size_t mcc_compact_counter_fused_workspace_nbytes(size_t in_features, size_t out_features,
                                                  size_t batch) {
    if (in_features == 0 || out_features == 0 || batch == 0) return 0;
    if (in_features > kIntMax || out_features > kIntMax || batch > kIntMax) return 0;
    // one f32[out,in] slice per token chunk of the contraction (one chunk for large layers)
    const size_t slices = mcc::gemm_tn_slices((int)batch, (int)out_features, (int)in_features);
    if (out_features > std::numeric_limits<size_t>::max() / sizeof(float) / in_features / slices) return 0;
    // ... and the hand-off words of a contraction that runs as one launch of equal spans
    return slices * out_features * in_features * sizeof(float) +
           mcc::gemm_tn_sync_nbytes((int)batch, (int)out_features, (int)in_features);
}

}  // extern "C"

namespace {

// How the fused step runs on a workspace smaller than the full one:
//   strip   the accumulator-resident kernel (in/out multiples of 128, rows of at least 768 weights:
//           its 512 bytes of partial sums per output row are then at most a sixth of the row);
//   banded  the two-kernel path applied to bands of `band_rows` output rows, one after the other
//           through a workspace of an eighth of the weight gradient -- any shape, slower (the bands
//           are small contractions), for the layers too small or too oddly shaped for the strips.
struct SmallPlan {
    enum Kind { kNone, kStrip, kBanded } kind = kNone;
    size_t nbytes = 0;
    int band_rows = 0;
    mcc::GemmTnPlan band_plan{};
};

SmallPlan small_workspace_plan(size_t in_features, size_t out_features, size_t batch) {
    SmallPlan p;
    if (in_features == 0 || out_features == 0 || batch == 0 || in_features % 4 != 0) return p;
    if (in_features > kIntMax || out_features > kIntMax || batch > kIntMax) return p;
    if (in_features >= 768 && mcc::fused_strip_supports(in_features, out_features, batch)) {
        p.kind = SmallPlan::kStrip;
        p.nbytes = mcc::fused_strip_workspace_nbytes(in_features, out_features, batch);
        return p;
    }
    // rows x token chunks the workspace may hold: an eighth of the gradient, so that a caller whose
    // allocator rounds up to a power of two still stays below a quarter
    const size_t budget_rows = out_features / 8 > 0 ? out_features / 8 : 1;
    size_t rows = budget_rows >= 8 ? budget_rows / 8 * 8 : budget_rows;
    mcc::GemmTnPlan plan = mcc::plan_gemm_tn((int)batch, (int)rows, (int)in_features);
    if ((size_t)plan.splits * rows > budget_rows) {
        // fewer token chunks than the band would take on its own
        const size_t splits = budget_rows / rows > 0 ? budget_rows / rows : 1;
        int chunk = (int)((batch + splits - 1) / splits);
        chunk = (chunk + 15) / 16 * 16;
        plan.chunk = chunk;
        plan.splits = (int)((batch + chunk - 1) / chunk);
    }
    p.kind = SmallPlan::kBanded;
    p.band_rows = (int)rows;
    p.band_plan = plan;
    p.nbytes = ((size_t)plan.splits * rows * in_features * sizeof(float) + 255) / 256 * 256;
    return p;
}

}  // namespace

extern "C" {

size_t mcc_compact_counter_fused_strip_workspace_nbytes(size_t in_features, size_t out_features,
                                                        size_t batch) {
    const SmallPlan p = small_workspace_plan(in_features, out_features, batch);
    const size_t full = mcc_compact_counter_fused_workspace_nbytes(in_features, out_features, batch);
    return p.kind != SmallPlan::kNone && p.nbytes < full ? p.nbytes : 0;
}

int mcc_compact_counter_fused_check(void* stream, const void* workspace, size_t workspace_nbytes,
                                    size_t in_features, size_t out_features, size_t batch) {
    (void)workspace; (void)workspace_nbytes; (void)in_features; (void)out_features; (void)batch;
    const hipError_t es = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (es != hipSuccess) return hip_fail(es, "compact-counter fused check: stream synchronize failed");
    int failures = 0;
    const hipError_t ec = mcc::fused_strip_take_failures(&failures);
    if (ec != hipSuccess) return hip_fail(ec, "compact-counter fused check: status read failed");
    if (failures != 0)
        return fail(MCC_E_RUNTIME,
                    "compact-counter fused strip update gave up waiting for a neighbouring tile in " +
                        std::to_string(failures) + " launch(es) on this GPU since the last check; in such a launch "
                        "whole strips of the tensor (128 or 256 rows) are left without their update (no strip is half-updated)");
    return MCC_OK;
}

}  // extern "C"

// Validation and launches of the fused step, shared by mcc_compact_counter_apply_update_fused and
// the entry point that brings its own workspace (noalloc.hip).  Allocates nothing on the device.
int mcc::fused_update(void* stream, uint8_t* state, size_t state_nbytes, float* scale, size_t scale_nbytes, float* v,
                      size_t v_nbytes, const float* grad_out, size_t grad_out_nbytes, const float* x, size_t x_nbytes,
                      void* workspace, size_t workspace_nbytes, size_t C, size_t in_features, size_t out_features,
                      size_t batch, float lr, float lr_scale, float rms_beta, float rms_eps, uint32_t seed) {
    const char* what = "compact-counter fused update";
    if (batch == 0) return fail(MCC_E_INVALID, "compact-counter fused update requires non-zero dimensions");
    if (!check_codec(what, C, in_features, out_features)) return MCC_E_INVALID;
    if (batch > kIntMax) return fail(MCC_E_INVALID, "compact-counter fused update batch exceeds 2^31-1");
    if (!std::isfinite(lr)) return fail(MCC_E_INVALID, "compact-counter fused update requires finite lr");
    if (!std::isfinite(lr_scale)) return fail(MCC_E_INVALID, "compact-counter fused update requires finite lr_scale");
    if (!std::isfinite(rms_beta)) return fail(MCC_E_INVALID, "compact-counter fused update requires finite rms_beta");
    if (!std::isfinite(rms_eps) || rms_eps < 0.0f)
        return fail(MCC_E_INVALID, "compact-counter fused update requires non-negative finite rms_eps");
    if (!state || !scale || !v || !grad_out || !x || !workspace)
        return fail(MCC_E_INVALID, "compact-counter fused update received a null buffer");
    const size_t n_groups = out_features * (in_features / 4);
    if (state_nbytes < n_groups * 3) return fail(MCC_E_INVALID, "compact-counter fused update state buffer is too small");
    if (scale_nbytes < out_features * sizeof(float) || v_nbytes < out_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter fused update per-row buffer is too small");
    if (batch > std::numeric_limits<size_t>::max() / sizeof(float) / in_features ||
        batch > std::numeric_limits<size_t>::max() / sizeof(float) / out_features)
        return fail(MCC_E_INVALID, "compact-counter fused update activation size overflows size_t");
    if (grad_out_nbytes < batch * out_features * sizeof(float) || x_nbytes < batch * in_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter fused update activation buffer is too small");
    // the hand-off words behind the slices are used when they are there; without them the
    // contraction is cut up differently and gives the same bits
    const size_t sync_nbytes = mcc::gemm_tn_sync_nbytes((int)batch, (int)out_features, (int)in_features);
    const size_t full_nbytes = mcc_compact_counter_fused_workspace_nbytes(in_features, out_features, batch);
    const bool small = workspace_nbytes < full_nbytes - sync_nbytes;
    SmallPlan plan;
    if (small) {
        plan = small_workspace_plan(in_features, out_features, batch);
        if (plan.kind == SmallPlan::kNone || workspace_nbytes < plan.nbytes)
            return fail(MCC_E_INVALID, "compact-counter fused update workspace is too small");
        if (plan.kind == SmallPlan::kStrip && reinterpret_cast<uintptr_t>(x) % 16)
            return fail(MCC_E_INVALID, "compact-counter fused update with the strip workspace requires 16-byte aligned x");
    }
    if (reinterpret_cast<uintptr_t>(workspace) % 16)
        return fail(MCC_E_INVALID, "compact-counter fused update workspace must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(grad_out) % alignof(float) || reinterpret_cast<uintptr_t>(x) % alignof(float) ||
        reinterpret_cast<uintptr_t>(scale) % alignof(float) || reinterpret_cast<uintptr_t>(v) % alignof(float))
        return fail(MCC_E_INVALID, "compact-counter fused update float buffers must be 4-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    float* grad_w = static_cast<float*>(workspace);
    hipError_t e;
    if (small && plan.kind == SmallPlan::kStrip) {
        ScopedKernelTimer timer("fused_strip", s);
        e = mcc::launch_fused_strip(s, state, scale, v, grad_out, x, workspace, (int)C, (int)in_features,
                                    (int)out_features, (int)batch, lr, lr_scale, rms_beta, rms_eps, seed,
                                    mcc::fused_strip_spin_limit(), workspace_nbytes);
        if (e != hipSuccess) return hip_fail(e, "compact-counter fused strip update launch failed");
        return MCC_OK;
    }
    if (small) {
        // band after band: contraction of the band's rows into the workspace, then their update
        const size_t groups_per_row = in_features / 4;
        for (size_t r0 = 0; r0 < out_features; r0 += (size_t)plan.band_rows) {
            const size_t rows = out_features - r0 < (size_t)plan.band_rows ? out_features - r0 : (size_t)plan.band_rows;
            {
                ScopedKernelTimer timer("gemm_tn_f32", s);
                e = mcc::launch_gemm_tn_f32(s, grad_out + r0, x, grad_w, (int)batch, (int)rows, (int)in_features, grad_w, 0,
                                            (int)out_features, &plan.band_plan);
            }
            if (e != hipSuccess) return hip_fail(e, "compact-counter fused update contraction launch failed");
            {
                ScopedKernelTimer timer("counter_update", s);
                e = mcc::launch_update_dense(s, state + r0 * groups_per_row * 3, scale + r0, v + r0, grad_w, (int)C,
                                             (int)in_features, (int)rows, lr, lr_scale, rms_beta, rms_eps, seed, (int)r0);
            }
            if (e != hipSuccess) return hip_fail(e, "compact-counter fused update launch failed");
        }
        return MCC_OK;
    }
    {
        ScopedKernelTimer timer("gemm_tn_f32", s);
        // the chunk slices start at grad_w: the chunk sums are reduced in place into slice 0
        int* sync_words = sync_nbytes && workspace_nbytes >= full_nbytes
                              ? reinterpret_cast<int*>(grad_w + out_features * in_features)
                              : nullptr;
        e = mcc::launch_gemm_tn_f32(s, grad_out, x, grad_w, (int)batch, (int)out_features, (int)in_features, grad_w,
                                    g_contraction_mode, 0, nullptr, sync_words);
    }
    if (e != hipSuccess) return hip_fail(e, "compact-counter fused update contraction launch failed");
    {
        ScopedKernelTimer timer("counter_update", s);
        e = mcc::launch_update_dense(s, state, scale, v, grad_w, (int)C, (int)in_features, (int)out_features, lr,
                                     lr_scale, rms_beta, rms_eps, seed);
    }
    if (e != hipSuccess) return hip_fail(e, "compact-counter fused update launch failed");
    return MCC_OK;
}

extern "C" {

int mcc_compact_counter_apply_update_fused(void* stream, uint8_t* state, size_t state_nbytes,
                                           float* scale, size_t scale_nbytes, float* v,
                                           size_t v_nbytes, const float* grad_out,
                                           size_t grad_out_nbytes, const float* x, size_t x_nbytes,
                                           void* workspace, size_t workspace_nbytes, size_t C,
                                           size_t in_features, size_t out_features, size_t batch,
                                           float lr, float lr_scale, float rms_beta, float rms_eps,
                                           uint32_t seed) {
    return mcc::fused_update(stream, state, state_nbytes, scale, scale_nbytes, v, v_nbytes, grad_out, grad_out_nbytes, x,
                             x_nbytes, workspace, workspace_nbytes, C, in_features, out_features, batch, lr, lr_scale,
                             rms_beta, rms_eps, seed);
}

// A list whose layers all sit on whole 256 x 256 tiles (and hold enough of them) is contracted as
// equal spans of the whole list, group of at most kSpanGroup tensors by group: one launch per
// group, no token chunks, a gradient of out * in floats per tensor.  Decided from the shapes (and
// the calling thread's contraction mode), so the size query and the call agree.
constexpr size_t kSpanGroup = 96;
static size_t span_groups(size_t n) { return (n + kSpanGroup - 1) / kSpanGroup; }
static void span_group_range(size_t n, size_t g, size_t* begin, size_t* end) {
    const size_t groups = span_groups(n), base = n / groups, rem = n % groups;
    *begin = g * base + (g < rem ? g : rem);
    *end = *begin + base + (g < rem ? 1 : 0);
}
static bool fused_batched_as_spans(const mcc_fused_tensor* tensors, size_t n) {
    if (g_contraction_mode != MCC_CONTRACTION_FP32 || n == 0) return false;
    std::vector<mcc::GemmTnJob> jobs(n);
    for (size_t i = 0; i < n; ++i) {
        const mcc_fused_tensor& t = tensors[i];
        if (t.batch == 0 || t.batch > kIntMax || t.in_features == 0 || t.in_features > kIntMax || t.out_features == 0 ||
            t.out_features > kIntMax)
            return false;
        jobs[i].a = nullptr; jobs[i].b = nullptr; jobs[i].out = nullptr;
        jobs[i].k = (int)t.batch; jobs[i].m = (int)t.out_features; jobs[i].n = (int)t.in_features;
    }
    for (size_t g = 0; g < span_groups(n); ++g) {
        size_t b, e;
        span_group_range(n, g, &b, &e);
        if (!mcc::gemm_tn_spans_group_applies(jobs.data() + b, e - b)) return false;
    }
    return true;
}
constexpr size_t kSpanWordsBytes = 1024;  // kWideSpanWorkgroups hand-off words behind the gradients

// Where tensor i's slices start in a batched fused workspace: each tensor gets what
// mcc_compact_counter_fused_workspace_nbytes asks for (as equal spans: its gradient alone), rounded
// up to 256 bytes.
static size_t fused_batched_region(const mcc_fused_tensor& t, bool spans) {
    if (spans) return (t.out_features * t.in_features * sizeof(float) + 255) / 256 * 256;
    const size_t full = mcc_compact_counter_fused_workspace_nbytes(t.in_features, t.out_features, t.batch);
    return full == 0 ? 0 : (full + 255) / 256 * 256;
}

size_t mcc_compact_counter_fused_batched_workspace_nbytes(const mcc_fused_tensor* tensors, size_t n_tensors) {
    if (!tensors) return 0;
    const bool spans = fused_batched_as_spans(tensors, n_tensors);
    size_t total = spans ? kSpanWordsBytes : 0;
    for (size_t i = 0; i < n_tensors; ++i) {
        const size_t r = fused_batched_region(tensors[i], spans);
        if (r == 0 || r > std::numeric_limits<size_t>::max() - total) return 0;
        total += r;
    }
    return total;
}

int mcc_compact_counter_apply_update_fused_batched(void* stream, const mcc_fused_tensor* tensors, size_t n_tensors,
                                                   void* workspace, size_t workspace_nbytes, size_t C,
                                                   float lr_scale, float rms_beta, float rms_eps) {
    if (n_tensors == 0) return MCC_OK;
    if (!tensors) return fail(MCC_E_INVALID, "compact-counter fused update received a null tensor list");
    if (!workspace) return fail(MCC_E_INVALID, "compact-counter fused update received a null buffer");
    if (reinterpret_cast<uintptr_t>(workspace) % 256)
        return fail(MCC_E_INVALID, "compact-counter batched fused update workspace must be 256-byte aligned");
    const size_t need = mcc_compact_counter_fused_batched_workspace_nbytes(tensors, n_tensors);
    if (need == 0) return fail(MCC_E_INVALID, "compact-counter fused update requires non-zero dimensions");
    if (workspace_nbytes < need) return fail(MCC_E_INVALID, "compact-counter fused update workspace is too small");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool spans = fused_batched_as_spans(tensors, n_tensors);
    std::vector<mcc::GemmTnJob> jobs(n_tensors);
    std::vector<mcc::UpdateTensor> upd(n_tensors);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    for (size_t i = 0; i < n_tensors; ++i) {
        const mcc_fused_tensor& t = tensors[i];
        const char* what = "compact-counter fused update";
        int rc = MCC_OK;
        if (t.batch == 0 || t.batch > kIntMax)
            rc = fail(MCC_E_INVALID, "compact-counter fused update batch must be in [1, 2^31-1]");
        else if (!check_codec(what, C, t.in_features, t.out_features))
            rc = MCC_E_INVALID;
        else if (!t.grad_out || !t.x)
            rc = fail(MCC_E_INVALID, "compact-counter fused update received a null buffer");
        else if (t.batch > std::numeric_limits<size_t>::max() / sizeof(float) / t.in_features ||
                 t.batch > std::numeric_limits<size_t>::max() / sizeof(float) / t.out_features)
            rc = fail(MCC_E_INVALID, "compact-counter fused update activation size overflows size_t");
        else if (t.grad_out_nbytes < t.batch * t.out_features * sizeof(float) ||
                 t.x_nbytes < t.batch * t.in_features * sizeof(float))
            rc = fail(MCC_E_INVALID, "compact-counter fused update activation buffer is too small");
        else if (reinterpret_cast<uintptr_t>(t.grad_out) % alignof(float) || reinterpret_cast<uintptr_t>(t.x) % alignof(float))
            rc = fail(MCC_E_INVALID, "compact-counter fused update float buffers must be 4-byte aligned");
        else if (spans && (reinterpret_cast<uintptr_t>(t.grad_out) % 16 || reinterpret_cast<uintptr_t>(t.x) % 16))
            rc = fail(MCC_E_INVALID, "compact-counter batched fused update of a list of 256-multiple layers requires "
                                     "16-byte aligned grad_out and x");
        if (rc == MCC_OK) {
            // the state side is checked as for the update-only step, with the tensor's region as gradient
            const mcc_counter_tensor c = {t.state, t.state_nbytes, t.scale, t.scale_nbytes, t.v, t.v_nbytes,
                                          reinterpret_cast<const float*>(ws),
                                          t.out_features * t.in_features * sizeof(float), t.in_features,
                                          t.out_features, t.lr, t.seed};
            rc = check_update_tensor(c, C, lr_scale, rms_beta, rms_eps, &upd[i]);
        }
        if (rc != MCC_OK) {
            g_error = "tensor " + std::to_string(i) + ": " + g_error;
            return rc;
        }
        jobs[i].a = t.grad_out;
        jobs[i].b = t.x;
        jobs[i].out = reinterpret_cast<float*>(ws);
        jobs[i].k = (int)t.batch;
        jobs[i].m = (int)t.out_features;
        jobs[i].n = (int)t.in_features;
        // the region ends with the hand-off words of a shape that uses them
        jobs[i].sync_words = !spans && mcc::gemm_tn_sync_nbytes(jobs[i].k, jobs[i].m, jobs[i].n)
                                 ? reinterpret_cast<int*>(jobs[i].out + mcc::gemm_tn_slices(jobs[i].k, jobs[i].m, jobs[i].n) *
                                                                           t.out_features * t.in_features)
                                 : nullptr;
        ws += fused_batched_region(t, spans);
    }
    int* span_words = reinterpret_cast<int*>(ws);  // behind the last region (equal spans only)
    if (n_tensors > 1) {
        std::vector<const void*> states(n_tensors);
        for (size_t i = 0; i < n_tensors; ++i) states[i] = tensors[i].state;
        if (has_duplicate(std::move(states)))
            return fail(MCC_E_INVALID, "compact-counter fused update received the same state twice in one list");
    }
    // every tensor has been validated: nothing below fails for a reason the arguments could show
    // another contraction mode than the fp32 instruction: tensor by tensor, each in its own region
    if (g_contraction_mode != MCC_CONTRACTION_FP32) {
        ws = static_cast<uint8_t*>(workspace);
        for (size_t i = 0; i < n_tensors; ++i) {
            const mcc_fused_tensor& t = tensors[i];
            const size_t region = fused_batched_region(t, false);
            const int rc = mcc_compact_counter_apply_update_fused(
                stream, t.state, t.state_nbytes, t.scale, t.scale_nbytes, t.v, t.v_nbytes, t.grad_out, t.grad_out_nbytes,
                t.x, t.x_nbytes, ws, region, C, t.in_features, t.out_features, t.batch, t.lr, lr_scale, rms_beta,
                rms_eps, t.seed);
            if (rc != MCC_OK) {
                g_error = "tensor " + std::to_string(i) + ": " + g_error;
                return rc;
            }
            ws += region;
        }
        return MCC_OK;
    }
    hipError_t e = hipSuccess;
    {
        ScopedKernelTimer timer("gemm_tn_f32", s);
        if (spans) {
            for (size_t g = 0; g < span_groups(n_tensors) && e == hipSuccess; ++g) {
                size_t b, en;
                span_group_range(n_tensors, g, &b, &en);
                e = mcc::launch_gemm_tn_wide_spans_group(s, jobs.data() + b, en - b, span_words);
            }
        } else {
            e = mcc::launch_gemm_tn_group(s, jobs.data(), n_tensors);
        }
    }
    if (e != hipSuccess) return hip_fail(e, "compact-counter fused update contraction launch failed");
    {
        ScopedKernelTimer timer("counter_update", s);
        e = mcc::launch_update_batch(s, upd.data(), n_tensors, (int)C, lr_scale, rms_beta, rms_eps);
    }
    if (e != hipSuccess) return hip_fail(e, "compact-counter fused update launch failed");
    return MCC_OK;
}

int mcc_set_contraction_mode(int mode) {
    if (mode != MCC_CONTRACTION_FP32 && mode != MCC_CONTRACTION_BF16X6)
        return fail(MCC_E_INVALID, "unknown contraction mode");
    g_contraction_mode = mode;
    return MCC_OK;
}

int mcc_get_contraction_mode(void) { return g_contraction_mode; }

int mcc_matmul_transpose_a_f32(void* stream, const float* a, size_t a_nbytes, const float* b,
                               size_t b_nbytes, float* c, size_t c_nbytes, size_t k, size_t m,
                               size_t n) {
    if (k == 0 || m == 0 || n == 0) return fail(MCC_E_INVALID, "matmul_transpose_a requires non-zero dimensions");
    if (k > kIntMax || m > kIntMax || n > kIntMax)
        return fail(MCC_E_INVALID, "matmul_transpose_a dimensions exceed 2^31-1");
    if (!a || !b || !c) return fail(MCC_E_INVALID, "matmul_transpose_a received a null buffer");
    if (k > std::numeric_limits<size_t>::max() / sizeof(float) / m ||
        k > std::numeric_limits<size_t>::max() / sizeof(float) / n ||
        m > std::numeric_limits<size_t>::max() / sizeof(float) / n)
        return fail(MCC_E_INVALID, "matmul_transpose_a buffer size overflows size_t");
    if (a_nbytes < k * m * sizeof(float) || b_nbytes < k * n * sizeof(float) || c_nbytes < m * n * sizeof(float))
        return fail(MCC_E_INVALID, "matmul_transpose_a buffer is too small");
    if (reinterpret_cast<uintptr_t>(a) % alignof(float) || reinterpret_cast<uintptr_t>(b) % alignof(float) ||
        reinterpret_cast<uintptr_t>(c) % alignof(float))
        return fail(MCC_E_INVALID, "matmul_transpose_a buffers must be 4-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    // small outputs split the token range; the chunk products live in a stream-ordered temporary
    const size_t slices = mcc::gemm_tn_slices((int)k, (int)m, (int)n);
    float* temp = nullptr;
    if (slices > 1) {
        const hipError_t ea = hipMallocAsync(reinterpret_cast<void**>(&temp), slices * m * n * sizeof(float), s);
        if (ea != hipSuccess) return hip_fail(ea, "matmul_transpose_a could not allocate its chunk buffer");
    }
    int* sync_words = nullptr;
    const size_t sync_nbytes = mcc::gemm_tn_sync_nbytes((int)k, (int)m, (int)n);
    if (sync_nbytes && hipMallocAsync(reinterpret_cast<void**>(&sync_words), sync_nbytes, s) != hipSuccess) {
        (void)hipGetLastError();
        sync_words = nullptr;  // the contraction runs without them
    }
    hipError_t e;
    {
        ScopedKernelTimer timer("gemm_tn_f32", s);
        e = mcc::launch_gemm_tn_f32(s, a, b, c, (int)k, (int)m, (int)n, temp, g_contraction_mode, 0, nullptr,
                                    sync_words);
    }
    if (temp) {
        const hipError_t ef = hipFreeAsync(temp, s);
        if (e == hipSuccess) e = ef;
    }
    if (sync_words) {
        const hipError_t ef = hipFreeAsync(sync_words, s);
        if (e == hipSuccess) e = ef;
    }
    if (e != hipSuccess) return hip_fail(e, "matmul_transpose_a launch failed");
    return MCC_OK;
}

int mcc_compact_counter_decode_weight(void* stream, const uint8_t* state, size_t state_nbytes,
                                      const float* scale, size_t scale_nbytes, float* weight,
                                      size_t weight_nbytes, size_t in_features, size_t out_features,
                                      size_t C) {
    if (!check_codec("compact-counter decode", C, in_features, out_features)) return MCC_E_INVALID;
    if (!state || !scale || !weight) return fail(MCC_E_INVALID, "compact-counter decode received a null buffer");
    const size_t groups = out_features * (in_features / 4);
    if (state_nbytes < groups * 3) return fail(MCC_E_INVALID, "compact-counter state buffer is too small");
    if (scale_nbytes < out_features * sizeof(float)) return fail(MCC_E_INVALID, "compact-counter scale buffer is too small");
    if (weight_nbytes < out_features * in_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter weight buffer is too small");
    ScopedKernelTimer timer("counter_decode_weight", static_cast<hipStream_t>(stream));
    const hipError_t e = mcc::launch_decode_weight(static_cast<hipStream_t>(stream), state, scale, weight, (int)C,
                                                   (int)in_features, (int)out_features);
    if (e != hipSuccess) return hip_fail(e, "compact-counter decode launch failed");
    return MCC_OK;
}

int mcc_compact_counter_forward_u8(void* stream, const float* x, size_t x_nbytes,
                                   const uint8_t* state, size_t state_nbytes, const float* scale,
                                   size_t scale_nbytes, float* out, size_t out_nbytes, size_t batch,
                                   size_t in_features, size_t out_features, size_t C) {
    if (batch == 0) return fail(MCC_E_INVALID, "compact-counter forward requires non-zero dimensions");
    if (!check_codec("compact-counter forward", C, in_features, out_features)) return MCC_E_INVALID;
    if (batch > kIntMax / 16) return fail(MCC_E_INVALID, "compact-counter forward batch is too large");
    if (!x || !state || !scale || !out) return fail(MCC_E_INVALID, "compact-counter forward received a null buffer");
    const size_t groups = out_features * (in_features / 4);
    if (state_nbytes < groups * 3) return fail(MCC_E_INVALID, "compact-counter forward state buffer is too small");
    if (scale_nbytes < out_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter forward scale buffer is too small");
    if (batch > std::numeric_limits<size_t>::max() / sizeof(float) / in_features ||
        batch > std::numeric_limits<size_t>::max() / sizeof(float) / out_features)
        return fail(MCC_E_INVALID, "compact-counter forward buffer size overflows size_t");
    if (x_nbytes < batch * in_features * sizeof(float) || out_nbytes < batch * out_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter forward activation buffer is too small");
    ScopedKernelTimer timer("counter_forward", static_cast<hipStream_t>(stream));
    const hipError_t e = mcc::launch_forward(static_cast<hipStream_t>(stream), x, state, scale, out, (int)C,
                                             (int)batch, (int)in_features, (int)out_features);
    if (e != hipSuccess) return hip_fail(e, "compact-counter forward launch failed");
    return MCC_OK;
}

int mcc_compact_counter_backward_input_u8(void* stream, const uint8_t* state, size_t state_nbytes,
                                          const float* scale, size_t scale_nbytes,
                                          const float* grad_out, size_t grad_out_nbytes,
                                          float* grad_x, size_t grad_x_nbytes, size_t batch,
                                          size_t in_features, size_t out_features, size_t C) {
    if (batch == 0) return fail(MCC_E_INVALID, "compact-counter backward-input requires non-zero dimensions");
    if (!check_codec("compact-counter backward-input", C, in_features, out_features)) return MCC_E_INVALID;
    if (batch > kIntMax) return fail(MCC_E_INVALID, "compact-counter backward-input batch is too large");
    if (!state || !scale || !grad_out || !grad_x)
        return fail(MCC_E_INVALID, "compact-counter backward-input received a null buffer");
    const size_t groups = out_features * (in_features / 4);
    if (state_nbytes < groups * 3) return fail(MCC_E_INVALID, "compact-counter state buffer is too small");
    if (scale_nbytes < out_features * sizeof(float)) return fail(MCC_E_INVALID, "compact-counter scale buffer is too small");
    if (batch > std::numeric_limits<size_t>::max() / sizeof(float) / in_features ||
        batch > std::numeric_limits<size_t>::max() / sizeof(float) / out_features)
        return fail(MCC_E_INVALID, "compact-counter backward-input buffer size overflows size_t");
    if (grad_out_nbytes < batch * out_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter grad_out buffer is too small");
    if (grad_x_nbytes < batch * in_features * sizeof(float))
        return fail(MCC_E_INVALID, "compact-counter grad_x buffer is too small");
    ScopedKernelTimer timer("counter_backward_input", static_cast<hipStream_t>(stream));
    const hipError_t e = mcc::launch_backward_input(static_cast<hipStream_t>(stream), grad_out, state, scale,
                                                    grad_x, (int)C, (int)batch, (int)in_features,
                                                    (int)out_features);
    if (e != hipSuccess) return hip_fail(e, "compact-counter backward-input launch failed");
    return MCC_OK;
}

// ---- storage ---------------------------------------------------------------
int mcc_device_alloc(void** ptr, size_t nbytes) {
    if (!ptr) return fail(MCC_E_INVALID, "device alloc received a null result pointer");
    if (nbytes == 0) return fail(MCC_E_INVALID, "cannot allocate zero-byte buffer");
    const size_t bucket = bucket_of(nbytes);
    Pool& p = pool();
    {
        std::lock_guard<std::mutex> lock(p.mu);
        auto it = p.free_blocks.find(bucket);
        if (it != p.free_blocks.end() && !it->second.empty()) {
            *ptr = it->second.back();
            it->second.pop_back();
            p.cached_bytes -= bucket;
            p.live[*ptr] = bucket;
            return MCC_OK;
        }
    }
    void* d = nullptr;
    const hipError_t e = hipMalloc(&d, bucket);
    if (e != hipSuccess) return hip_fail(e, "hipMalloc failed");
    track_alloc(bucket);
    {
        std::lock_guard<std::mutex> lock(p.mu);
        p.live[d] = bucket;
    }
    *ptr = d;
    return MCC_OK;
}

int mcc_device_free(void* ptr) {
    if (!ptr) return MCC_OK;
    Pool& p = pool();
    size_t bucket = 0;
    bool cache = false;
    {
        std::lock_guard<std::mutex> lock(p.mu);
        auto it = p.live.find(ptr);
        if (it == p.live.end()) return fail(MCC_E_INVALID, "device free of a pointer this library did not allocate");
        bucket = it->second;
        p.live.erase(it);
        if (p.cached_bytes + bucket <= kPoolMaxCachedBytes) {
            p.free_blocks[bucket].push_back(ptr);
            p.cached_bytes += bucket;
            cache = true;
        }
    }
    if (!cache) {
        const hipError_t e = hipFree(ptr);
        g_bytes_current.fetch_sub(bucket);
        if (e != hipSuccess) return hip_fail(e, "hipFree failed");
    }
    return MCC_OK;
}

int mcc_device_pool_clear(void) {
    Pool& p = pool();
    std::vector<std::pair<void*, size_t>> blocks;
    {
        std::lock_guard<std::mutex> lock(p.mu);
        for (auto& kv : p.free_blocks)
            for (void* b : kv.second) blocks.emplace_back(b, kv.first);
        p.free_blocks.clear();
        p.cached_bytes = 0;
    }
    int rc = MCC_OK;
    for (auto& b : blocks) {
        const hipError_t e = hipFree(b.first);
        g_bytes_current.fetch_sub(b.second);
        if (e != hipSuccess) rc = hip_fail(e, "hipFree failed");
    }
    return rc;
}

size_t mcc_device_bytes_current(void) { return g_bytes_current.load(); }
size_t mcc_device_bytes_peak(void) { return g_bytes_peak.load(); }
void mcc_device_bytes_reset_peak(void) { g_bytes_peak.store(g_bytes_current.load()); }

int mcc_memcpy_h2d(void* stream, void* dst, const void* src, size_t nbytes) {
    if (nbytes == 0) return MCC_OK;
    if (!dst || !src) return fail(MCC_E_INVALID, "memcpy received a null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);  // src may be pageable and reused by the caller
    if (e != hipSuccess) return hip_fail(e, "host-to-device copy failed");
    return MCC_OK;
}

int mcc_memcpy_d2h(void* stream, void* dst, const void* src, size_t nbytes) {
    if (nbytes == 0) return MCC_OK;
    if (!dst || !src) return fail(MCC_E_INVALID, "memcpy received a null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_fail(e, "device-to-host copy failed");
    return MCC_OK;
}

int mcc_sgd_update_f32(void* stream, float* param, size_t param_nbytes, const float* grad, size_t grad_nbytes,
                       size_t n, float lr) {
    if (n == 0) return fail(MCC_E_INVALID, "sgd_update requires a non-empty tensor");
    if (!param || !grad) return fail(MCC_E_INVALID, "sgd_update received a null buffer");
    if (n > std::numeric_limits<size_t>::max() / sizeof(float) || param_nbytes < n * sizeof(float) ||
        grad_nbytes < n * sizeof(float))
        return fail(MCC_E_INVALID, "sgd_update shape mismatch: a buffer is smaller than n floats");
    if (reinterpret_cast<uintptr_t>(param) % alignof(float) || reinterpret_cast<uintptr_t>(grad) % alignof(float))
        return fail(MCC_E_INVALID, "sgd_update buffers must be 4-byte aligned");
    ScopedKernelTimer timer("sgd_update", static_cast<hipStream_t>(stream));
    const hipError_t e = mcc::launch_sgd_update(static_cast<hipStream_t>(stream), param, grad, n, lr);
    if (e != hipSuccess) return hip_fail(e, "sgd_update launch failed");
    return MCC_OK;
}

int mcc_adam_update_f32(void* stream, float* param, size_t param_nbytes, const float* grad, size_t grad_nbytes,
                        float* m, size_t m_nbytes, float* v, size_t v_nbytes, size_t n, float lr, float beta1,
                        float beta2, float eps, int step, float weight_decay) {
    if (n == 0) return fail(MCC_E_INVALID, "adam_update requires a non-empty tensor");
    if (step <= 0) return fail(MCC_E_INVALID, "adam_update step must be positive");
    if (!param || !grad || !m || !v) return fail(MCC_E_INVALID, "adam_update received a null buffer");
    if (n > std::numeric_limits<size_t>::max() / sizeof(float)) return fail(MCC_E_INVALID, "adam_update size overflows");
    const size_t need = n * sizeof(float);
    if (param_nbytes < need || grad_nbytes < need || m_nbytes < need || v_nbytes < need)
        return fail(MCC_E_INVALID, "adam_update shape mismatch: a buffer is smaller than n floats");
    if (reinterpret_cast<uintptr_t>(param) % alignof(float) || reinterpret_cast<uintptr_t>(grad) % alignof(float) ||
        reinterpret_cast<uintptr_t>(m) % alignof(float) || reinterpret_cast<uintptr_t>(v) % alignof(float))
        return fail(MCC_E_INVALID, "adam_update buffers must be 4-byte aligned");
    const float inv_bias1 = 1.0f / (1.0f - std::pow(beta1, static_cast<float>(step)));
    const float inv_bias2 = 1.0f / (1.0f - std::pow(beta2, static_cast<float>(step)));
    ScopedKernelTimer timer("adam_update", static_cast<hipStream_t>(stream));
    const hipError_t e = mcc::launch_adam_update(static_cast<hipStream_t>(stream), param, grad, m, v, n, lr, beta1,
                                                 beta2, eps, inv_bias1, inv_bias2, weight_decay);
    if (e != hipSuccess) return hip_fail(e, "adam_update launch failed");
    return MCC_OK;
}

int mcc_memset_zero(void* stream, void* dst, size_t nbytes) {
    if (nbytes == 0) return MCC_OK;
    if (!dst) return fail(MCC_E_INVALID, "memset received a null pointer");
    // a fill kernel rather than hipMemsetAsync, so that the call stays valid under graph capture
    const unsigned blocks = (unsigned)((nbytes + 255) / 256 < 4096 ? (nbytes + 255) / 256 : 4096);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint8_t*>(dst), nbytes);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, "device memset failed");
    return MCC_OK;
}

void mcc_profiler_enable(int on) {
    Profiler& p = profiler();
    std::lock_guard<std::mutex> lock(p.mu);
    p.enabled = on != 0;
}

void mcc_profiler_reset(void) {
    Profiler& p = profiler();
    std::lock_guard<std::mutex> lock(p.mu);
    for (const TimedLaunch& r : p.records) {
        p.spare.push_back(r.start);
        p.spare.push_back(r.stop);
    }
    p.records.clear();
}

int mcc_profiler_query(const char* kernel_name, double* total_ms, uint64_t* launches) {
    if (!kernel_name || !total_ms || !launches) return fail(MCC_E_INVALID, "profiler query received a null pointer");
    Profiler& p = profiler();
    std::lock_guard<std::mutex> lock(p.mu);
    double sum = 0.0;
    uint64_t n = 0;
    for (const TimedLaunch& r : p.records) {
        if (std::string(r.name) != kernel_name) continue;
        hipError_t e = hipEventSynchronize(r.stop);
        float ms = 0.0f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, r.start, r.stop);
        if (e != hipSuccess) return hip_fail(e, "profiler query failed");
        sum += ms;
        ++n;
    }
    *total_ms = sum;
    *launches = n;
    return MCC_OK;
}

int mcc_stream_synchronize(void* stream) {
    const hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "stream synchronize failed");
    return MCC_OK;
}

}  // extern "C"
