// nn::CounterStateLinear on the HIP library.  Structure and ordering follow
// src/nn/compact_counter.cpp of MotifCL: the constructor packs the initial state
// (:55-85), the backward node computes grad_x from the pre-update state, then runs the fused
// update under NoGradGuard, then propagates (:30-51), and forward attaches that node whenever
// the layer is training, whether or not the input wants a gradient (:295-298).
#include <motifcl/nn/compact_counter.hpp>

#include <motifcl/autograd/node.hpp>
#include <motifcl/core/error.hpp>

#include <motifcl_amd.h>

#include <cmath>
#include <memory>
#include <random>
#include <string>
#include <vector>

namespace motifcl::nn {
namespace {

// Packed start state: every weight a ternary value drawn from {-1, 0, +1} with its counter at
// zero, code = (t + 1)(2C - 1) + (C - 1), four codes to a little-endian 24-bit word.  The draws
// are MotifCL's (std::mt19937(seed) through uniform_int_distribution<int>(-1, 1), row-major), so
// a layer built with the same seed and standard library starts from the same weights.
std::vector<std::uint8_t> initial_state(int out_features, int in_features, int C, std::uint32_t seed) {
    const std::size_t groups = static_cast<std::size_t>(out_features) * (in_features / 4);
    const std::uint32_t zero_counter = static_cast<std::uint32_t>(C - 1), levels = static_cast<std::uint32_t>(2 * C - 1);
    std::mt19937 rng(seed);
    std::uniform_int_distribution<int> ternary(-1, 1);
    std::vector<std::uint8_t> bytes(groups * 3);
    for (std::size_t g = 0; g < groups; ++g) {
        std::uint32_t word = 0;
        for (int k = 0; k < 4; ++k)
            word |= (static_cast<std::uint32_t>(ternary(rng) + 1) * levels + zero_counter) << (6 * k);
        bytes[3 * g] = static_cast<std::uint8_t>(word);
        bytes[3 * g + 1] = static_cast<std::uint8_t>(word >> 8);
        bytes[3 * g + 2] = static_cast<std::uint8_t>(word >> 16);
    }
    return bytes;
}

// What backward does for a counter layer (src/nn/compact_counter.cpp:30-51): the input gradient is
// taken from the state the forward pass saw, then the state is updated -- immediately, or recorded
// for one batched call -- and only then does the input's own backward run.  The update happens
// whether or not the input wants a gradient, so a layer fed with raw data still learns.
struct CounterBackwardNode : autograd::Node {
    CounterBackwardNode(Tensor input, CounterStateLinear* owner, std::uint32_t update_seed)
        : input_(std::move(input)), owner_(owner), update_seed_(update_seed) {}

    std::vector<Tensor> inputs() const override { return {input_}; }

    void backward(const Tensor& grad_out) override {
        Tensor grad_input;
        if (input_.requires_grad()) grad_input = owner_->backward_input_from_state(grad_out);
        {
            autograd::NoGradGuard no_graph;  // the update is a side effect, not part of the graph
            if (DeferredCounterUpdates* pending = owner_->deferred())
                pending->add(*owner_, grad_out, input_, update_seed_);
            else
                owner_->apply_update_backward(grad_out, input_, update_seed_);
        }
        if (grad_input.valid()) input_.backward(grad_input);
    }

private:
    Tensor input_;
    CounterStateLinear* owner_;
    std::uint32_t update_seed_;
};

const float* f32(const Tensor& t) { return static_cast<const float*>(t.data()); }
float* f32(Tensor& t) { return static_cast<float*>(t.data()); }

}  // namespace

CounterStateLinear::CounterStateLinear(Backend& backend, int in_features, int out_features, int C, float lr,
                                       float lr_scale, float init_gain, float rms_beta, float rms_eps,
                                       std::uint32_t seed)
    : backend_(&backend), in_(in_features), out_(out_features), C_(C), lr_(lr), lr_scale_(lr_scale),
      rms_beta_(rms_beta), rms_eps_(rms_eps), seed_(seed) {
    // the reference's conditions and messages (src/nn/compact_counter.cpp:60-62)
    MCL_CHECK(in_ > 0 && out_ > 0, "CounterStateLinear requires positive dimensions");
    MCL_CHECK(C_ > 0 && 3 * (2 * C_ - 1) <= 64, "C too large for 6-bit packed state encoding");
    MCL_CHECK(in_ % 4 == 0, "CounterStateLinear requires in_features divisible by 4 (6-bit packing)");

    const std::vector<std::uint8_t> packed = initial_state(out_, in_, C_, seed);
    state = Tensor::from_cpu(*backend_, {static_cast<int64_t>(packed.size())}, DType::U8, packed.data());
    // every row starts at init_gain * sqrt(3 / (2 in)) with an empty second moment
    const std::vector<float> start_scale(static_cast<std::size_t>(out_),
                                         init_gain * std::sqrt(3.0f / (2.0f * static_cast<float>(in_))));
    const std::vector<float> zeros(static_cast<std::size_t>(out_), 0.0f);
    scale = Tensor::from_cpu(*backend_, {out_}, DType::F32, start_scale.data());
    v = Tensor::from_cpu(*backend_, {out_}, DType::F32, zeros.data());
}

Tensor CounterStateLinear::decode_weight() const {
    Tensor w = Tensor::empty(*backend_, {out_, in_}, DType::F32);
    const int rc = mcc_compact_counter_decode_weight(
        backend_->hip_stream(), static_cast<const std::uint8_t*>(state.data()), state.nbytes(), f32(scale),
        scale.nbytes(), f32(w), w.nbytes(), static_cast<std::size_t>(in_), static_cast<std::size_t>(out_),
        static_cast<std::size_t>(C_));
    MCL_CHECK(rc == MCC_OK, std::string("hip compact-counter decode_weight failed: ") + mcc_last_error());
    return w;
}

void CounterStateLinear::apply_update_seed(const Tensor& grad_w, std::uint32_t seed) {
    MCL_CHECK(grad_w.dtype() == DType::F32 && grad_w.numel() == static_cast<int64_t>(out_) * in_,
              "apply_update_seed expects an f32 [out, in] gradient");
    const int rc = mcc_compact_counter_apply_update_dense(
        backend_->hip_stream(), static_cast<std::uint8_t*>(state.data()), state.nbytes(), f32(scale), scale.nbytes(),
        f32(v), v.nbytes(), f32(grad_w), grad_w.nbytes(), static_cast<std::size_t>(C_), static_cast<std::size_t>(in_),
        static_cast<std::size_t>(out_), lr_, lr_scale_, rms_beta_, rms_eps_, seed);
    MCL_CHECK(rc == MCC_OK, std::string("hip compact-counter update failed: ") + mcc_last_error());
}

void CounterStateLinear::apply_update_backward(const Tensor& grad_out, const Tensor& x, std::uint32_t seed) {
    MCL_CHECK(x.ndim() == 2 && grad_out.ndim() == 2, "apply_update_backward expects rank-2 tensors");
    const std::size_t N = static_cast<std::size_t>(x.shape()[0]);
    const std::size_t in = static_cast<std::size_t>(in_), out = static_cast<std::size_t>(out_);
    std::size_t ws = 0;
    if (fused_workspace_ == FusedWorkspace::Small)
        ws = mcc_compact_counter_fused_strip_workspace_nbytes(in, out, N);  // 0: no smaller way for this shape
    if (ws == 0) ws = mcc_compact_counter_fused_workspace_nbytes(in, out, N);
    void* scratch = backend_->workspace(ws);
    // exactly ws bytes are lent: the size selects how the step runs
    const int rc = mcc_compact_counter_apply_update_fused(
        backend_->hip_stream(), static_cast<std::uint8_t*>(state.data()), state.nbytes(), f32(scale), scale.nbytes(),
        f32(v), v.nbytes(), f32(grad_out), grad_out.nbytes(), f32(x), x.nbytes(), scratch, ws,
        static_cast<std::size_t>(C_), in, out, N, lr_, lr_scale_, rms_beta_, rms_eps_, seed);
    MCL_CHECK(rc == MCC_OK, std::string("hip compact-counter fused update failed: ") + mcc_last_error());
    last_fused_ws_ = ws;
    last_fused_batch_ = N;
}

void DeferredCounterUpdates::add(CounterStateLinear& layer, const Tensor& grad_out, const Tensor& x,
                                 std::uint32_t seed) {
    MCL_CHECK(x.ndim() == 2 && grad_out.ndim() == 2, "apply_update_backward expects rank-2 tensors");
    MCL_CHECK(items_.empty() || items_.front().layer->backend_ == layer.backend_,
              "DeferredCounterUpdates collects layers of one backend");
    MCL_CHECK(items_.empty() || (items_.front().layer->C_ == layer.C_ && items_.front().layer->lr_scale_ == layer.lr_scale_ &&
                                 items_.front().layer->rms_beta_ == layer.rms_beta_ &&
                                 items_.front().layer->rms_eps_ == layer.rms_eps_),
              "DeferredCounterUpdates collects layers with the same C, lr_scale, rms_beta and rms_eps");
    items_.push_back(Item{&layer, grad_out, x, seed});
}

void DeferredCounterUpdates::flush() {
    if (items_.empty()) return;
    std::vector<mcc_fused_tensor> list(items_.size());
    for (std::size_t i = 0; i < items_.size(); ++i) {
        Item& it = items_[i];
        CounterStateLinear& l = *it.layer;
        mcc_fused_tensor& t = list[i];
        t.state = static_cast<std::uint8_t*>(l.state.data());
        t.state_nbytes = l.state.nbytes();
        t.scale = f32(l.scale);
        t.scale_nbytes = l.scale.nbytes();
        t.v = f32(l.v);
        t.v_nbytes = l.v.nbytes();
        t.grad_out = f32(it.grad_out);
        t.grad_out_nbytes = it.grad_out.nbytes();
        t.x = f32(it.x);
        t.x_nbytes = it.x.nbytes();
        t.in_features = static_cast<std::size_t>(l.in_);
        t.out_features = static_cast<std::size_t>(l.out_);
        t.batch = static_cast<std::size_t>(it.x.shape()[0]);
        t.lr = l.lr_;
        t.seed = it.seed;
    }
    CounterStateLinear& first = *items_.front().layer;
    const std::size_t ws = mcc_compact_counter_fused_batched_workspace_nbytes(list.data(), list.size());
    MCL_CHECK(ws != 0, "hip compact-counter fused update failed: batched workspace size is zero");
    void* scratch = first.backend_->workspace(ws);
    const int rc = mcc_compact_counter_apply_update_fused_batched(
        first.backend_->hip_stream(), list.data(), list.size(), scratch, ws, static_cast<std::size_t>(first.C_),
        first.lr_scale_, first.rms_beta_, first.rms_eps_);
    MCL_CHECK(rc == MCC_OK, std::string("hip compact-counter fused update failed: ") + mcc_last_error());
    for (Item& it : items_) it.layer->last_fused_ws_ = 0;  // nothing to check across workgroups on this path
    items_.clear();  // releases grad_out and x (the stream keeps them until the kernels have run)
}

void CounterStateLinear::check_fused_update() const {
    // the library counts given-up strip steps per GPU, not per workspace: the answer covers every
    // layer's step on this GPU since the last check
    const int rc = mcc_compact_counter_fused_check(backend_->hip_stream(), backend_->workspace(1), 1,
                                                   static_cast<std::size_t>(in_), static_cast<std::size_t>(out_),
                                                   last_fused_batch_ ? last_fused_batch_ : 1);
    MCL_CHECK(rc == MCC_OK, std::string("hip compact-counter fused update failed: ") + mcc_last_error());
}

Tensor CounterStateLinear::backward_input_from_state(const Tensor& grad_out) const {
    MCL_CHECK(grad_out.backend_ptr() == backend_, "CounterStateLinear backward_input backend mismatch");
    const int N = static_cast<int>(grad_out.shape()[0]);
    Tensor grad_x = Tensor::empty(*backend_, {N, in_}, DType::F32);
    const int rc = mcc_compact_counter_backward_input_u8(
        backend_->hip_stream(), static_cast<const std::uint8_t*>(state.data()), state.nbytes(), f32(scale),
        scale.nbytes(), f32(grad_out), grad_out.nbytes(), f32(grad_x), grad_x.nbytes(), static_cast<std::size_t>(N),
        static_cast<std::size_t>(in_), static_cast<std::size_t>(out_), static_cast<std::size_t>(C_));
    MCL_CHECK(rc == MCC_OK, std::string("hip compact-counter backward_input failed: ") + mcc_last_error());
    return grad_x;
}

Tensor CounterStateLinear::forward(const Tensor& x) {
    MCL_CHECK(x.dtype() == DType::F32 && x.ndim() == 2, "CounterStateLinear expects rank-2 f32 input");
    MCL_CHECK(x.shape()[1] == in_, "CounterStateLinear input feature mismatch");
    Tensor y = Tensor::empty(*backend_, {x.shape()[0], out_}, DType::F32);
    const int rc = mcc_compact_counter_forward_u8(
        backend_->hip_stream(), f32(x), x.nbytes(), static_cast<const std::uint8_t*>(state.data()), state.nbytes(),
        f32(scale), scale.nbytes(), f32(y), y.nbytes(), static_cast<std::size_t>(x.shape()[0]),
        static_cast<std::size_t>(in_), static_cast<std::size_t>(out_), static_cast<std::size_t>(C_));
    MCL_CHECK(rc == MCC_OK, std::string("hip compact-counter forward failed: ") + mcc_last_error());
    if (autograd::is_enabled() && training_) {  // gate on training, not on x.requires_grad
        y.set_requires_grad(true);
        y._set_grad_fn(std::make_shared<CounterBackwardNode>(x, this, next_seed()));
    }
    return y;
}

}  // namespace motifcl::nn
