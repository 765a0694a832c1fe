// nn::CounterStateLinear with the public surface of
// include/motifcl/nn/compact_counter.hpp:16-60 of MotifCL, implemented on the HIP library.
#pragma once

#include <cstddef>
#include <cstdint>
#include <vector>

#include <motifcl/nn/module.hpp>
#include <motifcl/runtime/backend.hpp>

namespace motifcl::nn {

// How the fused update holds the weight gradient while it needs the whole row's RMS:
//   Full   contraction into f32[out,in] workspace slices, then the update kernel: the fastest way
//          (about 10 percent on a 7B-sized layer; on small ones the only way to keep the GPU busy,
//          their token range being split over many workgroups).  The default.
//   Small  no weight-sized buffer exists at any time, as in the reference
//          (tests/test_memory_truth_gate.cpp:109-113).  Layers of 128-multiples with rows of at
//          least 768 weights keep the gradient in the contraction's registers and exchange 512
//          bytes of partial row sums per output row between the tiles of a strip of 128 or 256 rows; every
//          other layer is updated band by band of an eighth of its rows through a workspace of that
//          size.  Any lr_scale.  check_fused_update() reports a strip step that gave up an
//          inter-tile wait (such a step leaves whole strips without their update).
// Small and Full give identical bytes wherever neither splits the tokens into chunks (fewer than
// 512 tokens, or at least 1024 tiles of 128 x 128); elsewhere they add chunk sums in different
// order and differ by that rounding, both within the tolerance the contraction is held to.
enum class FusedWorkspace { Full, Small };

class CounterStateLinear;

// Collects the fused updates of a backward pass and applies them in one batched call
// (mcc_compact_counter_apply_update_fused_batched): models made of small layers are bound by the
// three launches per layer of the immediate update.  Not in the reference, whose
// CounterBackwardNode updates at once (src/nn/compact_counter.cpp:30-51); the results are the
// same bytes, because no layer's update reads another layer's state and grad_x is taken from the
// pre-update state either way.  The recorded grad_out and x stay alive until flush().
//
//     DeferredCounterUpdates pending;
//     for (auto* l : layers) l->set_deferred(&pending);
//     loss.backward();          // records (layer, grad_out, x, seed) per layer
//     pending.flush();          // one call for all of them
class DeferredCounterUpdates {
public:
    void add(CounterStateLinear& layer, const Tensor& grad_out, const Tensor& x, std::uint32_t seed);
    void flush();
    std::size_t size() const { return items_.size(); }

private:
    struct Item {
        CounterStateLinear* layer;
        Tensor grad_out, x;
        std::uint32_t seed;
    };
    std::vector<Item> items_;
};

// Ternary finite-state "counter" linear layer trained as a per-synapse automaton: the whole
// trainable state is a packed 6-bit code per weight plus a per-row scale and a per-row RMS
// second moment; the update is fused into backward.
class CounterStateLinear : public Module {
public:
    CounterStateLinear(Backend& backend, int in_features, int out_features, int C = 11,
                       float lr = 3e-3f, float lr_scale = 0.0f, float init_gain = 1.0f,
                       float rms_beta = 0.9f, float rms_eps = 1e-3f, std::uint32_t seed = 12345u);

    Tensor forward(const Tensor& x) override;
    std::vector<Parameter*> parameters() override { return {}; }  // self-updating

    Tensor decode_weight() const;                                      // dense [out, in] f32
    void apply_update_seed(const Tensor& grad_w, std::uint32_t seed);  // update-only (dense grad_w)
    void apply_update_backward(const Tensor& grad_out, const Tensor& x, std::uint32_t seed);  // fused
    Tensor backward_input_from_state(const Tensor& grad_out) const;   // grad_x [N, in]
    std::uint32_t next_seed() { return seed_++; }
    // Resume rule of tools/train_ternary15m.cpp:112-121: seeds advance once per update, so a
    // layer built with seed `base` continues an interrupted run from `base + completed_steps`.
    void set_next_seed(std::uint32_t seed) { seed_ = seed; }

    void set_training(bool t) { training_ = t; }
    bool training() const { return training_; }
    void set_fused_workspace(FusedWorkspace w) { fused_workspace_ = w; }
    // With a collector set, backward records the update instead of applying it (see above).
    void set_deferred(DeferredCounterUpdates* d) { deferred_ = d; }
    DeferredCounterUpdates* deferred() const { return deferred_; }
    FusedWorkspace fused_workspace() const { return fused_workspace_; }
    // Waits for the backend and throws if a Small-workspace step on this GPU gave up an inter-tile
    // wait since the last check.
    void check_fused_update() const;
    void set_lr(float lr) { lr_ = lr; }
    float lr() const { return lr_; }

    int in_features() const { return in_; }
    int out_features() const { return out_; }

    // Persistent state (saved/restored as buffers, not optimizer-touched).
    Tensor state;  // U8  [out * in/4 * 3]
    Tensor scale;  // F32 [out]
    Tensor v;      // F32 [out]

private:
    Backend* backend_ = nullptr;
    int in_ = 0;
    int out_ = 0;
    int C_ = 11;
    float lr_ = 3e-3f;
    float lr_scale_ = 0.0f;
    float rms_beta_ = 0.9f;
    float rms_eps_ = 1e-3f;
    std::uint32_t seed_ = 12345u;
    bool training_ = true;
    FusedWorkspace fused_workspace_ = FusedWorkspace::Full;
    DeferredCounterUpdates* deferred_ = nullptr;
    friend class DeferredCounterUpdates;
    std::size_t last_fused_ws_ = 0, last_fused_batch_ = 0;
};

}  // namespace motifcl::nn
