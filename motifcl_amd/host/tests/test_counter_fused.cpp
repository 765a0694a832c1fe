// Forward, grad_x and the exact state transition of CounterStateLinear, in the shape of
// MotifCL's tests/test_vulkan_counter_fused.cpp:57-140: rows=37, in=68, out=35, C=3, lr=1,
// lr_scale=0.05, eps=1e-6, seed 777.  The autograd-driven update must equal, byte for byte, a
// twin layer updated by a direct apply_update_backward with the same seed.
#include "test_util.hpp"

using namespace motifcl;

int main() {
    return host_test::run("test_counter_fused", [](Backend& backend) {
        constexpr int rows = 37, in_features = 68, out_features = 35, C = 3;
        constexpr std::uint32_t seed = 777u;
        std::vector<float> x_host(rows * in_features), go_host(rows * out_features);
        host_test::fill_deterministic(x_host, 0x1234u, 0.8f);
        host_test::fill_deterministic(go_host, 0x5678u, 0.9f);

        nn::CounterStateLinear fast(backend, in_features, out_features, C, 1.0f, 0.05f, 1.0f, 0.9f, 1.0e-6f, seed);
        nn::CounterStateLinear twin(backend, in_features, out_features, C, 1.0f, 0.05f, 1.0f, 0.9f, 1.0e-6f, seed);
        const auto state_before = twin.state.to_vector<std::uint8_t>();
        const auto scale_before = twin.scale.to_vector<float>();
        host_test::require_exact(fast.state.to_vector<std::uint8_t>(), state_before, "initial packed state");
        host_test::require_exact(fast.scale.to_vector<float>(), scale_before, "initial scale");

        auto x_fast = Tensor::from_cpu(backend, {rows, in_features}, DType::F32, x_host.data());
        auto x_twin = Tensor::from_cpu(backend, {rows, in_features}, DType::F32, x_host.data());
        auto grad_out = Tensor::from_cpu(backend, {rows, out_features}, DType::F32, go_host.data());
        x_fast.set_requires_grad(true);

        const auto w = twin.decode_weight().to_vector<float>();
        std::vector<float> y_ref(rows * out_features), gx_ref(rows * in_features);
        for (int r = 0; r < rows; ++r)
            for (int o = 0; o < out_features; ++o) {
                float acc = 0.0f;
                for (int i = 0; i < in_features; ++i) acc += x_host[r * in_features + i] * w[o * in_features + i];
                y_ref[r * out_features + o] = acc;
            }
        for (int r = 0; r < rows; ++r)
            for (int i = 0; i < in_features; ++i) {
                float acc = 0.0f;
                for (int o = 0; o < out_features; ++o) acc += go_host[r * out_features + o] * w[o * in_features + i];
                gx_ref[r * in_features + i] = acc;
            }

        auto y_fast = fast.forward(x_fast);
        if (!y_fast._grad_fn()) throw std::runtime_error("training forward attached no update node");
        host_test::require_close(y_fast.to_vector<float>(), y_ref, 2.0e-5f, "counter forward");

        y_fast.backward(grad_out);
        if (!x_fast.grad()) throw std::runtime_error("backward produced no grad_x");
        host_test::require_close(x_fast.grad()->to_vector<float>(), gx_ref, 2.0e-5f, "counter grad_x");

        twin.apply_update_backward(grad_out, x_twin, seed);
        backend.finish();
        const auto expected_state = twin.state.to_vector<std::uint8_t>();
        const auto expected_scale = twin.scale.to_vector<float>();
        host_test::require_exact(fast.state.to_vector<std::uint8_t>(), expected_state, "counter state transition");
        host_test::require_exact(fast.scale.to_vector<float>(), expected_scale, "counter scale transition");
        host_test::require_exact(fast.v.to_vector<float>(), twin.v.to_vector<float>(), "counter RMS transition");
        if (expected_state == state_before || expected_scale == scale_before)
            throw std::runtime_error("update witness produced no packed-state/scale delta");

        // inference mode attaches nothing; a grad-less input still updates the layer
        fast.set_training(false);
        if (fast.forward(x_twin)._grad_fn()) throw std::runtime_error("inference forward attached an update node");
        fast.set_training(true);
        const auto s0 = fast.state.to_vector<std::uint8_t>();
        fast.forward(x_twin).backward(grad_out);
        if (fast.state.to_vector<std::uint8_t>() == s0) throw std::runtime_error("grad-less input did not update the layer");
        if (x_twin.grad()) throw std::runtime_error("grad-less input received a gradient");
    });
}
