// Error convention of the layer: motifcl::Error with the "MotifCL check failed:" prefix
// (include/motifcl/core/error.hpp:19-27), raised for the cases the reference rejects
// (src/nn/compact_counter.cpp:60-62,267-268; tests/test_vulkan_runtime_standalone.cpp:19-23).
#include "test_util.hpp"

using namespace motifcl;

template <typename F>
static void expect_error(const char* what, F f) {
    try {
        f();
    } catch (const Error& e) {
        if (std::string(e.what()).rfind("MotifCL check failed:", 0) != 0)
            throw std::runtime_error(std::string(what) + ": wrong message prefix");
        return;
    }
    throw std::runtime_error(std::string(what) + ": no error raised");
}

int main() {
    return host_test::run("test_layer_errors", [](Backend& backend) {
        expect_error("in % 4", [&] { nn::CounterStateLinear l(backend, 6, 2); });
        expect_error("C too large", [&] { nn::CounterStateLinear l(backend, 8, 2, 12); });
        expect_error("non-positive dims", [&] { nn::CounterStateLinear l(backend, 8, 0); });
        nn::CounterStateLinear layer(backend, 8, 2, 3);
        std::vector<float> xh(3 * 4, 0.5f);
        auto bad = Tensor::from_cpu(backend, {3, 4}, DType::F32, xh.data());
        expect_error("feature mismatch", [&] { layer.forward(bad); });
        layer.set_lr(std::nanf(""));
        std::vector<float> x8(2 * 8, 0.1f), g2(2 * 2, 0.1f);
        auto x = Tensor::from_cpu(backend, {2, 8}, DType::F32, x8.data());
        auto go = Tensor::from_cpu(backend, {2, 2}, DType::F32, g2.data());
        expect_error("NaN lr", [&] { layer.apply_update_backward(go, x, 1u); });
        const auto before = layer.state.to_vector<std::uint8_t>();
        if (layer.state.to_vector<std::uint8_t>() != before) throw std::runtime_error("rejected update touched state");
    });
}
