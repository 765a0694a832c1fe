// The side-optimizer checks of MotifCL's tests/test_adam.cpp:11-42 that concern adam_update and
// the decoupled weight decay (the Parameter/optimizer classes around them are outside this
// mirror), plus sgd_update and the argument checks of src/ops/optim.cpp:17-20,49-51,66.
#include "test_util.hpp"

using namespace motifcl;

int main() {
    return host_test::run("test_adam", [](Backend& backend) {
        std::vector<float> ph = {1, 2, 3, 4};
        std::vector<float> gh = {0.1f, -0.2f, 0.3f, -0.4f};
        auto P = Tensor::from_cpu(backend, {4}, DType::F32, ph.data());
        auto G = Tensor::from_cpu(backend, {4}, DType::F32, gh.data());
        auto M = Tensor::zeros(backend, {4});
        auto V = Tensor::zeros(backend, {4});
        adam_update(P, G, M, V, 1e-3f, 0.9f, 0.999f, 1e-8f, 1);
        auto out = P.to_vector<float>();
        for (std::size_t i = 0; i < out.size(); ++i) {
            if (!std::isfinite(out[i])) throw std::runtime_error("adam produced a non-finite value");
            // first step from zero moments: |delta| = lr
            const float want = ph[i] - (gh[i] > 0 ? 1e-3f : -1e-3f);
            if (std::fabs(out[i] - want) > 1e-6f) throw std::runtime_error("adam first step is not lr * sign(g)");
        }

        // tests/test_adam.cpp:22-42: g = 1, lr = 1e-2, weight decay 0.1 -> p0 - lr - lr * wd * p0
        for (int i = 0; i < 5; ++i) {
            const float p0 = static_cast<float>(i + 1), one = 1.0f;
            auto p = Tensor::from_cpu(backend, {1}, DType::F32, &p0);
            auto g = Tensor::from_cpu(backend, {1}, DType::F32, &one);
            auto m = Tensor::zeros(backend, {1});
            auto v = Tensor::zeros(backend, {1});
            adam_update_fast(p, g, m, v, 1e-2f, 0.9f, 0.999f, 1e-8f, 1, 0.1f);
            const float expected = p0 - 1e-2f - 1e-2f * 0.1f * p0;
            if (std::fabs(p.to_vector<float>()[0] - expected) > 1e-4f)
                throw std::runtime_error("decoupled weight decay differs from the reference's expectation");
        }

        auto S = Tensor::from_cpu(backend, {4}, DType::F32, ph.data());
        sgd_update(S, G, 0.5f);
        host_test::require_exact(S.to_vector<float>(), {1 - 0.5f * 0.1f, 2 + 0.5f * 0.2f, 3 - 0.5f * 0.3f, 4 + 0.5f * 0.4f},
                                 "sgd_update");

        auto expect_error = [](auto body, const std::string& needle) {
            try {
                body();
            } catch (const Error& e) {
                if (std::string(e.what()).find(needle) != std::string::npos) return;
                throw std::runtime_error(std::string("wrong message: ") + e.what());
            }
            throw std::runtime_error("no Error for: " + needle);
        };
        auto G3 = Tensor::zeros(backend, {3});
        auto U8 = Tensor::zeros(backend, {4}, DType::U8);
        expect_error([&] { sgd_update(P, G3, 0.1f); }, "sgd_update shape mismatch");
        expect_error([&] { sgd_update(P, U8, 0.1f); }, "sgd_update supports f32 only");
        expect_error([&] { adam_update(P, G3, M, V, 1e-3f, 0.9f, 0.999f, 1e-8f, 1); }, "adam_update shape mismatch");
        expect_error([&] { adam_update(P, G, M, V, 1e-3f, 0.9f, 0.999f, 1e-8f, 0); }, "step must be positive");
    });
}
