// Deferred counter updates: a stack of three CounterStateLinear layers run forward and backward
// twice -- once updating inside backward as MotifCL does (src/nn/compact_counter.cpp:30-51),
// once recording the updates and applying them in one batched call -- must end in the same
// state, scale and v bytes, step after step (the second step starts from the updated state).
#include "test_util.hpp"

using namespace motifcl;

namespace {

struct Stack {
    nn::CounterStateLinear a, b, c;
    explicit Stack(Backend& be) : a(be, 64, 96, 11, 0.01f, 0.0f, 1.0f, 0.9f, 1e-3f, 101u),
                                  b(be, 96, 288, 11, 0.02f, 0.0f, 1.0f, 0.9f, 1e-3f, 202u),
                                  c(be, 288, 32, 11, 0.01f, 0.0f, 1.0f, 0.9f, 1e-3f, 303u) {}
    Tensor forward(const Tensor& x) { return c.forward(b.forward(a.forward(x))); }
    std::vector<nn::CounterStateLinear*> layers() { return {&a, &b, &c}; }
};

}  // namespace

int main() {
    return host_test::run("test_deferred_updates", [](Backend& backend) {
        const int N = 200;
        std::vector<float> xh(N * 64), gh(N * 32);
        host_test::fill_deterministic(xh, 5u, 1.0f);
        host_test::fill_deterministic(gh, 6u, 0.01f);
        Stack now(backend), later(backend);
        nn::DeferredCounterUpdates pending;
        for (auto* l : later.layers()) l->set_deferred(&pending);
        for (int step = 0; step < 3; ++step) {
            auto x1 = Tensor::from_cpu(backend, {N, 64}, DType::F32, xh.data());
            auto x2 = Tensor::from_cpu(backend, {N, 64}, DType::F32, xh.data());
            auto g1 = Tensor::from_cpu(backend, {N, 32}, DType::F32, gh.data());
            auto g2 = Tensor::from_cpu(backend, {N, 32}, DType::F32, gh.data());
            now.forward(x1).backward(g1);
            later.forward(x2).backward(g2);
            if (pending.size() != 3) throw std::runtime_error("expected three recorded updates");
            // nothing has been applied yet: the deferred stack still holds the previous state
            if (step == 0 && later.c.state.to_vector<std::uint8_t>() == now.c.state.to_vector<std::uint8_t>())
                throw std::runtime_error("the immediate update did not change the state");
            pending.flush();
            if (pending.size() != 0) throw std::runtime_error("flush left updates behind");
            backend.finish();
            auto ln = now.layers(), ll = later.layers();
            for (std::size_t i = 0; i < ln.size(); ++i) {
                const std::string tag = "step " + std::to_string(step) + " layer " + std::to_string(i);
                host_test::require_exact(ll[i]->state.to_vector<std::uint8_t>(), ln[i]->state.to_vector<std::uint8_t>(),
                                         tag + " state");
                host_test::require_exact(ll[i]->scale.to_vector<float>(), ln[i]->scale.to_vector<float>(), tag + " scale");
                host_test::require_exact(ll[i]->v.to_vector<float>(), ln[i]->v.to_vector<float>(), tag + " v");
            }
        }
        // layers with different update constants cannot share a call
        nn::CounterStateLinear other(backend, 64, 64, 11, 0.01f, 0.0f, 1.0f, 0.5f, 1e-3f, 1u);
        auto x = Tensor::from_cpu(backend, {N, 64}, DType::F32, xh.data());
        std::vector<float> gh2(N * 64, 0.01f);
        auto g = Tensor::from_cpu(backend, {N, 64}, DType::F32, gh2.data());
        pending.add(later.a, Tensor::from_cpu(backend, {N, 96}, DType::F32, std::vector<float>(N * 96, 0.0f).data()), x, 1u);
        bool threw = false;
        try {
            pending.add(other, g, x, 1u);
        } catch (const Error&) {
            threw = true;
        }
        if (!threw) throw std::runtime_error("mixing rms_beta values must be rejected");
        pending.flush();
    });
}
