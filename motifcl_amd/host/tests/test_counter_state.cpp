// Teacher recovery, after MotifCL's tests/test_counter_state.cpp:21-85: a 16x16 ternary teacher
// must be recovered by the in-backward counter update (N=256, C=11, lr 0.005, 800 steps,
// mse <= 5e-3, ternary accuracy >= 0.9).  The input has no requires_grad.  The mean-squared-
// error gradient 2 (pred - y) / numel is formed on the host: the loss op is not part of this
// library.
#include <random>

#include "test_util.hpp"

using namespace motifcl;

int main() {
    return host_test::run("test_counter_state", [](Backend& backend) {
        const int n = 16, N = 256, C = 11, steps = 800;
        const float teacher_scale = 0.25f, lr = 0.005f;
        std::mt19937 rng(0);
        std::uniform_int_distribution<int> tern(-1, 1);
        std::normal_distribution<float> gauss(0.0f, 1.0f);
        std::vector<int> tw(n * n);
        for (int& w : tw) w = tern(rng);
        std::vector<float> xh(N * n), yh(N * n, 0.0f);
        for (float& xi : xh) xi = gauss(rng);
        for (int r = 0; r < N; ++r)
            for (int o = 0; o < n; ++o) {
                float a = 0.0f;
                for (int i = 0; i < n; ++i) a += xh[r * n + i] * (teacher_scale * (float)tw[o * n + i]);
                yh[r * n + o] = a;
            }
        auto x = Tensor::from_cpu(backend, {N, n}, DType::F32, xh.data());
        const float base = std::sqrt(3.0f / (2.0f * (float)n));
        nn::CounterStateLinear layer(backend, n, n, C, lr, 0.0f, teacher_scale / base);

        std::vector<float> gh(N * n);
        for (int s = 0; s < steps; ++s) {
            auto pred = layer.forward(x);
            const auto ph = pred.to_vector<float>();
            for (int k = 0; k < N * n; ++k) gh[k] = 2.0f * (ph[k] - yh[k]) / (float)(N * n);
            pred.backward(Tensor::from_cpu(backend, {N, n}, DType::F32, gh.data()));
        }
        autograd::set_enabled(false);
        const auto ph = layer.forward(x).to_vector<float>();
        autograd::set_enabled(true);
        double mse = 0.0;
        for (int k = 0; k < N * n; ++k) { const double d = (double)ph[k] - (double)yh[k]; mse += d * d; }
        mse /= (double)(N * n);
        const auto sh = layer.state.to_vector<std::uint8_t>();
        const int lv = 2 * C - 1, gpr = n / 4;
        int hit = 0;
        for (int row = 0; row < n; ++row)
            for (int g = 0; g < gpr; ++g) {
                const std::uint8_t* p = sh.data() + (static_cast<std::size_t>(row) * gpr + g) * 3;
                const std::uint32_t word = p[0] | (p[1] << 8) | (p[2] << 16);
                for (int kk = 0; kk < 4; ++kk)
                    if ((int)((word >> (6 * kk)) & 63u) / lv - 1 == tw[row * n + g * 4 + kk]) ++hit;
            }
        const float acc = (float)hit / (float)(n * n);
        std::cout << "teacher recovery: mse=" << mse << " acc=" << acc << '\n';
        if (mse > 5e-3 || acc < 0.9f) throw std::runtime_error("counter teacher-recovery failed");
    });
}
