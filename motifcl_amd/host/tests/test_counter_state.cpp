// The behaviour MotifCL's tests/test_counter_state.cpp:21-85 asks of the layer: trained only by
// the update that runs inside backward (the input carries no gradient), a 16 x 16 counter layer
// recovers a ternary teacher -- mse <= 5e-3 and at least 90 % of the ternary values after 800
// steps on 256 fixed samples (C = 11, lr = 0.005, teacher scale 0.25).  The loss gradient
// 2 (pred - y) / numel is formed on the host: the loss op is not part of this library.
// A second, shorter run is the single-layer witness of tests/test_vulkan_memory_native.cpp:48-108:
// 128 samples, 200 steps; the loss must at least halve and 80 % of the decoded weights must lie
// within half a scale of the teacher's.
#include <utility>

#include "test_util.hpp"

using namespace motifcl;

namespace {

struct Problem {
    int width, samples;
    std::vector<int> teacher;      // [width, width] ternary
    std::vector<float> inputs;     // [samples, width]
    std::vector<float> targets;    // [samples, width] = inputs . (scale * teacher)^T
};

Problem make_problem(int width, int samples, float scale) {
    Problem p{width, samples, {}, {}, {}};
    p.teacher.resize((std::size_t)width * width);
    for (std::size_t k = 0; k < p.teacher.size(); ++k) p.teacher[k] = host_test::ternary_at(11u, (std::uint32_t)k);
    p.inputs.resize((std::size_t)samples * width);
    host_test::fill_normal(p.inputs, 12u, 1.0f);
    p.targets.assign((std::size_t)samples * width, 0.0f);
    for (int s = 0; s < samples; ++s)
        for (int o = 0; o < width; ++o) {
            float dot = 0.0f;
            for (int i = 0; i < width; ++i) dot += p.inputs[s * width + i] * (scale * (float)p.teacher[o * width + i]);
            p.targets[s * width + o] = dot;
        }
    return p;
}

// ternary value of weight (row, col) in a packed state: code / (2C - 1) - 1
int ternary_of(const std::vector<std::uint8_t>& packed, int row, int col, int width, int C) {
    const std::uint8_t* g = packed.data() + ((std::size_t)row * (width / 4) + col / 4) * 3;
    const std::uint32_t word = g[0] | (g[1] << 8) | (g[2] << 16);
    return (int)((word >> (6 * (col % 4))) & 63u) / (2 * C - 1) - 1;
}

// Trains a fresh layer on the problem; returns {first loss, last loss} and leaves the layer trained.
std::pair<double, double> train(Backend& backend, nn::CounterStateLinear& layer, const Problem& p, int steps) {
    const int numel = p.samples * p.width;
    auto x = Tensor::from_cpu(backend, {p.samples, p.width}, DType::F32, p.inputs.data());
    std::vector<float> grad(numel);
    double first = 0.0, last = 0.0;
    for (int step = 0; step < steps; ++step) {
        auto pred = layer.forward(x);
        const auto out = pred.to_vector<float>();
        double loss = 0.0;
        for (int k = 0; k < numel; ++k) {
            const float d = out[k] - p.targets[k];
            loss += (double)d * d;
            grad[k] = 2.0f * d / (float)numel;
        }
        loss /= numel;
        if (step == 0) first = loss;
        last = loss;
        pred.backward(Tensor::from_cpu(backend, {p.samples, p.width}, DType::F32, grad.data()));
    }
    return {first, last};
}

}  // namespace

int main() {
    return host_test::run("test_counter_state", [](Backend& backend) {
        const int C = 11;
        const float scale = 0.25f;
        {
            const Problem p = make_problem(16, 256, scale);
            const int numel = p.samples * p.width;
            // init_gain chosen so that the layer starts at the teacher's scale
            nn::CounterStateLinear layer(backend, p.width, p.width, C, 0.005f, 0.0f,
                                         scale / std::sqrt(3.0f / (2.0f * (float)p.width)));
            train(backend, layer, p, 800);
            auto x = Tensor::from_cpu(backend, {p.samples, p.width}, DType::F32, p.inputs.data());
            autograd::set_enabled(false);
            const auto out = layer.forward(x).to_vector<float>();
            autograd::set_enabled(true);
            double mse = 0.0;
            for (int k = 0; k < numel; ++k) mse += ((double)out[k] - p.targets[k]) * ((double)out[k] - p.targets[k]);
            mse /= numel;
            const auto packed = layer.state.to_vector<std::uint8_t>();
            int recovered = 0;
            for (int r = 0; r < p.width; ++r)
                for (int c = 0; c < p.width; ++c) recovered += ternary_of(packed, r, c, p.width, C) == p.teacher[r * p.width + c];
            const float acc = (float)recovered / (float)(p.width * p.width);
            std::cout << "teacher recovery: mse=" << mse << " acc=" << acc << '\n';
            if (mse > 5e-3 || acc < 0.9f) throw std::runtime_error("counter teacher-recovery failed");
        }
        {
            const Problem p = make_problem(16, 128, scale);
            nn::CounterStateLinear layer(backend, p.width, p.width, C, 0.005f, 0.0f,
                                         scale / std::sqrt(3.0f / (2.0f * (float)p.width)));
            const auto loss = train(backend, layer, p, 200);
            const auto w = layer.decode_weight().to_vector<float>();
            int close = 0;
            for (std::size_t k = 0; k < w.size(); ++k) close += std::fabs(w[k] - scale * (float)p.teacher[k]) <= 0.5f * scale;
            const float acc = (float)close / (float)w.size();
            std::cout << "short run: loss " << loss.first << " -> " << loss.second << ", decoded acc=" << acc << '\n';
            if (!(loss.second < 0.5 * loss.first) || acc < 0.8f) throw std::runtime_error("short teacher-recovery run failed");
        }
    });
}
