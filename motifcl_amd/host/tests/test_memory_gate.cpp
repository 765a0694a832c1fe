// Device-memory accounting and grad_x parity, after MotifCL's tests/test_memory_truth_gate.cpp:
// D=256, N=64, C=11, grad ~ 0.01 N(0,1).  (1) a fused update, after warm-up, creates no new
// device buffer (< 1/4 of a dense weight); its gradient strip is ONE workspace per backend,
// sized for the largest layer and reported below -- not one buffer per layer; (2) the dense-G
// path does create a weight-sized buffer (the gate has teeth); (3) in-kernel grad_x agrees with
// a host product of the decoded weight to 1e-4 and allocates only its [N,in] output.
#include <random>

#include "test_util.hpp"

using namespace motifcl;

int main() {
    return host_test::run("test_memory_gate", [](Backend& backend) {
        const int D = 256, N = 64, C = 11;
        std::mt19937 rng(0);
        std::normal_distribution<float> g(0.0f, 1.0f);
        std::vector<float> xh(N * D), gh(N * D);
        for (float& v : xh) v = g(rng);
        for (float& v : gh) v = 0.01f * g(rng);
        auto x = Tensor::from_cpu(backend, {N, D}, DType::F32, xh.data());
        auto grad_out = Tensor::from_cpu(backend, {N, D}, DType::F32, gh.data());
        nn::CounterStateLinear layer(backend, D, D, C, 0.003f);

        layer.apply_update_backward(grad_out, x, 1u);
        { auto gw = matmul_transpose_a(grad_out, x); layer.apply_update_seed(gw, 1u); }
        backend.finish();
        const std::size_t weight_bytes = (std::size_t)D * D * sizeof(float);

        clear_memory_pool();
        device_bytes_reset_peak();
        const std::size_t base_f = device_bytes_current();
        layer.apply_update_backward(grad_out, x, 7u);
        backend.finish();
        const std::size_t peak_fused = device_bytes_peak() - base_f;

        clear_memory_pool();
        device_bytes_reset_peak();
        const std::size_t base_r = device_bytes_current();
        { auto gw = matmul_transpose_a(grad_out, x); layer.apply_update_seed(gw, 7u); }
        backend.finish();
        const std::size_t peak_ref = device_bytes_peak() - base_r;

        clear_memory_pool();
        device_bytes_reset_peak();
        const std::size_t base_gx = device_bytes_current();
        auto gx_kernel = layer.backward_input_from_state(grad_out);
        backend.finish();
        const std::size_t peak_gx = device_bytes_peak() - base_gx;
        const auto w = layer.decode_weight().to_vector<float>();
        const auto a = gx_kernel.to_vector<float>();
        double num = 0.0, den = 0.0;
        for (int r = 0; r < N; ++r)
            for (int i = 0; i < D; ++i) {
                double ref = 0.0;
                for (int o = 0; o < D; ++o) ref += (double)gh[r * D + o] * (double)w[o * D + i];
                const double d = (double)a[r * D + i] - ref;
                num += d * d; den += ref * ref;
            }
        const double relerr = den > 0.0 ? std::sqrt(num / den) : 0.0;
        std::cout << "weight_bytes=" << weight_bytes << " peak_fused(new buffers)=" << peak_fused
                  << " peak_dense=" << peak_ref << " peak_gx=" << peak_gx << " gx_relerr=" << relerr
                  << " (persistent fused workspace: " << weight_bytes << " B per backend)\n";
        if (relerr > 1e-4) throw std::runtime_error("in-kernel grad_x parity failed");
        if (peak_gx >= weight_bytes / 2) throw std::runtime_error("grad_x allocated a weight-sized buffer");
        if (peak_fused >= weight_bytes / 4) throw std::runtime_error("fused update created a weight-sized buffer");
        if (peak_ref < weight_bytes / 2) throw std::runtime_error("dense path did not allocate a weight-sized buffer");
    });
}
