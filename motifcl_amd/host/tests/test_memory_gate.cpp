// Device-memory accounting and grad_x parity, after MotifCL's tests/test_memory_truth_gate.cpp:
// D=256, N=64, C=11, grad ~ 0.01 N(0,1).  (1) a fused update, after warm-up, creates no new
// device buffer (< 1/4 of a dense weight); what it keeps is ONE workspace per backend of 32 KiB
// per 128 output rows, which is reported, and on a 1024 x 1024 layer even a cold start (workspace
// allocation included) stays below 1/4 of the weight; with the Full policy the same cold start
// does allocate a weight-sized buffer, as does (2) the dense-G path (the gate has teeth);
// (3) in-kernel grad_x agrees with a host product of the decoded weight to 1e-4 and allocates
// only its [N,in] output.
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
        layer.set_fused_workspace(nn::FusedWorkspace::Strip);  // the memory-native way at every size

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
        const std::size_t ws_small = backend.workspace_nbytes();

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
        // cold starts on a larger layer, workspace allocation counted
        const int D2 = 1024;
        std::vector<float> x2(N * D2), g2(N * D2);
        for (float& v : x2) v = g(rng);
        for (float& v : g2) v = 0.01f * g(rng);
        auto xl = Tensor::from_cpu(backend, {N, D2}, DType::F32, x2.data());
        auto gl = Tensor::from_cpu(backend, {N, D2}, DType::F32, g2.data());
        nn::CounterStateLinear big(backend, D2, D2, C, 0.003f);
        const std::size_t big_weight = (std::size_t)D2 * D2 * sizeof(float);
        std::size_t cold[2];
        const nn::FusedWorkspace policies[2] = {nn::FusedWorkspace::Strip, nn::FusedWorkspace::Full};
        for (int p = 0; p < 2; ++p) {
            backend.release_workspace();
            clear_memory_pool();
            device_bytes_reset_peak();
            const std::size_t base = device_bytes_current();
            big.set_fused_workspace(policies[p]);
            big.apply_update_backward(gl, xl, 3u);
            big.check_fused_update();
            cold[p] = device_bytes_peak() - base;
        }
        std::cout << "1024x1024 cold start: strip policy " << cold[0] << " B, full policy " << cold[1]
                  << " B, weight " << big_weight << " B\n";
        if (cold[0] >= big_weight / 4) throw std::runtime_error("strip policy allocated a weight-sized buffer");
        if (cold[1] < big_weight) throw std::runtime_error("full policy did not allocate its f32[out,in] workspace");

        std::cout << "weight_bytes=" << weight_bytes << " peak_fused(new buffers)=" << peak_fused
                  << " peak_dense=" << peak_ref << " peak_gx=" << peak_gx << " gx_relerr=" << relerr
                  << " (persistent fused workspace for 256x256: "
                  << ws_small << " B)\n";
        if (relerr > 1e-4) throw std::runtime_error("in-kernel grad_x parity failed");
        if (peak_gx >= weight_bytes / 2) throw std::runtime_error("grad_x allocated a weight-sized buffer");
        if (peak_fused >= weight_bytes / 4) throw std::runtime_error("fused update created a weight-sized buffer");
        if (peak_ref < weight_bytes / 2) throw std::runtime_error("dense path did not allocate a weight-sized buffer");
    });
}
