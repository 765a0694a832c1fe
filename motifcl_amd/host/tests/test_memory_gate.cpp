// Device-memory accounting of the fused update and of grad_x, after the property MotifCL's
// tests/test_memory_truth_gate.cpp:94-118 checks: the fused update must not create a buffer of the
// size of the weight gradient (gate: a quarter of out*in*4 bytes), while the dense-gradient path
// does (the gate has teeth), and the in-kernel grad_x agrees with a host product of the decoded
// weight to 1e-4 while allocating only its [N, in] output.  Here every allocation is counted from
// a cold start -- the layer's transient workspace included -- and the gate is asked of the Small
// workspace policy at the reference's D = 256, with lr_scale = 0.05 (the hyper-parameters of
// tests/test_vulkan_counter_fused.cpp:68), at D = 288 (the 15M model's width, not a multiple of
// 128) and at 2048 (the strip path: 512 bytes of partial sums per output row, which the pooled
// allocator of this mirror rounds up to a power of two).  A last part runs two layers through the one workspace of
// the backend, one on the strip path with its waits forced to give up, and asks that the failure
// is still reported after the other layer has used the workspace.
#include "test_util.hpp"

#include <motifcl_amd_diag.h>

using namespace motifcl;

namespace {

struct Peaks {
    std::size_t small_ws, full_ws, dense, grad_x;
    double grad_x_relerr;
};

Peaks measure(Backend& backend, int D, int N, float lr_scale) {
    const int C = 11;
    std::vector<float> xh((std::size_t)N * D), gh((std::size_t)N * D);
    host_test::fill_normal(xh, 21u + (std::uint32_t)D, 1.0f);
    host_test::fill_normal(gh, 22u + (std::uint32_t)D, 0.01f);
    auto x = Tensor::from_cpu(backend, {N, D}, DType::F32, xh.data());
    auto grad_out = Tensor::from_cpu(backend, {N, D}, DType::F32, gh.data());
    nn::CounterStateLinear layer(backend, D, D, C, 0.003f, lr_scale);
    Peaks p{};
    const nn::FusedWorkspace policies[2] = {nn::FusedWorkspace::Small, nn::FusedWorkspace::Full};
    for (int k = 0; k < 2; ++k) {
        backend.release_workspace();
        clear_memory_pool();
        device_bytes_reset_peak();
        const std::size_t base = device_bytes_current();
        layer.set_fused_workspace(policies[k]);
        layer.apply_update_backward(grad_out, x, 7u + k);
        layer.check_fused_update();
        (k == 0 ? p.small_ws : p.full_ws) = device_bytes_peak() - base;
    }
    backend.release_workspace();
    clear_memory_pool();
    device_bytes_reset_peak();
    std::size_t base = device_bytes_current();
    { auto gw = matmul_transpose_a(grad_out, x); layer.apply_update_seed(gw, 9u); }
    backend.finish();
    p.dense = device_bytes_peak() - base;

    clear_memory_pool();
    device_bytes_reset_peak();
    base = device_bytes_current();
    auto gx = layer.backward_input_from_state(grad_out);
    backend.finish();
    p.grad_x = device_bytes_peak() - base;
    const auto w = layer.decode_weight().to_vector<float>();
    const auto got = gx.to_vector<float>();
    double num = 0.0, den = 0.0;
    for (int r = 0; r < N; ++r)
        for (int i = 0; i < D; ++i) {
            double ref = 0.0;
            for (int o = 0; o < D; ++o) ref += (double)gh[(std::size_t)r * D + o] * (double)w[(std::size_t)o * D + i];
            const double d = (double)got[(std::size_t)r * D + i] - ref;
            num += d * d;
            den += ref * ref;
        }
    p.grad_x_relerr = den > 0.0 ? std::sqrt(num / den) : 0.0;
    return p;
}

}  // namespace

int main() {
    return host_test::run("test_memory_gate", [](Backend& backend) {
        const struct { int D, N; float lr_scale; } cases[] = {{256, 64, 0.0f}, {256, 64, 0.05f}, {288, 64, 0.05f},
                                                             {2048, 64, 0.0f}, {2048, 64, 0.05f}};
        for (const auto& c : cases) {
            const Peaks p = measure(backend, c.D, c.N, c.lr_scale);
            const std::size_t weight = (std::size_t)c.D * c.D * sizeof(float);
            std::cout << "D=" << c.D << " lr_scale=" << c.lr_scale << ": weight gradient " << weight
                      << " B; cold fused update, small workspace " << p.small_ws << " B, full workspace " << p.full_ws
                      << " B; dense path " << p.dense << " B; grad_x " << p.grad_x << " B, relerr " << p.grad_x_relerr
                      << "\n";
            if (p.small_ws >= weight / 4) throw std::runtime_error("fused update created a weight-sized buffer");
            if (p.full_ws < weight) throw std::runtime_error("full policy did not allocate its f32[out,in] workspace");
            if (p.dense < weight / 2) throw std::runtime_error("dense path did not allocate a weight-sized buffer");
            if (p.grad_x >= weight / 2) throw std::runtime_error("grad_x allocated a weight-sized buffer");
            if (p.grad_x_relerr > 1e-4) throw std::runtime_error("in-kernel grad_x parity failed");
        }

        // two layers, one workspace: a strip step whose waits give up, then another layer's step
        const int N = 32;
        nn::CounterStateLinear wide(backend, 4096, 256, 11, 0.003f), other(backend, 256, 256, 11, 0.003f);
        wide.set_fused_workspace(nn::FusedWorkspace::Small);
        std::vector<float> xw((std::size_t)N * 4096), gw((std::size_t)N * 256), xo((std::size_t)N * 256);
        host_test::fill_normal(xw, 31u, 1.0f);
        host_test::fill_normal(gw, 32u, 0.01f);
        host_test::fill_normal(xo, 33u, 1.0f);
        auto x_wide = Tensor::from_cpu(backend, {N, 4096}, DType::F32, xw.data());
        auto g_both = Tensor::from_cpu(backend, {N, 256}, DType::F32, gw.data());
        auto x_other = Tensor::from_cpu(backend, {N, 256}, DType::F32, xo.data());
        mcc_compact_counter_fused_strip_set_spin_limit(1);
        wide.apply_update_backward(g_both, x_wide, 1u);
        backend.finish();
        mcc_compact_counter_fused_strip_set_spin_limit(0);
        other.apply_update_backward(g_both, x_other, 2u);  // full workspace over the same memory
        bool reported = false;
        try {
            wide.check_fused_update();
        } catch (const Error& e) {
            reported = std::string(e.what()).find("gave up waiting") != std::string::npos;
        }
        if (!reported) throw std::runtime_error("a given-up strip step went unreported after another layer's step");
        wide.check_fused_update();  // cleared by the report
        wide.apply_update_backward(g_both, x_wide, 3u);
        wide.check_fused_update();
    });
}
