// MCLTEN tensor files and the per-layer checkpoint of the counter trainer
// (src/serialization.cpp:21-63,121-136, tools/train_ternary15m.cpp:112-121,204-257 of MotifCL):
// the written bytes are compared with a hand-assembled file, version-1 files load, damaged files
// are refused with an Error, and a layer restored from its three files continues bit-identically
// once its seed is advanced by the number of completed updates.
#include <cstdio>
#include <fstream>
#include <iterator>

#include <unistd.h>

#include "test_util.hpp"

using namespace motifcl;

namespace {

std::vector<unsigned char> slurp(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    return std::vector<unsigned char>(std::istreambuf_iterator<char>(in), {});
}

void spit(const std::string& path, const std::vector<unsigned char>& bytes) {
    std::ofstream out(path, std::ios::binary);
    out.write(reinterpret_cast<const char*>(bytes.data()), static_cast<std::streamsize>(bytes.size()));
}

template <typename F>
void require_error(F body, const std::string& needle, const std::string& label) {
    try {
        body();
    } catch (const Error& e) {
        if (std::string(e.what()).find(needle) == std::string::npos)
            throw std::runtime_error(label + ": wrong message: " + e.what());
        return;
    }
    throw std::runtime_error(label + ": no Error raised");
}

}  // namespace

int main() {
    return host_test::run("test_checkpoint", [](Backend& backend) {
        const std::string dir = "/tmp/mcc_ckpt_" + std::to_string(::getpid());
        const std::string path = dir + "_t.mt";

        // ---- byte layout -------------------------------------------------------------------
        const std::vector<std::uint8_t> six = {0, 1, 2, 3, 4, 5};
        save_tensor(Tensor::from_cpu(backend, {6}, DType::U8, six.data()), path);
        const std::vector<unsigned char> expected = {
            'M', 'C', 'L', 'T', 'E', 'N', '2', 0,  // magic
            3, 0, 0, 0,                             // dtype U8
            1, 0, 0, 0, 0, 0, 0, 0,                 // ndim
            6, 0, 0, 0, 0, 0, 0, 0,                 // dims[0]
            6, 0, 0, 0, 0, 0, 0, 0,                 // nbytes
            0x00, 0x00, 0x80, 0x3f,                 // quant_scale = 1.0f
            0, 0, 0, 0,                             // has_quant_scales
            0xff, 0xff, 0xff, 0xff,                 // quant_scale_axis = -1
            0, 0, 0, 0, 0, 0, 0, 0,                 // quant_block_size
            0, 1, 2, 3, 4, 5};
        if (slurp(path) != expected) throw std::runtime_error("MCLTEN2 bytes differ from the stated layout");
        auto back = load_tensor(backend, path);
        if (back.dtype() != DType::U8 || back.shape() != Shape{6}) throw std::runtime_error("reloaded header differs");
        host_test::require_exact(back.to_vector<std::uint8_t>(), six, "reloaded payload");

        // an f32 matrix round trip
        std::vector<float> m(12);
        host_test::fill_deterministic(m, 7u, 2.0f);
        save_tensor(Tensor::from_cpu(backend, {3, 4}, DType::F32, m.data()), path);
        auto mb = load_tensor(backend, path);
        if (mb.shape() != Shape{3, 4} || mb.dtype() != DType::F32) throw std::runtime_error("f32 header differs");
        host_test::require_exact(mb.to_vector<float>(), m, "f32 payload");

        // ---- version 1: no quantization block ----------------------------------------------
        std::vector<unsigned char> v1 = {'M', 'C', 'L', 'T', 'E', 'N', '1', 0, 3, 0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0,
                                         3, 0, 0, 0, 0, 0, 0, 0, 3, 0, 0, 0, 0, 0, 0, 0, 9, 8, 7};
        spit(path, v1);
        host_test::require_exact(load_tensor(backend, path).to_vector<std::uint8_t>(), {9, 8, 7}, "v1 payload");

        // ---- damaged files -----------------------------------------------------------------
        auto bad = expected;
        bad[6] = '9';
        spit(path, bad);
        require_error([&] { load_tensor(backend, path); }, "magic mismatch", "bad magic");
        bad = expected;
        bad[28] = 7;  // nbytes != numel * size
        spit(path, bad);
        require_error([&] { load_tensor(backend, path); }, "does not match dtype/shape", "size mismatch");
        bad = expected;
        bad.resize(bad.size() - 2);
        spit(path, bad);
        require_error([&] { load_tensor(backend, path); }, "failed to read tensor payload", "truncated payload");
        bad = expected;
        bad[8] = 5;  // Q4_0
        spit(path, bad);
        require_error([&] { load_tensor(backend, path); }, "dtype", "quantized dtype");
        bad = expected;
        bad[40] = 1;  // has_quant_scales
        spit(path, bad);
        require_error([&] { load_tensor(backend, path); }, "quantization scales", "quant scales");
        require_error([&] { load_tensor(backend, dir + "_missing.mt"); }, "failed to open", "missing file");

        // ---- a layer saved after 3 updates and resumed ---------------------------------------
        const int in = 256, out = 128, N = 32, C = 11;
        const std::uint32_t base_seed = 4000u;
        std::vector<float> xh(N * in), gh(N * out);
        host_test::fill_deterministic(xh, 1u, 1.0f);
        host_test::fill_deterministic(gh, 2u, 0.02f);
        auto x = Tensor::from_cpu(backend, {N, in}, DType::F32, xh.data());
        auto go = Tensor::from_cpu(backend, {N, out}, DType::F32, gh.data());
        nn::CounterStateLinear a(backend, in, out, C, 0.05f, 0.0f, 1.0f, 0.9f, 1e-3f, base_seed);
        for (int s = 0; s < 3; ++s) a.apply_update_backward(go, x, a.next_seed());
        save_counter_layer(a, dir + "_l0_wq");
        for (int s = 0; s < 2; ++s) a.apply_update_backward(go, x, a.next_seed());

        nn::CounterStateLinear b(backend, in, out, C, 0.05f, 0.0f, 1.0f, 0.9f, 1e-3f, base_seed);
        load_counter_layer(b, backend, dir + "_l0_wq");
        b.set_next_seed(base_seed + 3u);
        for (int s = 0; s < 2; ++s) b.apply_update_backward(go, x, b.next_seed());
        backend.finish();
        host_test::require_exact(b.state.to_vector<std::uint8_t>(), a.state.to_vector<std::uint8_t>(), "resumed state");
        host_test::require_exact(b.scale.to_vector<float>(), a.scale.to_vector<float>(), "resumed scale");
        host_test::require_exact(b.v.to_vector<float>(), a.v.to_vector<float>(), "resumed v");

        nn::CounterStateLinear wrong(backend, in, out * 2, C);
        require_error([&] { load_counter_layer(wrong, backend, dir + "_l0_wq"); }, "does not fit the layer",
                      "shape check");

        for (const char* suffix : {"_t.mt", "_l0_wq_state.mt", "_l0_wq_scale.mt", "_l0_wq_v.mt"})
            std::remove((dir + suffix).c_str());
    });
}
