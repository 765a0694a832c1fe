// Helpers shared by the host-mirror tests: exit code 77 = skipped (no GPU), as MotifCL's
// CTest convention (tests/CMakeLists.txt:62-70).
#pragma once

#include <cmath>
#include <cstdint>
#include <iostream>
#include <stdexcept>
#include <string>
#include <vector>

#include <motifcl/motifcl.hpp>

namespace host_test {

// Deterministic filler used by the reference's Vulkan tests (tests/vulkan_p0_test_utils.hpp:51-60):
// a 32-bit LCG, 16 bits of each state mapped to [-scale, scale].
inline void fill_deterministic(std::vector<float>& values, std::uint32_t seed, float scale) {
    std::uint32_t s = seed;
    for (float& v : values) {
        s = s * 1664525u + 1013904223u;
        v = (static_cast<float>((s >> 8) & 0xffffu) / 32767.5f - 1.0f) * scale;
    }
}

// Counter-based generator of this build: lowbias32 of the index and the stream, 24 bits to a
// uniform in (0, 1), Box-Muller for normals.  The same values on every host and standard library
// (std::normal_distribution and std::uniform_int_distribution are implementation-defined).
inline std::uint32_t mix32(std::uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}
inline float uniform_open(std::uint32_t stream, std::uint32_t index) {
    return (static_cast<float>(mix32(index ^ mix32(stream)) >> 8) + 0.5f) * (1.0f / 16777216.0f);
}
inline float normal_at(std::uint32_t stream, std::uint32_t index) {
    const float u1 = uniform_open(stream, 2u * index), u2 = uniform_open(stream, 2u * index + 1u);
    return std::sqrt(-2.0f * std::log(u1)) * std::cos(6.28318530717958647692f * u2);
}
inline void fill_normal(std::vector<float>& values, std::uint32_t stream, float sigma) {
    for (std::size_t i = 0; i < values.size(); ++i) values[i] = sigma * normal_at(stream, static_cast<std::uint32_t>(i));
}
inline int ternary_at(std::uint32_t stream, std::uint32_t index) {
    return static_cast<int>(mix32(index ^ mix32(stream)) % 3u) - 1;
}

template <typename T>
void require_exact(const std::vector<T>& actual, const std::vector<T>& expected, const std::string& label) {
    if (actual != expected) throw std::runtime_error(label + " exact mismatch");
}

inline void require_close(const std::vector<float>& actual, const std::vector<float>& expected, float tol,
                          const std::string& label) {
    if (actual.size() != expected.size()) throw std::runtime_error(label + " size mismatch");
    float worst = 0.0f;
    for (std::size_t i = 0; i < actual.size(); ++i) worst = std::fmax(worst, std::fabs(actual[i] - expected[i]));
    if (!std::isfinite(worst) || worst > tol)
        throw std::runtime_error(label + " max error " + std::to_string(worst) + " exceeds " + std::to_string(tol));
}

// Runs `body` on a fresh HIP backend; 77 when no device is present.
template <typename F>
int run(const char* name, F body) {
    try {
        motifcl::Backend backend = motifcl::Backend::create_hip();
        body(backend);
        std::cout << "PASS " << name << " on " << backend.device_info().name << '\n';
        return 0;
    } catch (const motifcl::Error& e) {
        if (std::string(e.what()).find("no HIP device") != std::string::npos) {
            std::cout << "SKIP " << name << ": " << e.what() << '\n';
            return 77;
        }
        std::cerr << "FAIL " << name << ": " << e.what() << '\n';
        return 1;
    } catch (const std::exception& e) {
        std::cerr << "FAIL " << name << ": " << e.what() << '\n';
        return 1;
    }
}

}  // namespace host_test
