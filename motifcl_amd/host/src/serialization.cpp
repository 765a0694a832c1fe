// MCLTEN1/2 tensor files (src/serialization.cpp:21-63,121-136 of MotifCL); the layout is stated in
// the header.
#include <motifcl/serialization.hpp>

#include <cstdint>
#include <cstring>
#include <fstream>
#include <vector>

#include <motifcl/core/error.hpp>

namespace motifcl {
namespace {

constexpr char kMagicV1[8] = {'M', 'C', 'L', 'T', 'E', 'N', '1', '\0'};
constexpr char kMagicV2[8] = {'M', 'C', 'L', 'T', 'E', 'N', '2', '\0'};
constexpr std::uint64_t kMaxRank = 8;  // nothing on this path has more; bounds a corrupt header

template <typename T>
void put(std::ostream& out, T value) {
    out.write(reinterpret_cast<const char*>(&value), sizeof(T));
    MCL_CHECK(out.good(), "failed to write serialization stream");
}

template <typename T>
T get(std::istream& in) {
    T value{};
    in.read(reinterpret_cast<char*>(&value), sizeof(T));
    MCL_CHECK(in.good(), "failed to read serialization stream");
    return value;
}

DType checked_dtype(std::int32_t raw) {
    MCL_CHECK(raw >= 0 && raw <= static_cast<std::int32_t>(DType::U8),
              "serialized tensor has a dtype the counter path does not store (quantized formats are not supported)");
    return static_cast<DType>(raw);
}

}  // namespace

void save_tensor(const Tensor& tensor, const std::string& path) {
    std::ofstream out(path, std::ios::binary);
    MCL_CHECK(out.good(), "failed to open tensor file for write: " + path);
    out.write(kMagicV2, sizeof(kMagicV2));
    put<std::int32_t>(out, static_cast<std::int32_t>(tensor.dtype()));
    put<std::uint64_t>(out, static_cast<std::uint64_t>(tensor.shape().dims.size()));
    for (auto dim : tensor.shape().dims) put<std::int64_t>(out, static_cast<std::int64_t>(dim));
    put<std::uint64_t>(out, static_cast<std::uint64_t>(tensor.nbytes()));
    put<float>(out, 1.0f);           // quant_scale
    put<std::int32_t>(out, 0);       // has_quant_scales
    put<std::int32_t>(out, -1);      // quant_scale_axis
    put<std::int64_t>(out, 0);       // quant_block_size
    std::vector<std::uint8_t> bytes(tensor.nbytes());
    if (!bytes.empty()) tensor.to_cpu(bytes.data(), bytes.size());
    out.write(reinterpret_cast<const char*>(bytes.data()), static_cast<std::streamsize>(bytes.size()));
    MCL_CHECK(out.good(), "failed to write tensor payload");
}

Tensor load_tensor(Backend& backend, const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    MCL_CHECK(in.good(), "failed to open tensor file for read: " + path);
    char magic[8] = {};
    in.read(magic, sizeof(magic));
    MCL_CHECK(in.good(), "failed to read serialization magic");
    const bool v1 = std::memcmp(magic, kMagicV1, 8) == 0;
    const bool v2 = std::memcmp(magic, kMagicV2, 8) == 0;
    MCL_CHECK(v1 || v2, "serialization magic mismatch");
    const DType dtype = checked_dtype(get<std::int32_t>(in));
    const auto ndim = get<std::uint64_t>(in);
    MCL_CHECK(ndim <= kMaxRank, "serialized tensor rank is implausible");
    std::vector<int64_t> dims(static_cast<std::size_t>(ndim));
    for (auto& dim : dims) {
        dim = get<std::int64_t>(in);
        MCL_CHECK(dim >= 0, "serialized tensor has a negative dimension");
    }
    const auto nbytes = get<std::uint64_t>(in);
    if (v2) {
        (void)get<float>(in);  // quant_scale: meaningful for quantized dtypes only
        MCL_CHECK(get<std::int32_t>(in) == 0, "serialized tensor carries quantization scales (not supported)");
        (void)get<std::int32_t>(in);
        (void)get<std::int64_t>(in);
    }
    Shape shape(std::move(dims));
    MCL_CHECK(dtype_storage_nbytes(dtype, static_cast<std::size_t>(shape.numel())) == nbytes,
              "serialized tensor byte size does not match dtype/shape");
    std::vector<std::uint8_t> bytes(static_cast<std::size_t>(nbytes));
    if (!bytes.empty()) in.read(reinterpret_cast<char*>(bytes.data()), static_cast<std::streamsize>(bytes.size()));
    MCL_CHECK(in.good(), "failed to read tensor payload");
    return Tensor::from_cpu(backend, shape, dtype, bytes.data());
}

void save_counter_layer(const nn::CounterStateLinear& layer, const std::string& prefix) {
    save_tensor(layer.state, prefix + "_state.mt");
    save_tensor(layer.scale, prefix + "_scale.mt");
    save_tensor(layer.v, prefix + "_v.mt");
}

void load_counter_layer(nn::CounterStateLinear& layer, Backend& backend, const std::string& prefix) {
    Tensor state = load_tensor(backend, prefix + "_state.mt");
    Tensor scale = load_tensor(backend, prefix + "_scale.mt");
    Tensor v = load_tensor(backend, prefix + "_v.mt");
    const int64_t state_bytes = static_cast<int64_t>(layer.out_features()) * (layer.in_features() / 4) * 3;
    MCL_CHECK(state.dtype() == DType::U8 && state.numel() == state_bytes,
              "counter checkpoint: state does not fit the layer");
    MCL_CHECK(scale.dtype() == DType::F32 && scale.numel() == layer.out_features() && v.dtype() == DType::F32 &&
                  v.numel() == layer.out_features(),
              "counter checkpoint: scale / v do not fit the layer");
    layer.state = state;
    layer.scale = scale;
    layer.v = v;
}

}  // namespace motifcl
