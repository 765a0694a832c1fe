#include <motifcl/core/dtype.hpp>
#include <motifcl/core/error.hpp>
#include <motifcl/core/shape.hpp>

namespace motifcl {

std::size_t dtype_size(DType dtype) {
    switch (dtype) {
        case DType::F32: return 4;
        case DType::F16: return 2;
        case DType::I32: return 4;
        case DType::U8: return 1;
    }
    return 0;
}

std::size_t dtype_storage_nbytes(DType dtype, std::size_t numel) { return dtype_size(dtype) * numel; }

const char* dtype_name(DType dtype) {
    switch (dtype) {
        case DType::F32: return "f32";
        case DType::F16: return "f16";
        case DType::I32: return "i32";
        case DType::U8: return "u8";
    }
    return "?";
}

int64_t Shape::numel() const {
    int64_t n = 1;
    for (int64_t d : dims) n *= d;
    return n;
}

int64_t Shape::operator[](int index) const {
    const int n = static_cast<int>(dims.size());
    const int i = index < 0 ? index + n : index;
    MCL_CHECK(i >= 0 && i < n, "shape index out of range");
    return dims[static_cast<std::size_t>(i)];
}

std::string Shape::str() const {
    std::string s = "[";
    for (std::size_t i = 0; i < dims.size(); ++i) s += (i ? ", " : "") + std::to_string(dims[i]);
    return s + "]";
}

std::vector<int64_t> contiguous_strides(const Shape& shape) {
    std::vector<int64_t> strides(shape.dims.size(), 1);
    for (int i = static_cast<int>(shape.dims.size()) - 2; i >= 0; --i)
        strides[static_cast<std::size_t>(i)] = strides[static_cast<std::size_t>(i) + 1] * shape.dims[static_cast<std::size_t>(i) + 1];
    return strides;
}

}  // namespace motifcl
