// Element types of the host mirror (include/motifcl/core/dtype.hpp:8-26 of MotifCL); only the
// types the counter path touches are storable here.
#pragma once

#include <cstddef>

namespace motifcl {

enum class DType { F32, F16, I32, U8 };

std::size_t dtype_size(DType dtype);
std::size_t dtype_storage_nbytes(DType dtype, std::size_t numel);
const char* dtype_name(DType dtype);

}  // namespace motifcl
