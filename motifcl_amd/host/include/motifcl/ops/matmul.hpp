// include/motifcl/ops/matmul.hpp:8 of MotifCL: the dense weight-gradient producer.
#pragma once

#include <motifcl/tensor/tensor.hpp>

namespace motifcl {

// c[m,n] = a[k,m]^T . b[k,n]
Tensor matmul_transpose_a(const Tensor& a, const Tensor& b);

}  // namespace motifcl
