// include/motifcl/ops/optim.hpp of MotifCL: the FP32 side optimizers a counter model uses for its
// embedding and norm gains (tools/train_ternary15m.cpp:374-379).  In place; same argument order.
#pragma once

#include <motifcl/tensor/tensor.hpp>

namespace motifcl {

void sgd_update(Tensor& param, const Tensor& grad, float lr);
void adam_update(Tensor& param, const Tensor& grad, Tensor& m, Tensor& v, float lr, float beta1, float beta2,
                 float eps, int step);
void adam_update_fast(Tensor& param, const Tensor& grad, Tensor& m, Tensor& v, float lr, float beta1, float beta2,
                      float eps, int step, float weight_decay = 0.0f);

}  // namespace motifcl
