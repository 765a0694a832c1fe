// src/ops/optim.cpp:17-86 of MotifCL on the HIP library: same checks, same messages.
#include <motifcl/ops/optim.hpp>

#include <string>

#include <motifcl/core/error.hpp>
#include <motifcl/runtime/backend.hpp>
#include <motifcl_amd.h>

namespace motifcl {

void sgd_update(Tensor& param, const Tensor& grad, float lr) {
    MCL_CHECK(param.dtype() == DType::F32 && grad.dtype() == DType::F32, "sgd_update supports f32 only");
    MCL_CHECK(param.shape() == grad.shape(), "sgd_update shape mismatch");
    MCL_CHECK(param.backend_ptr() == grad.backend_ptr(), "sgd_update requires tensors on the same backend");
    const int rc = mcc_sgd_update_f32(param.backend().hip_stream(), static_cast<float*>(param.data()), param.nbytes(),
                                      static_cast<const float*>(grad.data()), grad.nbytes(),
                                      static_cast<std::size_t>(param.numel()), lr);
    MCL_CHECK(rc == MCC_OK, std::string("hip sgd_update failed: ") + mcc_last_error());
}

void adam_update(Tensor& param, const Tensor& grad, Tensor& m, Tensor& v, float lr, float beta1, float beta2,
                 float eps, int step) {
    adam_update_fast(param, grad, m, v, lr, beta1, beta2, eps, step);
}

void adam_update_fast(Tensor& param, const Tensor& grad, Tensor& m, Tensor& v, float lr, float beta1, float beta2,
                      float eps, int step, float weight_decay) {
    MCL_CHECK(param.dtype() == DType::F32 && grad.dtype() == DType::F32 && m.dtype() == DType::F32 &&
                  v.dtype() == DType::F32,
              "adam_update supports f32 only");
    MCL_CHECK(param.shape() == grad.shape() && param.shape() == m.shape() && param.shape() == v.shape(),
              "adam_update shape mismatch");
    MCL_CHECK(step > 0, "adam_update step must be positive");
    const int rc = mcc_adam_update_f32(param.backend().hip_stream(), static_cast<float*>(param.data()), param.nbytes(),
                                       static_cast<const float*>(grad.data()), grad.nbytes(),
                                       static_cast<float*>(m.data()), m.nbytes(), static_cast<float*>(v.data()),
                                       v.nbytes(), static_cast<std::size_t>(param.numel()), lr, beta1, beta2, eps,
                                       step, weight_decay);
    MCL_CHECK(rc == MCC_OK, std::string("hip adam_update failed: ") + mcc_last_error());
}

}  // namespace motifcl
