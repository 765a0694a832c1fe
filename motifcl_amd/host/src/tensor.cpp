#include <motifcl/tensor/tensor.hpp>

#include <motifcl/autograd/node.hpp>
#include <motifcl/core/error.hpp>
#include <motifcl/ops/matmul.hpp>
#include <motifcl/runtime/backend.hpp>

#include <motifcl_amd.h>

#include <atomic>

namespace motifcl {
namespace {
std::atomic<int> g_next_id{1};
thread_local bool g_grad_enabled = true;
}  // namespace

namespace autograd {
bool is_enabled() { return g_grad_enabled; }
void set_enabled(bool enabled) { g_grad_enabled = enabled; }
NoGradGuard::NoGradGuard() : previous_(g_grad_enabled) { g_grad_enabled = false; }
NoGradGuard::~NoGradGuard() { g_grad_enabled = previous_; }
}  // namespace autograd

Tensor::Tensor(Backend& backend, Shape shape, DType dtype, std::shared_ptr<Storage> storage) {
    impl_ = std::make_shared<TensorImpl>();
    impl_->id = g_next_id.fetch_add(1);
    impl_->backend = &backend;
    impl_->backend_lifetime = backend.lifetime_handle();
    impl_->storage = std::move(storage);
    impl_->shape = std::move(shape);
    impl_->dtype = dtype;
}

Backend& Tensor::backend() const {
    MCL_CHECK(impl_ && impl_->backend, "tensor has no backend");
    MCL_CHECK(impl_->backend_lifetime && impl_->backend_lifetime->alive, "tensor outlived its backend");
    return *impl_->backend;
}
Backend* Tensor::backend_ptr() const { return impl_ ? impl_->backend : nullptr; }
Storage& Tensor::storage() const {
    MCL_CHECK(impl_ && impl_->storage, "tensor has no storage");
    return *impl_->storage;
}
void* Tensor::data() const { return storage().hip_ptr; }
const Shape& Tensor::shape() const {
    MCL_CHECK(impl_, "invalid tensor");
    return impl_->shape;
}
DType Tensor::dtype() const {
    MCL_CHECK(impl_, "invalid tensor");
    return impl_->dtype;
}
int Tensor::id() const { return impl_ ? impl_->id : 0; }

bool Tensor::requires_grad() const { return impl_ && impl_->requires_grad; }
void Tensor::set_requires_grad(bool value) {
    MCL_CHECK(impl_, "invalid tensor");
    impl_->requires_grad = value;
}
std::shared_ptr<Tensor> Tensor::grad() const { return impl_ ? impl_->grad : nullptr; }
void Tensor::zero_grad() {
    if (impl_) impl_->grad = nullptr;
}
void Tensor::_set_grad_fn(std::shared_ptr<autograd::Node> node) {
    MCL_CHECK(impl_, "invalid tensor");
    impl_->grad_fn = std::move(node);
}
std::shared_ptr<autograd::Node> Tensor::_grad_fn() const { return impl_ ? impl_->grad_fn : nullptr; }

void Tensor::_accumulate_grad(const Tensor& grad) {
    MCL_CHECK(impl_, "invalid tensor");
    // a leaf keeps the last gradient it was given; summing gradients of a tensor that feeds
    // several consumers is outside what a stack of counter layers needs
    MCL_CHECK(!impl_->grad, "gradient accumulation over several consumers is not supported");
    impl_->grad = std::make_shared<Tensor>(grad);
}

void Tensor::backward(const Tensor& grad_output) {
    MCL_CHECK(impl_, "invalid tensor");
    MCL_CHECK(grad_output.shape() == shape(), "backward: gradient shape mismatch");
    if (impl_->grad_fn) {
        // the node is consumed by its backward pass, as the reference's engine visits it once
        std::shared_ptr<autograd::Node> node = std::move(impl_->grad_fn);
        impl_->grad_fn = nullptr;
        autograd::NoGradGuard guard;
        node->backward(grad_output);
    } else if (impl_->requires_grad) {
        _accumulate_grad(grad_output);
    }
}

void Tensor::to_cpu(void* out, std::size_t bytes) const {
    const std::size_t n = bytes ? bytes : nbytes();
    MCL_CHECK(n <= nbytes(), "to_cpu: destination larger than the tensor");
    MCL_CHECK(mcc_memcpy_d2h(backend().hip_stream(), out, data(), n) == MCC_OK,
              std::string("device-to-host copy failed: ") + mcc_last_error());
}

Tensor Tensor::empty(Backend& backend, const Shape& shape, DType dtype) {
    const std::size_t bytes = dtype_storage_nbytes(dtype, static_cast<std::size_t>(shape.numel()));
    return Tensor(backend, shape, dtype, std::make_shared<Storage>(backend, bytes));
}

Tensor Tensor::from_cpu(Backend& backend, const Shape& shape, DType dtype, const void* data) {
    Tensor t = empty(backend, shape, dtype);
    MCL_CHECK(mcc_memcpy_h2d(backend.hip_stream(), t.data(), data, t.nbytes()) == MCC_OK,
              std::string("host-to-device copy failed: ") + mcc_last_error());
    return t;
}

Tensor Tensor::zeros(Backend& backend, const Shape& shape, DType dtype) {
    Tensor t = empty(backend, shape, dtype);
    MCL_CHECK(mcc_memset_zero(backend.hip_stream(), t.data(), t.nbytes()) == MCC_OK,
              std::string("device memset failed: ") + mcc_last_error());
    return t;
}

Tensor matmul_transpose_a(const Tensor& a, const Tensor& b) {
    MCL_CHECK(a.dtype() == DType::F32 && b.dtype() == DType::F32 && a.ndim() == 2 && b.ndim() == 2,
              "matmul_transpose_a expects rank-2 f32 tensors");
    MCL_CHECK(a.shape()[0] == b.shape()[0], "matmul_transpose_a: leading dimensions differ");
    Backend& backend = a.backend();
    Tensor c = Tensor::empty(backend, {a.shape()[1], b.shape()[1]}, DType::F32);
    const int rc = mcc_matmul_transpose_a_f32(backend.hip_stream(), static_cast<const float*>(a.data()), a.nbytes(),
                                              static_cast<const float*>(b.data()), b.nbytes(),
                                              static_cast<float*>(c.data()), c.nbytes(),
                                              static_cast<std::size_t>(a.shape()[0]), static_cast<std::size_t>(a.shape()[1]),
                                              static_cast<std::size_t>(b.shape()[1]));
    MCL_CHECK(rc == MCC_OK, std::string("matmul_transpose_a failed: ") + mcc_last_error());
    return c;
}

}  // namespace motifcl
