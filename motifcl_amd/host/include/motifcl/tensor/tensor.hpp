// Tensor handle of the host mirror: the subset of include/motifcl/tensor/tensor.hpp:41-103 of
// MotifCL that CounterStateLinear, its autograd node and their tests use.  Same ownership:
// a Tensor is a shared handle, Storage owns the device buffer, tensors refuse work once their
// backend is gone.
#pragma once

#include <cstddef>
#include <memory>
#include <vector>

#include <motifcl/core/dtype.hpp>
#include <motifcl/core/shape.hpp>
#include <motifcl/tensor/storage.hpp>

namespace motifcl {

class Backend;
struct BackendLifetime;
namespace autograd { class Node; }

class Tensor;

struct TensorImpl {
    int id = 0;
    Backend* backend = nullptr;
    std::shared_ptr<BackendLifetime> backend_lifetime;
    std::shared_ptr<Storage> storage;
    Shape shape;
    DType dtype = DType::F32;
    bool requires_grad = false;
    std::shared_ptr<Tensor> grad;
    std::shared_ptr<autograd::Node> grad_fn;
};

class Tensor {
public:
    Tensor() = default;
    Tensor(Backend& backend, Shape shape, DType dtype, std::shared_ptr<Storage> storage);

    bool valid() const { return impl_ != nullptr; }
    Backend& backend() const;
    Backend* backend_ptr() const;
    Storage& storage() const;
    void* data() const;  // device pointer
    const Shape& shape() const;
    DType dtype() const;
    int id() const;
    int64_t ndim() const { return shape().ndim(); }
    int64_t numel() const { return shape().numel(); }
    std::size_t nbytes() const { return dtype_storage_nbytes(dtype(), static_cast<std::size_t>(numel())); }

    bool requires_grad() const;
    void set_requires_grad(bool value = true);
    std::shared_ptr<Tensor> grad() const;
    void zero_grad();
    void backward(const Tensor& grad_output);

    void to_cpu(void* out, std::size_t bytes = 0) const;

    template <typename T>
    std::vector<T> to_vector() const {
        std::vector<T> result(static_cast<std::size_t>(numel()));
        to_cpu(result.data(), result.size() * sizeof(T));
        return result;
    }

    static Tensor empty(Backend& backend, const Shape& shape, DType dtype = DType::F32);
    static Tensor from_cpu(Backend& backend, const Shape& shape, DType dtype, const void* data);
    static Tensor zeros(Backend& backend, const Shape& shape, DType dtype = DType::F32);

    void _set_grad_fn(std::shared_ptr<autograd::Node> node);
    std::shared_ptr<autograd::Node> _grad_fn() const;
    void _accumulate_grad(const Tensor& grad);

private:
    std::shared_ptr<TensorImpl> impl_;
};

}  // namespace motifcl
