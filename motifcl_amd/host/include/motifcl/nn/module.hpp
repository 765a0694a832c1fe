// include/motifcl/nn/module.hpp:10-17 of MotifCL.
#pragma once

#include <vector>

#include <motifcl/tensor/tensor.hpp>

namespace motifcl::nn {

struct Parameter {
    Tensor value;
};

class Module {
public:
    virtual ~Module() = default;
    virtual Tensor forward(const Tensor& x) = 0;
    virtual std::vector<Parameter*> parameters() = 0;
    virtual void zero_grad() {}
};

}  // namespace motifcl::nn
