// include/motifcl/autograd/node.hpp:9-25 of MotifCL: the three-method node interface and the
// thread-local enable flag.  The engine here walks one chain of nodes (Tensor::backward calls
// the node, the node calls backward on its inputs), which is all a stack of counter layers
// with the loss gradient supplied by the caller needs.
#pragma once

#include <vector>

#include <motifcl/tensor/tensor.hpp>

namespace motifcl::autograd {

class Node {
public:
    virtual ~Node() = default;
    virtual std::vector<Tensor> inputs() const { return {}; }
    virtual void backward(const Tensor& grad_output) = 0;
};

bool is_enabled();
void set_enabled(bool enabled);

class NoGradGuard {
public:
    NoGradGuard();
    ~NoGradGuard();

private:
    bool previous_ = true;
};

}  // namespace motifcl::autograd
