#pragma once

#include <motifcl/autograd/node.hpp>
#include <motifcl/core/dtype.hpp>
#include <motifcl/core/error.hpp>
#include <motifcl/core/shape.hpp>
#include <motifcl/nn/compact_counter.hpp>
#include <motifcl/ops/matmul.hpp>
#include <motifcl/ops/optim.hpp>
#include <motifcl/runtime/backend.hpp>
#include <motifcl/serialization.hpp>
#include <motifcl/tensor/tensor.hpp>
