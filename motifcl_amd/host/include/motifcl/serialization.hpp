// Single-tensor checkpoint files of MotifCL (include/motifcl/serialization.hpp:12-13,
// src/serialization.cpp:21-63,121-136): the on-disk form of a counter layer's state / scale / v,
// byte-compatible in both directions so that state can move between MotifCL and this build.
//
// Layout, all little-endian and unpadded:
//   char[8]  magic            "MCLTEN2\0" (written) or "MCLTEN1\0" (also read)
//   int32    dtype            F32 = 0, F16 = 1, I32 = 2, U8 = 3
//   uint64   ndim
//   int64    dims[ndim]
//   uint64   nbytes           must equal the dtype's storage size for the shape
//   -- version 2 only --
//   float    quant_scale      1.0 for unquantized tensors
//   int32    has_quant_scales 0 here; files that carry a scale tensor are refused
//   int32    quant_scale_axis -1
//   int64    quant_block_size 0
//   -- payload --
//   uint8    bytes[nbytes]
// Quantized dtypes (Q8_0 ...) are not part of the counter path and are refused on load.
#pragma once

#include <string>

#include <motifcl/nn/compact_counter.hpp>
#include <motifcl/tensor/tensor.hpp>

namespace motifcl {

void save_tensor(const Tensor& tensor, const std::string& path);
Tensor load_tensor(Backend& backend, const std::string& path);

// The three files per layer that tools/train_ternary15m.cpp:204-228,249-257 writes and reads:
// <prefix>_state.mt, <prefix>_scale.mt, <prefix>_v.mt.  Loading checks the shapes against the
// layer.  Resuming a run also needs the layer's next seed set to base + completed steps
// (tools/train_ternary15m.cpp:112-121): see CounterStateLinear::set_next_seed.
void save_counter_layer(const nn::CounterStateLinear& layer, const std::string& prefix);
void load_counter_layer(nn::CounterStateLinear& layer, Backend& backend, const std::string& prefix);

}  // namespace motifcl
