// Wave64 cross-lane helpers shared by the update kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mcc {

// lane l <- value of lane l + N of the same 16-lane row (DPP row_shl); lanes whose source
// falls outside the row keep their own value, which no later step of the tree reads.
template <int N>
__device__ __forceinline__ uint32_t row_from_above(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x100 + N, 0xf, 0xf, false);
}

// lg[lid] += lg[lid + s] for s = 32, 16, 8, 4, 2, 1 (kernels/compact_counter.cl:88-91): the
// same pairing and order as the reference's LDS tree.  The two steps that cross 16-lane rows
// go through the LDS crossbar, the other four are DPP operands of the add itself.
__device__ __forceinline__ float tree_sum(float a, int lane) {
    a = a + __uint_as_float((uint32_t)__builtin_amdgcn_ds_bpermute((lane + 32) << 2, (int)__float_as_uint(a)));
    a = a + __uint_as_float((uint32_t)__builtin_amdgcn_ds_bpermute((lane + 16) << 2, (int)__float_as_uint(a)));
    a = a + __uint_as_float(row_from_above<8>(__float_as_uint(a)));
    a = a + __uint_as_float(row_from_above<4>(__float_as_uint(a)));
    a = a + __uint_as_float(row_from_above<2>(__float_as_uint(a)));
    a = a + __uint_as_float(row_from_above<1>(__float_as_uint(a)));
    return __uint_as_float((uint32_t)__builtin_amdgcn_readfirstlane((int)__float_as_uint(a)));
}

}  // namespace mcc
