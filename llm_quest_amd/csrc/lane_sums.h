// Sums over aligned groups of lanes on the VALU (DPP), not through the LDS crossbar: ds_bpermute (what __shfl_xor compiles to) costs an LDS round trip
// per step of every reduction, and the recurrence kernels that use these are one dependent chain per time step.
#pragma once
#include "common.h"

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int W>
__device__ __forceinline__ float lanes_sum(float v) {  // all-reduce over aligned groups of W (4, 8 or 16) lanes
    static_assert(W == 4 || W == 8 || W == 16, "lanes_sum: 4, 8 or 16");
    if constexpr (W == 16) {
        v += dpp_f<0x128>(v);  // row_ror:8
        v += dpp_f<0x124>(v);  // row_ror:4
        v += dpp_f<0x122>(v);  // row_ror:2
        v += dpp_f<0x121>(v);  // row_ror:1
    } else {
        v += dpp_f<0xB1>(v);  // quad_perm:[1,0,3,2]
        v += dpp_f<0x4E>(v);  // quad_perm:[2,3,0,1]
        if constexpr (W == 8) v += dpp_f<0x141>(v);  // row_half_mirror: the other quad of the 8-lane group
    }
    return v;
}
