// Forward formulas of the gated activations (SiLU, exact erf GELU), shared by the activation
// kernels and by the quantizer that applies the activation on load: one definition, so that the
// fused and the two-step paths round identically.
#pragma once
#include "pt_common.h"

namespace pt {

enum : int { ACT_SILU = 0, ACT_GELU = 1 };

// SiLU through the hardware exponential and reciprocal (v_exp_f32, v_rcp_f32: about one ulp each,
// far inside the 16-bit output's rounding): g * 1 / (1 + 2^(-g log2 e)). A very negative g gives
// 2^(+big) = inf, 1 / inf = 0 and -0 as the library formula does; a very positive one gives g.
template <int ACT> __device__ __forceinline__ float act_fwd(float g) {
    if constexpr (ACT == ACT_SILU)
        return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
    else
        return 0.5f * g * (1.0f + erff(g * 0.7071067811f));
}

} // namespace pt
