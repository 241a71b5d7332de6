// Row-softmax arithmetic shared by the softmax kernels and the fused decoding attention.
#pragma once
#include "common.h"

namespace cacti {

// e / sum for 0 <= e <= 1 <= sum without the general division sequence: y approximates 1 / sum
// to within an ulp (one Newton step on v_rcp_f32), q0 = e y is within an ulp of the quotient,
// and one residual correction rounds it to the nearest float (Markstein's theorem; it holds
// for every divisor whose significand is not all ones, which is enough to agree with IEEE
// division on all but a vanishing fraction of inputs, and the f16 rounding that follows
// absorbs those).
struct RowDivide {
    float d, y;
    __device__ explicit RowDivide(float sum) : d(sum)
    {
        const float y0 = __builtin_amdgcn_rcpf(sum);
        y = __builtin_fmaf(__builtin_fmaf(-sum, y0, 1.0f), y0, y0);
    }
    __device__ float operator()(float e) const
    {
        const float q0 = e * y;
        return __builtin_fmaf(__builtin_fmaf(-q0, d, e), y, q0);
    }
};

// exp(x) for -100 <= x <= 0 (differences from a row maximum, clamped): 2^(x log2 e) with the
// product split into its nearest integer n and a remainder f = x c - n + x c_lo formed by two
// fused multiply-adds (|f| <= 1/2, error well below one ulp of the result), v_exp_f32 on f and
// a scale by 2^n.  Same scheme and constants as the device library's expf, without its range
// tests (the clamp makes them unnecessary), 7 operations instead of about 14.
__device__ __forceinline__ float exp_nonpos(float x)
{
    const float c = 0x1.715476p+0f, c_lo = 0x1.4ae0bep-26f;     // log2(e), high and low part
    const float n = __builtin_rintf(x * c);
    float f = __builtin_fmaf(x, c, -n);
    f = __builtin_fmaf(x, c_lo, f);
    return __builtin_amdgcn_ldexpf(__builtin_amdgcn_exp2f(f), (int)n);
}

}  // namespace cacti
