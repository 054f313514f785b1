// Device math shared by the row kernels and the GEMM epilogue, so that a fused epilogue and the
// separate op give the same bits.
#pragma once

#include <hip/hip_runtime.h>

namespace fth {

// erf-form GELU, (0.5 x)(1 + erf(x / sqrt 2)) (gelu_value_f32, crates/ft-kernel-cpu/src/lib.rs:
// 36966-36969), without a branch. With t = min(|x| / sqrt 2, 4):
//     erfc(t) = 2^(t Q(t)),   Q a degree-7 polynomial fitted to log2(erfc(t)) / t on [0, 4]
// (weighted so that the ABSOLUTE error of erfc is uniform: 7e-8, about one ulp of 1; beyond t = 4
// erfc < 1.6e-8 and 1 - erfc rounds to 1). The two tails are kept apart, 1 + erf = erfc(t) for
// x < 0 and 2 - erfc(t) otherwise, so the negative tail is not computed as 1 - (1 - e). Against
// erf in double precision over [-8, 8]: |gelu error| <= 4e-7 absolute, 8e-8 of |x| + 1, the same
// size as a 1-ulp erff. NaN propagates (the comparison is false for it and every later step is
// arithmetic).
// About 16 vector instructions per element where the library erff costs more than 40 and
// branches, which made the streaming GELU kernel arithmetic-bound (0.68 of the HBM peak against
// 0.76 for a plain copy of the same shape).
__device__ __forceinline__ float gelu_erf(float x) {
    const float z = x * 0.70710678118654752440f;
    const float az = __builtin_fabsf(z);
    const float t = __builtin_fminf(az, 4.0f);
    float q = -4.5356831833487377e-05f;
    q = __builtin_fmaf(q, t, 0.000445490499259904f);
    q = __builtin_fmaf(q, t, -0.0014893790939822793f);
    q = __builtin_fmaf(q, t, -0.0007747409981675446f);
    q = __builtin_fmaf(q, t, 0.028253784403204918f);
    q = __builtin_fmaf(q, t, -0.14848166704177856f);
    q = __builtin_fmaf(q, t, -0.9184163808822632f);
    q = __builtin_fmaf(q, t, -1.6279085874557495f);
    // erfc(t), in [0, 1]; exactly 0 beyond 4, where the reference's 1 + erff is exactly 0 as well
    // (so gelu(-inf) is -inf * 0 = NaN and gelu(-6) is -0, as there)
    const float e = az > 4.0f ? 0.0f : __builtin_amdgcn_exp2f(q * t);
    const float h = 0.5f * x;
    return x < 0.0f ? h * e : h * (2.0f - e);
}

}  // namespace fth
