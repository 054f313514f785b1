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

// 2^t in double precision for the softmax weights of the fp64 attention kernel: t is a score minus a reference
// maximum, so it is bounded above (a few units) and may be -inf. n = round(t), f = t - n in [-1/2, 1/2],
// 2^f by its Taylor series to degree 12 (remainder 1.7e-16 at |f| = 1/2), scaled by 2^n with ldexp, which
// underflows gradually and gives exactly 0 for the clamped -1100. Eighteen fp64 vector instructions where the
// library exp costs about forty; in a kernel whose MFMAs and vector instructions share issue cycles that is the
// difference that counts.
__device__ __forceinline__ double exp2_softmax(double t) {
    t = __builtin_fmax(t, -1100.0);
    const double n = __builtin_rint(t);
    const double f = t - n;
    double p = 0x1.c3bd650fc2986p-36;
    p = __builtin_fma(p, f, 0x1.e8cac7351bb25p-32);
    p = __builtin_fma(p, f, 0x1.e4cf5158b8ecap-28);
    p = __builtin_fma(p, f, 0x1.b5253d395e7c4p-24);
    p = __builtin_fma(p, f, 0x1.62c0223a5c824p-20);
    p = __builtin_fma(p, f, 0x1.ffcbfc588b0c7p-17);
    p = __builtin_fma(p, f, 0x1.430912f86c787p-13);
    p = __builtin_fma(p, f, 0x1.5d87fe78a6731p-10);
    p = __builtin_fma(p, f, 0x1.3b2ab6fba4e77p-7);
    p = __builtin_fma(p, f, 0x1.c6b08d704a0c0p-5);
    p = __builtin_fma(p, f, 0x1.ebfbdff82c58fp-3);
    p = __builtin_fma(p, f, 0x1.62e42fefa39efp-1);
    p = __builtin_fma(p, f, 1.0);
    return __builtin_ldexp(p, (int)n);
}

// exp(x) = 2^(x * log2 e) on the hardware exp2 unit. The product x * log2 e is carried in two
// pieces (t + r, with the rounding error of the multiply recovered by an FMA and the low bits of
// log2 e added), and 2^r is folded back as 1 + r ln 2, so the result stays within about 1.5 ULP
// instead of the |x| * 2^-24 relative error of a bare exp2(x * log2e). -inf (and anything below -126)
// maps to exactly 0 and NaN propagates, which the softmax special cases rely on. Results below 2^-126 flush to
// zero. Meant for arguments that are not large and positive (a value minus a maximum): where 2^t overflows the
// correction term gives NaN, not +inf.
__device__ __forceinline__ float exp_hw(float x) {
    const float kL2eHi = 1.44269502162933349609375f;  // float(log2 e)
    const float kL2eLo = 1.925963033500011e-8f;       // log2 e - float(log2 e)
    const float kLn2 = 0.693147182464599609375f;
    const float t = x * kL2eHi;
    float r = __builtin_fmaf(x, kL2eHi, -t);
    r = __builtin_fmaf(x, kL2eLo, r);
    r = (x < -126.0f) ? 0.0f : r;  // 2^t is 0 from here on; keeps t = -inf (x = -inf, or x * log2 e overflowing) out of r
    const float e = __builtin_amdgcn_exp2f(t);
    return __builtin_fmaf(e * r, kLn2, e);
}

}  // namespace fth
