// Activation functors shared by the streaming kernels and the GEMM epilogues.
#pragma once

#include "device_common.h"

namespace cubert {

// GELU in its erf form, x * Phi(x) with Phi(x) = 0.5 * (1 + erf(x / sqrt 2))  (reference: op/GELU.cpp:13),
// written as  relu(x) - |x| * h(|x|),  h(t) = 0.5 * erfc(t / sqrt 2)  (the upper normal tail), which
// needs no sign handling and no cancellation for negative x.  A library erff costs about 35 VALU
// instructions per element, which makes this kernel instruction-bound rather than HBM-bound, so h is
// evaluated with the two classical rational approximations of erfc (Abramowitz & Stegun 7.1.26, 7.1.28)
// with 1/sqrt 2 and the factor 0.5 folded into the coefficients:
//
//  fp32 storage:  h(t) = u (a1 + u (a2 + u (a3 + u (a4 + u a5)))) exp(-t^2 / 2),  u = 1 / (1 + p t)
//                 |error of erfc| <= 1.5e-7, i.e. |error of GELU| <= 1e-7 |x|: the size of the rounding
//                 error of the reference's own fp32 formula (measured: max deviation from it 4.8e-7,
//                 about 2 ulp of the output for |x| >= 1).  12 VALU + v_rcp + v_exp per element.
//  fp16 storage:  h(t) = (c0 + c1 t + ... + c6 t^6)^-16, |error of erfc| <= 3e-7 plus fp32 rounding
//                 amplified by the 16th power (total |error of GELU| <= 7.1e-7, three orders of magnitude
//                 below fp16 resolution).  13 VALU + v_rcp per element.
struct GeluOpExp {
    __device__ __forceinline__ float operator()(float x) const {
        const float t = fabsf(x);
        const float u = __builtin_amdgcn_rcpf(fmaf(t, 0.23164189f, 1.0f));  // p / sqrt 2
        float poly = 0.5307027145f;                              // a5 / 2
        poly = fmaf(poly, u, -0.7265760135f);                    // a4 / 2
        poly = fmaf(poly, u, 0.7107068705f);                     // a3 / 2
        poly = fmaf(poly, u, -0.142248368f);                     // a2 / 2
        poly = fmaf(poly, u, 0.127414796f);                      // a1 / 2
        const float e = __builtin_amdgcn_exp2f((x * x) * -0.72134752044f);  // exp(-x^2/2) = 2^(-x^2 log2(e)/2)
        const float h = (poly * u) * e;
        return fmaf(-t, h, fmaxf(x, 0.f));
    }
};
struct GeluOpPow {
    __device__ __forceinline__ float operator()(float x) const {
        const float t = fabsf(x);
        // 2^(1/16) * (1 + sum a_k (t / sqrt 2)^k)
        float p = 5.6212997e-06f;
        p = fmaf(p, t, 5.1055209e-05f);
        p = fmaf(p, t, 3.9686137e-05f);
        p = fmaf(p, t, 3.4227392e-03f);
        p = fmaf(p, t, 2.2076998e-02f);
        p = fmaf(p, t, 5.2075163e-02f);
        p = fmaf(p, t, 1.0442737824f);
        p = p * p;
        p = p * p;
        p = p * p;
        p = p * p;
        return fmaf(-t, __builtin_amdgcn_rcpf(p), fmaxf(x, 0.f));  // p may overflow to inf for huge |x|: 1/inf = 0, as wanted
    }
};
template <typename T>
struct GeluOp;
template <>
struct GeluOp<float> : GeluOpExp {};
template <>
struct GeluOp<half_t> : GeluOpPow {};

}  // namespace cubert
