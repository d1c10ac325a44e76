// tanh below 1 for the Tanh transform, in a form that a host compiler builds to the same bits as the device: fused
// multiply-adds and two plain products, nothing the compiler may contract or reorder.
//   tanh(x) = x + x t R(t),  t = x^2,  R = a degree-7 fit of (tanh(x) / x - 1) / t over t in [0, 1]
// (0.01 ULP of tanh).  Over every float of magnitude below 1 the result is at most 1 ULP from the correctly rounded
// value and at most 2 ULP from the C library's tanhf (glibc 2.35, itself up to 2 ULP off there); the host test
// tests/test_host_math.py runs these lines against the library over a strided sample, or over all of them on request.
#pragma once

#if defined(__HIPCC__)
#define ND4J_TANH_POLY_FN __host__ __device__ __forceinline__
#else
#define ND4J_TANH_POLY_FN inline
#endif

namespace nd4j_amd {

// for 0 <= x < 1 (and NaN, which stays NaN)
ND4J_TANH_POLY_FN float tanhBelowOneMagnitude(float x) {
    const float t = x * x;
    float p = 1.2146954396e-04f;
    p = __builtin_fmaf(p, t, -8.4113248158e-04f);
    p = __builtin_fmaf(p, t, 3.0785864219e-03f);
    p = __builtin_fmaf(p, t, -8.5951080546e-03f);
    p = __builtin_fmaf(p, t, 2.1784728393e-02f);
    p = __builtin_fmaf(p, t, -5.3953096271e-02f);
    p = __builtin_fmaf(p, t, 1.3333199918e-01f);
    p = __builtin_fmaf(p, t, -3.3333328366e-01f);
    const float q = t * p;
    return __builtin_fmaf(x, q, x);
}
// for |x| < 1: odd, and -0 stays -0 (the sum above would make it +0)
ND4J_TANH_POLY_FN float tanhBelowOne(float x) {
    return __builtin_copysignf(tanhBelowOneMagnitude(__builtin_fabsf(x)), x);
}

}  // namespace nd4j_amd
