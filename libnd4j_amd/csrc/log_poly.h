// Natural logarithm for the Log transform, in a form that a host compiler builds to the same bits as the device: integer
// manipulation of the argument's bits, fused multiply-adds and one plain product.
//   x = 2^e m with m in [2/3, 4/3), f = m - 1 (exact), log(x) = e ln 2 + f - f^2 / 2 + f^3 Q(f),
// Q a degree-8 fit of (log1p(f) - f + f^2 / 2) / f^3 over [-1/3, 1/3] (0.02 ULP of the result).  Over every positive float,
// denormals included, the result is at most 1 ULP from the C library's logf (glibc 2.35) and from the correctly rounded
// value; tests/test_host_math.py runs these lines against the library over a strided sample, or over all of them on
// request.  Zero gives -infinity, negative arguments NaN, +infinity and NaN themselves, as logf does.
#pragma once

#if defined(__HIPCC__)
#define ND4J_LOG_POLY_FN __host__ __device__ __forceinline__
#else
#define ND4J_LOG_POLY_FN inline
#endif

namespace nd4j_amd {

ND4J_LOG_POLY_FN float logNear(float a) {
    unsigned i = __builtin_bit_cast(unsigned, a);
    float scale = 0.0f;
    if (i - 0x00800000u >= 0x7f800000u - 0x00800000u) {  // zero, denormal, negative, infinite or NaN
        if ((i << 1) == 0) return -__builtin_inff();
        if (i == 0x7f800000u) return a;
        if ((i >> 31) != 0 || (i << 1) > 0xff000000u) return __builtin_nanf("");
        a *= 0x1p23f;  // a denormal, brought into the normal range
        i = __builtin_bit_cast(unsigned, a);
        scale = -23.0f;
    }
    const int e = (int)(i - 0x3f2aaaabu) >> 23;  // 0x3f2aaaab is 2/3
    const float m = __builtin_bit_cast(float, i - ((unsigned)e << 23));
    const float f = m - 1.0f;
    const float fe = (float)e + scale;
    const float s = f * f;
    float q = 1.231396273e-01f;
    q = __builtin_fmaf(q, f, -1.286628097e-01f);
    q = __builtin_fmaf(q, f, 1.067204773e-01f);
    q = __builtin_fmaf(q, f, -1.219179481e-01f);
    q = __builtin_fmaf(q, f, 1.431193948e-01f);
    q = __builtin_fmaf(q, f, -1.667979658e-01f);
    q = __builtin_fmaf(q, f, 1.999933720e-01f);
    q = __builtin_fmaf(q, f, -2.499981672e-01f);
    q = __builtin_fmaf(q, f, 3.333333731e-01f);
    float r = __builtin_fmaf(q, f, -0.5f);
    r = __builtin_fmaf(r, s, f);
    return __builtin_fmaf(fe, 0.693147182464599609375f, r);
}

}  // namespace nd4j_amd
