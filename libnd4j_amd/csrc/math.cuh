// Device math for the op functors.
//
// The reference evaluates every op through libm: nd4j_tanh<float> is tanhf, nd4j_exp<float> is expf and
// so on (include/templatemath.h:537-1100).  To stay within 2 ULP of those float routines without
// re-deriving each of them, the float overloads evaluate the double-precision routine and round once,
// which is within 0.5 ULP of the exact value (+ a negligible double-rounding term); the functions the
// measured configurations lean on (exp, log, sin, cos, tanh) restate the C library's float algorithms
// instead.  Operations that are exact or correctly rounded in IEEE arithmetic (sqrt, floor, fmod ...)
// stay in float.
//
// Device code is compiled with -ffp-contract=off: the reference build targets plain x86-64 without
// FMA, so a*b+c there rounds twice.
#pragma once

#include <hip/hip_runtime.h>

#include "libm_float.cuh"
#include "tanh_poly.h"
#include "log_poly.h"

namespace nd4j_amd {
namespace m {

#define ND4J_VIA_DOUBLE(name, fn)                                                       \
    __device__ __forceinline__ float name(float v) { return (float)::fn((double)v); }   \
    __device__ __forceinline__ double name(double v) { return ::fn(v); }

// exp, log, sin, cos, tanh in float restate the host C library's own float algorithms (libm_float.cuh)
__device__ __forceinline__ float exp_(float v) { return lm::expf_(v); }
__device__ __forceinline__ double exp_(double v) { return ::exp(v); }
__device__ __forceinline__ float log_(float v) { return lm::logf_(v); }
__device__ __forceinline__ double log_(double v) { return ::log(v); }
__device__ __forceinline__ float tanh_(float v) { return lm::tanhf_(v); }
__device__ __forceinline__ double tanh_(double v) { return ::tanh(v); }
// tanh for the Tanh transform itself, whose results are asked to lie within 2 ULP of the C library's tanhf (which is
// itself up to 2 ULP off the correctly rounded value below 1, within 1 from there on).  Below 1: the polynomial of
// tanh_poly.h, never more than 2 ULP from the library's value over every float below 1.  From 1 on: 1 - 2 / (exp(2|x|) + 1) on the hardware's exp2 and reciprocal, at most
// 1 ULP from the library's value over all those floats.  Some 30 instructions for both, against 90 for lm::tanhf_.
__device__ __forceinline__ float tanhAboveOne_(float ax) {
    const float l2eHi = 1.44269502162933349609375f, l2eLo = 1.925963033500011e-8f, ln2 = 0.693147182464599609375f;
    const float a = 2.0f * __builtin_fminf(ax, 22.0f);  // tanhf is 1 from 22 on
    const float t = a * l2eHi;
    float r = __builtin_fmaf(a, l2eHi, -t);
    r = __builtin_fmaf(a, l2eLo, r);
    const float p = __builtin_amdgcn_exp2f(t);
    const float d = __builtin_fmaf(p, r * ln2, p) + 1.0f;  // exp(2|x|) + 1
    float q = __builtin_amdgcn_rcpf(d);
    q = __builtin_fmaf(__builtin_fmaf(-d, q, 1.0f), q, q);
    return __builtin_fmaf(-2.0f, q, 1.0f);
}
__device__ __forceinline__ float tanhNear_(float v) {
    const float ax = __builtin_fabsf(v);
    // (NaN goes the polynomial's way and stays NaN)
    return __builtin_copysignf(ax >= 1.0f ? tanhAboveOne_(ax) : tanhBelowOneMagnitude(ax), v);
}
__device__ __forceinline__ double tanhNear_(double v) { return ::tanh(v); }
// log for the Log transform itself: log_poly.h, at most 1 ULP from the C library's logf over every float (the bar is 2),
// some 25 instructions and no lookup table against the replay's 45 and its table in LDS
__device__ __forceinline__ float logNear_(float v) { return logNear(v); }
__device__ __forceinline__ double logNear_(double v) { return ::log(v); }
__device__ __forceinline__ float sin_(float v) {
    if (((lm::asU32(v) >> 20) & 0x7ff) < 0x42f) return lm::sincosCore(v, false);
    return (float)::sin((double)v);
}
__device__ __forceinline__ double sin_(double v) { return ::sin(v); }
__device__ __forceinline__ float cos_(float v) {
    if (((lm::asU32(v) >> 20) & 0x7ff) < 0x42f) return lm::sincosCore(v, true);
    return (float)::cos((double)v);
}
__device__ __forceinline__ double cos_(double v) { return ::cos(v); }

// exp for the softmax family (arguments x - max <= 0): 2^(v log2 e) on the hardware's exp2 with the product carried as a
// rounded part and its exact remainder, about 1.5 ULP.  Those ops are held to the 1e-5 of reductions (their row sums
// are re-associated anyway), and the C library's algorithm, replayed bit for bit in exp_, costs four times as many
// instructions - which is what bounded every softmax kernel.  Below -87 the result is a denormal, or zero from where
// the C library's is (-103.972): it is computed 2^64 times too large and scaled down by a multiplication, which rounds
// it into the denormal range once.  NaN stays NaN.
__device__ __forceinline__ float expSoftCore_(float v) {
    const float l2eHi = 1.44269502162933349609375f, l2eLo = 1.925963033500011e-8f, ln2 = 0.693147182464599609375f;
    const float t = v * l2eHi;
    float r = __builtin_fmaf(v, l2eHi, -t);
    r = __builtin_fmaf(v, l2eLo, r);
    const float p = __builtin_amdgcn_exp2f(t);
    return __builtin_fmaf(p, r * ln2, p);
}
__device__ __forceinline__ float expSoft_(float v) {
    const bool far = !(v >= -87.0f);
    // a branch on the whole wave (so that it stays a branch): the shifted argument and the scale for the lanes that need them
    float scale = 1.0f;
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(far) != 0ull, 0)) {
        if (far) { v += 44.3614196f; scale = 0x1p-64f; }  // 64 ln 2; NaN stays NaN, what lies below -103.972 rounds to zero below
        const float r = expSoftCore_(v) * scale;
        return (far && v < -103.972084f + 44.3614196f) ? 0.0f : r;
    }
    return expSoftCore_(v);
}
__device__ __forceinline__ double expSoft_(double v) { return ::exp(v); }
// log to go with it: the hardware's log2 (1 ULP) times ln 2; denormal arguments are scaled into the normal range first
__device__ __forceinline__ float logSoft_(float v) {
    const float ln2 = 0.693147182464599609375f;
    const bool tiny = v < 1.17549435e-38f;
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(tiny) != 0ull, 0))  // 0 -> -inf, negative -> NaN
        return (__builtin_amdgcn_logf(tiny ? v * 0x1p64f : v) - (tiny ? 64.0f : 0.0f)) * ln2;
    return __builtin_amdgcn_logf(v) * ln2;
}
__device__ __forceinline__ double logSoft_(double v) { return ::log(v); }

ND4J_VIA_DOUBLE(tan_, tan)
ND4J_VIA_DOUBLE(cosh_, cosh)
ND4J_VIA_DOUBLE(sinh_, sinh)
ND4J_VIA_DOUBLE(acos_, acos)
ND4J_VIA_DOUBLE(asin_, asin)
ND4J_VIA_DOUBLE(atan_, atan)
ND4J_VIA_DOUBLE(acosh_, acosh)
ND4J_VIA_DOUBLE(atanh_, atanh)
ND4J_VIA_DOUBLE(erf_, erf)
ND4J_VIA_DOUBLE(erfc_, erfc)
#undef ND4J_VIA_DOUBLE

__device__ __forceinline__ float pow_(float a, float b) { return lm::powf_(a, b); }
__device__ __forceinline__ double pow_(double a, double b) { return ::pow(a, b); }
__device__ __forceinline__ float atan2_(float a, float b) { return (float)::atan2((double)a, (double)b); }
__device__ __forceinline__ double atan2_(double a, double b) { return ::atan2(a, b); }

// sqrtf under -fhip-fp32-correctly-rounded-divide-sqrt is the IEEE square root (__fsqrt_rn is not: it maps to
// the native approximate instruction)
__device__ __forceinline__ float sqrt_(float v) { return sqrtf(v); }
__device__ __forceinline__ double sqrt_(double v) { return sqrt(v); }
__device__ __forceinline__ float abs_(float v) { return ::fabsf(v); }
__device__ __forceinline__ double abs_(double v) { return ::fabs(v); }
__device__ __forceinline__ float floor_(float v) { return ::floorf(v); }
__device__ __forceinline__ double floor_(double v) { return ::floor(v); }
__device__ __forceinline__ float ceil_(float v) { return ::ceilf(v); }
__device__ __forceinline__ double ceil_(double v) { return ::ceil(v); }
__device__ __forceinline__ float round_(float v) { return ::roundf(v); }
__device__ __forceinline__ double round_(double v) { return ::round(v); }
__device__ __forceinline__ float rint_(float v) { return ::rintf(v); }
__device__ __forceinline__ double rint_(double v) { return ::rint(v); }
__device__ __forceinline__ float fmod_(float a, float b) { return ::fmodf(a, b); }
__device__ __forceinline__ double fmod_(double a, double b) { return ::fmod(a, b); }
__device__ __forceinline__ float remainder_(float a, float b) { return ::remainderf(a, b); }
__device__ __forceinline__ double remainder_(double a, double b) { return ::remainder(a, b); }

template <typename C> __device__ __forceinline__ bool isnan_(C v) { return v != v; }
__device__ __forceinline__ bool isinf_(float v) { return ::fabsf(v) == __builtin_inff(); }
__device__ __forceinline__ bool isinf_(double v) { return ::fabs(v) == __builtin_inf(); }

// nd4j_max / nd4j_min (templatemath.h:447-470): plain comparisons, so NaN handling is positional.
template <typename C> __device__ __forceinline__ C max_(C a, C b) { return a > b ? a : b; }
template <typename C> __device__ __forceinline__ C min_(C a, C b) { return a < b ? a : b; }
template <typename C> __device__ __forceinline__ C sgn_(C v) { return v < (C)0 ? (C)-1 : (v > (C)0 ? (C)1 : (C)0); }

// nd4j_sigmoid (templatemath.h:147-150): 1 / (1 + exp(-x)) evaluated step by step in the compute type.
template <typename C> __device__ __forceinline__ C sigmoid_(C v) { return (C)1 / ((C)1 + exp_(-v)); }

// nd4j_re (templatemath.h): relative error |a-b| / (|a|+|b|), 0 when both are 0.
template <typename C> __device__ __forceinline__ C re_(C a, C b) {
    if (a == (C)0 && b == (C)0) return (C)0;
    return abs_(a - b) / (abs_(a) + abs_(b));
}

// (T)(int) casts as x86 performs them: out-of-range and NaN become INT_MIN (cvttss2si).
__device__ __forceinline__ int toIntX86(float v) {
    if (!(v > -2147483904.0f && v < 2147483648.0f)) return (int)0x80000000;
    return (int)v;
}
__device__ __forceinline__ int toIntX86(double v) {
    if (!(v > -2147483649.0 && v < 2147483648.0)) return (int)0x80000000;
    return (int)v;
}

}  // namespace m
}  // namespace nd4j_amd
