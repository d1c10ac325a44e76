// Elementwise op functors, selected at compile time by opNum.
//
// Semantics follow the reference functors simdOps::* (include/ops/ops.h) and the opNum tables of
// include/loops/legacy_ops.h: TRANSFORM_OPS (49-141), PAIRWISE_TRANSFORM_OPS (243-283), BROADCAST_OPS
// (20-44).  C is the compute type (float for fp32 and fp16 storage, double for fp64); P is the lazily
// read extraParams view.  Ops whose reference functor is a whole-array routine (requiresSpecial:
// im2col, softmax, pooling ...) and the two unseeded dropout transforms have no entry: valid == false
// makes the dispatcher report them.
#pragma once

#include "math.cuh"
#include "types.h"

namespace nd4j_amd {

// simdOps::MatchCondition::op and the CompareAndSet family share this mode table (ops.h:1557-1590).
template <typename C>
__device__ __forceinline__ bool matchMode(int mode, C v, C compare, C eps, bool &known) {
    known = true;
    switch (mode) {
        case 0: return m::abs_(v - compare) <= eps;
        case 1: return m::abs_(v - compare) > eps;
        case 2: return v < compare;
        case 3: return v > compare;
        case 4: return v <= compare;
        case 5: return v >= compare;
        case 6: return m::abs_(v) < compare;
        case 7: return m::abs_(v) > compare;
        case 8: return m::isinf_(v);
        case 9: return m::isnan_(v);
        case 10: return v == compare;
        case 11: return v != compare;
        case 12: return m::abs_(v) >= compare;
        case 13: return m::abs_(v) <= compare;
        default: known = false; return false;
    }
}

// MatchCondition::op: 1/0 by mode extra[2] against extra[0] with eps extra[1]; an unknown mode returns
// the input (ops.h:1591-1594).
template <typename C, typename P>
__device__ __forceinline__ C matchConditionOp(C d1, P p) {
    bool known;
    bool r = matchMode<C>((int)p[2], d1, p[0], p[1], known);
    if (!known) return d1;
    return r ? (C)1 : (C)0;
}

// ------------------------------------------------------------------------------------------------
template <int OP> struct TransformOp { static constexpr bool valid = false; };

#define ND4J_TRANSFORM(OP, NAME, BODY)                                                   \
    template <> struct TransformOp<OP> {                                                 \
        static constexpr bool valid = true;                                              \
        static constexpr const char *name = #NAME;                                       \
        template <typename C, typename P> static __device__ __forceinline__ C op(C d1, P p) { BODY } \
    };

ND4J_TRANSFORM(0, Abs, return m::abs_(d1);)
ND4J_TRANSFORM(1, Ceiling, return m::ceil_(d1);)
ND4J_TRANSFORM(2, Cosine, return m::cos_(d1);)
ND4J_TRANSFORM(3, Exp, return m::exp_(d1);)
ND4J_TRANSFORM(4, Floor, return m::floor_(d1);)
ND4J_TRANSFORM(5, Log, return m::logNear_(d1);)
ND4J_TRANSFORM(6, Neg, return -d1;)
ND4J_TRANSFORM(7, Pow, return m::pow_(d1, p[0]);)
ND4J_TRANSFORM(8, Round, return m::round_(d1);)
ND4J_TRANSFORM(9, SetRange, {
    C mn = p[0];
    C mx = p[1];
    if (d1 >= mn && d1 <= mx) return d1;
    if (mn == (C)0 && mx == (C)1) {
        C val = (C)1 / ((C)1 + m::exp_(-d1));
        return m::floor_(val * (mx - mn)) + mn;
    }
    return m::floor_(d1 * (mx - mn)) + mn;
})
ND4J_TRANSFORM(10, Sigmoid, return m::sigmoid_(d1);)
ND4J_TRANSFORM(11, Sign, return (C)((d1 > (C)0) - (d1 < (C)0));)
ND4J_TRANSFORM(12, Sin, return m::sin_(d1);)
// (the logarithm of these is the Log transform's routine, at most 1 ULP from logf on the same argument; exp stays the replay)
ND4J_TRANSFORM(13, SoftPlus, return m::logNear_((C)1 + m::exp_(d1));)
ND4J_TRANSFORM(14, Sqrt, return m::sqrt_(d1);)
ND4J_TRANSFORM(15, Tanh, return m::tanhNear_(d1);)
ND4J_TRANSFORM(16, ACos, return m::acos_(d1);)
ND4J_TRANSFORM(17, ASin, return m::asin_(d1);)
ND4J_TRANSFORM(18, ATan, return m::atan_(d1);)
ND4J_TRANSFORM(19, HardTanh, {
    if (d1 < (C)-1) return (C)-1;
    if (d1 > (C)1) return (C)1;
    return d1;
})
ND4J_TRANSFORM(20, SoftSign, return d1 / ((C)1 + m::abs_(d1));)
ND4J_TRANSFORM(21, ELU, {
    if (d1 >= (C)0) return d1;
    return m::exp_(d1) - (C)1;
})
ND4J_TRANSFORM(22, ELUDerivative, {
    if (d1 >= (C)0) return (C)1;
    return m::exp_(d1);
})
ND4J_TRANSFORM(23, TanhDerivative, {
    // the C library's tanhf bit for bit, not the cheaper tanhNear_: near saturation one ULP of tanh is many of 1 - tanh^2
    C t = m::tanh_(d1);
    return (C)1 - t * t;
})
ND4J_TRANSFORM(24, TimesOneMinus, return d1 * ((C)1 - d1);)
ND4J_TRANSFORM(25, HardTanhDerivative, return (d1 >= (C)-1 && d1 <= (C)1) ? (C)1 : (C)0;)
ND4J_TRANSFORM(26, Ones, return (C)1;)
ND4J_TRANSFORM(27, Identity, return d1;)
ND4J_TRANSFORM(28, Stabilize, {
    // MIN_CUTFOFF = -3.79297773665f (ops.h:24)
    C k = p[0];
    const C cut = (C)-3.79297773665f;
    if (d1 * k > -cut) return -cut / k;
    if (d1 * k < cut) return cut / k;
    return d1;
})
ND4J_TRANSFORM(29, SigmoidDerivative, {
    C s = m::sigmoid_(d1);
    return s * ((C)1 - s);
})
ND4J_TRANSFORM(30, SoftSignDerivative, {
    C y = (C)1 + m::abs_(d1);
    return (C)1 / (y * y);
})
ND4J_TRANSFORM(31, LeakyRELU, {
    if (d1 < (C)0) return p[0] * d1;
    return d1;
})
ND4J_TRANSFORM(32, LeakyRELUDerivative, {
    if (d1 >= (C)0) return (C)1;
    return p[0];
})
ND4J_TRANSFORM(33, RELU, {
    C c = p[0];
    return d1 < c ? c : d1;
})
ND4J_TRANSFORM(34, Step, return d1 > p[0] ? (C)1 : (C)0;)
ND4J_TRANSFORM(35, OneMinus, return (C)1 - d1;)
// The whole-array ops have a per-element op() as well, which is what the strided entry point runs for them
// (special_ops.h:361, 665, 885, 1131, 1416: identity; 1567, 1724, 1938, 2446: softplus); the shapeInfo entry point
// routes these opNums to their own routines before it gets here.
ND4J_TRANSFORM(36, Col2Im, return d1;)
ND4J_TRANSFORM(37, Im2col, return d1;)
ND4J_TRANSFORM(38, SoftMax, return m::logNear_((C)1 + m::exp_(d1));)
ND4J_TRANSFORM(39, SoftMaxDerivative, return m::logNear_((C)1 + m::exp_(d1));)
ND4J_TRANSFORM(40, LogSoftMax, return m::logNear_((C)1 + m::exp_(d1));)
ND4J_TRANSFORM(41, IsMax, return m::logNear_((C)1 + m::exp_(d1));)
ND4J_TRANSFORM(48, Histogram, return d1;)
ND4J_TRANSFORM(70, Reverse, return d1;)
ND4J_TRANSFORM(71, Pooling2D, return d1;)
ND4J_TRANSFORM(42, SpecialDerivative, return d1 * ((C)1 - d1);)
ND4J_TRANSFORM(45, CompareAndSet, {
    bool known;
    bool r = matchMode<C>((int)p[3], d1, p[0], p[2], known);
    return (known && r) ? (C)p[1] : d1;
})
ND4J_TRANSFORM(46, ReplaceNans, return m::isnan_(d1) ? (C)p[0] : d1;)
ND4J_TRANSFORM(47, StabilizeFP16, {
    if (d1 <= (C)0) return (C)0.001;
    return d1;
})
ND4J_TRANSFORM(49, Cube, return d1 * d1 * d1;)
ND4J_TRANSFORM(50, CubeDerivative, return (C)3 * d1 * d1;)
ND4J_TRANSFORM(51, HardSigmoid, return m::min_((C)1, m::max_((C)0, (C)0.2f * d1 + (C)0.5f));)
ND4J_TRANSFORM(52, HardSigmoidDerivative, return (d1 < (C)-2.5f || d1 > (C)2.5f) ? (C)0 : (C)0.2f;)
ND4J_TRANSFORM(53, RationalTanh, {
    // the four-term sum is added with the constant last, the order the reference's -fassociative-math build
    // settles on; 1 - 1/(1 + a) amplifies a last-place difference of that sum
    C dis = ((C)2 / (C)3) * d1;
    C a = ((m::abs_(dis) + m::pow_(dis, (C)2)) + (C)1.41645f * m::pow_(dis, (C)4)) + (C)1;
    C t = m::sgn_(dis) * ((C)1 - ((C)1 / a));
    return (C)1.7159f * t;
})
ND4J_TRANSFORM(54, RationalTanhDerivative, {
    C dis = ((C)2 / (C)3) * d1;
    C a = ((m::abs_(dis) + m::pow_(dis, (C)2)) + (C)1.41645f * m::pow_(dis, (C)4)) + (C)1;
    C tDeriv = ((C)1 + m::sgn_(dis) * ((C)2 * dis + (C)4 * (C)1.41645f * m::pow_(dis, (C)3))) / (a * a);
    return (C)1.7159f * ((C)2 / (C)3) * tDeriv;
})
ND4J_TRANSFORM(55, LogX, return m::log_(d1) / m::log_((C)p[0]);)
ND4J_TRANSFORM(59, Not, return d1 == p[0] ? (C)1 : (C)0;)
// (the Tanh transform's routine, within 2 ULP of the C library's tanhf: the maximum with 0 keeps that distance)
ND4J_TRANSFORM(61, RectifiedTanh, return m::max_((C)0, m::tanhNear_(d1));)
ND4J_TRANSFORM(62, RectifiedTanhDerivative, {
    if (!(d1 > (C)0)) return (C)0;
    C t = m::tanh_(d1);
    return (C)1 - t * t;
})
ND4J_TRANSFORM(63, Sinh, return m::sinh_(d1);)
ND4J_TRANSFORM(64, Cosh, return m::cosh_(d1);)
ND4J_TRANSFORM(65, Tan, return m::tan_(d1);)
ND4J_TRANSFORM(66, TanDerivative, return (C)1 / m::pow_(m::cos_(d1), (C)2);)
ND4J_TRANSFORM(67, SELU, {
    // SELU_ALPHA / SELU_LAMBDA (ops.h:47-48), each rounded to the compute type first as (T) casts do
    const C alpha = (C)1.6732632423543772848170429916717;
    const C lambda = (C)1.0507009873554804934193349852946;
    // alpha * e - alpha is evaluated as alpha * (e - 1): the reference's release flags (-fassociative-math) let
    // GCC factor it, and for small |d1| the two forms differ by far more than rounding (e - 1 is exact)
    return d1 > (C)0 ? lambda * d1 : lambda * (alpha * (m::exp_(d1) - (C)1));
})
ND4J_TRANSFORM(68, SELUDerivative, {
    const C alpha = (C)1.6732632423543772848170429916717;
    const C lambda = (C)1.0507009873554804934193349852946;
    return d1 > (C)0 ? lambda : alpha * lambda * m::exp_(d1);
})
ND4J_TRANSFORM(72, MatchCondition, return matchConditionOp<C>(d1, p);)
ND4J_TRANSFORM(73, ClipByValue, {
    C lo = p[0];
    C hi = p[1];
    if (d1 > hi) return hi;
    if (d1 < lo) return lo;
    return d1;
})
ND4J_TRANSFORM(74, Swish, return d1 * m::sigmoid_(d1);)
ND4J_TRANSFORM(75, SwishDerivative, {
    // the reference mixes in double literals here: (ex * (d1 + ex + 1.)) / pow((ex + 1.), 2)
    C ex = m::pow_((C)2.718281828459045, d1);
    double num = (double)ex * ((double)(d1 + ex) + 1.0);
    C den = m::pow_((C)((double)ex + 1.0), (C)2);
    return (C)(num / (double)den);
})
ND4J_TRANSFORM(76, RSqrt, return (C)1 / m::sqrt_(d1);)
ND4J_TRANSFORM(77, Log1p, return m::logNear_((C)1 + d1);)
ND4J_TRANSFORM(78, Erf, return m::erf_(d1);)
ND4J_TRANSFORM(79, IsInf, return m::isinf_(d1) ? (C)1 : (C)0;)
ND4J_TRANSFORM(80, IsNan, return m::isnan_(d1) ? (C)1 : (C)0;)
ND4J_TRANSFORM(81, IsFinite, return (!m::isnan_(d1) && !m::isinf_(d1)) ? (C)1 : (C)0;)
ND4J_TRANSFORM(82, ACosh, return m::acosh_(d1);)
ND4J_TRANSFORM(83, ACoshDerivative, return (C)1 / (m::sqrt_(d1 - (C)1) * m::sqrt_(d1 + (C)1));)
ND4J_TRANSFORM(84, ASinh, return m::log_(m::sqrt_(m::pow_(d1, (C)2) + (C)1) + d1);)
ND4J_TRANSFORM(85, ASinhDerivative, return (C)1 / m::sqrt_(m::pow_(d1, (C)2) + (C)1);)
ND4J_TRANSFORM(86, SinhDerivative, return m::cosh_(d1);)
ND4J_TRANSFORM(87, Rint, return m::rint_(d1);)
ND4J_TRANSFORM(88, LogSigmoid, return m::logNear_(m::sigmoid_(d1));)
ND4J_TRANSFORM(89, LogSigmoidDerivative, {
    C ex = m::pow_((C)2.718281828459045, d1);
    return (C)1 / (ex + (C)1);
})
ND4J_TRANSFORM(90, Erfc, return m::erfc_(d1);)
ND4J_TRANSFORM(91, Expm1, return m::exp_(d1) - (C)1;)
ND4J_TRANSFORM(92, PowDerivative, {
    C e = p[0];
    return e * m::pow_(d1, e - (C)1);
})
ND4J_TRANSFORM(93, ATanh, return m::atanh_(d1);)
ND4J_TRANSFORM(94, Reciprocal, return (C)1 / d1;)
ND4J_TRANSFORM(95, Sqr, return m::pow_(d1, (C)2);)
ND4J_TRANSFORM(96, RELU6, {
    C c = p[0];
    C r = d1 < c ? c : d1;
    return r < (C)6 ? r : (C)6;
})
#undef ND4J_TRANSFORM

static constexpr int kTransformOpCount = 97;

// Transforms that evaluate none of exp / log / pow in float, directly or through sigmoid and the like: their
// kernels skip loading the lookup tables of those routines.  Anything not listed loads them.
__host__ __device__ constexpr bool transformIsPlain(int op) {
    switch (op) {
        case 0: case 1: case 2: case 4: case 5: case 6: case 8: case 11: case 12: case 14: case 15: case 19: case 20: case 23: case 24:
        case 25: case 26: case 27: case 61: case 62:
        case 31: case 32: case 33: case 34: case 35: case 42: case 49: case 50: case 51: case 52: case 76: case 79:
        case 80: case 81: case 87: case 94: case 96:
            return true;
        default:
            return false;
    }
}

// ------------------------------------------------------------------------------------------------
// Two-operand functors.  `op3` is the (x, y, params) overload that pairwise calls
// (pairwise_transform.h:154-424); `op2` is the (x, y) overload that broadcast calls
// (cpu/broadcasting.cpp:102).  They differ for AMax/AMin/Axpy/And/Or/Xor (ops.h:2234-2240, 419-470).
enum BinaryKind {
    B_Add, B_Subtract, B_Multiply, B_Divide, B_ReverseDivide, B_ReverseSubtract, B_Copy, B_EqualTo,
    B_GreaterThan, B_GreaterThanOrEqual, B_LessThan, B_LessThanOrEqual, B_NotEqualTo, B_Min, B_Max,
    B_AMin, B_AMax, B_SquaredSubtract, B_FloorMod, B_FloorDiv, B_ReverseMod, B_SafeDivide, B_Mod,
    B_TruncateDiv, B_Pow, B_Epsilon, B_Axpy, B_CompareAndSet, B_CompareAndReplace, B_And, B_Or, B_Xor,
    B_Remainder, B_FMod, B_Atan2, B_RelativeError, B_BinaryRelativeError,
    B_BinaryMinimumAbsoluteRelativeError, B_PowDerivative, B_LogPoisonLoss, B_LogPoisonLossFull, B_Invalid
};

template <int KIND> struct BinaryOp;

// Two-operand functors without exp / log / pow (see transformIsPlain)
__host__ __device__ constexpr bool binaryIsPlain(int kind) {
    return kind <= B_AMax || kind == B_FloorDiv || kind == B_SafeDivide || kind == B_Axpy;
}

#define ND4J_BINARY(KIND, BODY3, BODY2)                                                                   \
    template <> struct BinaryOp<KIND> {                                                                   \
        template <typename C, typename P> static __device__ __forceinline__ C op3(C d1, C d2, P p) { BODY3 } \
        template <typename C> static __device__ __forceinline__ C op2(C d1, C d2) { BODY2 }               \
    };
#define ND4J_BINARY_SAME(KIND, BODY) ND4J_BINARY(KIND, BODY, BODY)

ND4J_BINARY_SAME(B_Add, return d1 + d2;)
ND4J_BINARY_SAME(B_Subtract, return d1 - d2;)
ND4J_BINARY_SAME(B_Multiply, return d1 * d2;)
ND4J_BINARY_SAME(B_Divide, return d1 / d2;)
ND4J_BINARY_SAME(B_ReverseDivide, return d2 / d1;)
ND4J_BINARY_SAME(B_ReverseSubtract, return d2 - d1;)
ND4J_BINARY_SAME(B_Copy, return d2;)
ND4J_BINARY_SAME(B_EqualTo, return (C)(d1 == d2);)
ND4J_BINARY_SAME(B_GreaterThan, return (C)(d1 > d2);)
ND4J_BINARY_SAME(B_GreaterThanOrEqual, return (C)(d1 >= d2);)
ND4J_BINARY_SAME(B_LessThan, return (C)(d1 < d2);)
ND4J_BINARY_SAME(B_LessThanOrEqual, return (C)(d1 <= d2);)
ND4J_BINARY_SAME(B_NotEqualTo, return (C)(d1 != d2);)
ND4J_BINARY_SAME(B_Min, return m::min_(d1, d2);)
ND4J_BINARY_SAME(B_Max, return m::max_(d1, d2);)
ND4J_BINARY(B_AMin, return m::min_(m::abs_(d1), m::abs_(d2));, return m::abs_(d1) < m::abs_(d2) ? d1 : d2;)
ND4J_BINARY(B_AMax, return m::max_(m::abs_(d1), m::abs_(d2));, return m::abs_(d1) > m::abs_(d2) ? d1 : d2;)
ND4J_BINARY_SAME(B_SquaredSubtract, return m::pow_(d1 - d2, (C)2);)
ND4J_BINARY_SAME(B_FloorMod, {
    C mm = m::fmod_(d1, d2);
    return ((d1 < (C)0) == (d2 < (C)0)) ? mm : m::fmod_(mm + d2, d2);
})
ND4J_BINARY_SAME(B_FloorDiv, return m::floor_(d1 / d2);)
// Mod / ReverseMod / TruncateDiv go through int; a zero divisor traps on the reference's CPU, here the
// result is 0.
ND4J_BINARY_SAME(B_ReverseMod, {
    int a = m::toIntX86(d2);
    int b = m::toIntX86(d1);
    if (b == 0) return (C)0;
    if (b == -1) return (C)0;
    return (C)(a % b);
})
ND4J_BINARY_SAME(B_SafeDivide, {
    if (d2 == (C)0) return (C)0;
    return d1 / d2;
})
ND4J_BINARY_SAME(B_Mod, {
    int a = m::toIntX86(d1);
    int b = m::toIntX86(d2);
    if (b == 0) return (C)0;
    if (b == -1) return (C)0;
    return (C)(a % b);
})
ND4J_BINARY_SAME(B_TruncateDiv, {
    int a = m::toIntX86(d1);
    int b = m::toIntX86(d2);
    if (b == 0) return (C)0;
    if (b == -1) return (C)(int)(0u - (unsigned)a);
    return (C)(a / b);
})
ND4J_BINARY_SAME(B_Pow, return m::pow_(d1, d2);)
ND4J_BINARY(B_Epsilon, {
    // MIN = 1e-12 (ops.h:20), compared after the (T) cast
    return m::abs_(d1 - d2) <= (C)1e-12 ? (C)1 : (C)0;
}, return d1;)
ND4J_BINARY(B_Axpy, return p[0] * d1 + d2;, return d2 + d1;)
ND4J_BINARY(B_CompareAndSet, {
    int mode = (int)p[3];
    bool known;
    // modes 12/13 test the first operand, all others the second (ops.h:3786-3797)
    C probe = (mode == 12 || mode == 13) ? d1 : d2;
    bool r = matchMode<C>(mode, probe, p[0], p[2], known);
    return (known && r) ? d2 : d1;
}, return d1;)
ND4J_BINARY(B_CompareAndReplace, {
    bool known;
    bool r = matchMode<C>((int)p[3], d1, p[0], p[2], known);
    return (known && r) ? d2 : d1;
}, return d1;)
ND4J_BINARY(B_And, {
    C comp = p[0];
    return (d1 != comp && d2 != comp) ? (C)1 : (C)0;
}, return d2 + d1;)
ND4J_BINARY(B_Or, {
    C comp = p[0];
    return (d1 != comp || d2 != comp) ? (C)1 : (C)0;
}, return d2 + d1;)
ND4J_BINARY(B_Xor, {
    C comp = p[0];
    return ((d1 == comp && d2 != comp) || (d1 != comp && d2 == comp)) ? (C)1 : (C)0;
}, return d2 + d1;)
ND4J_BINARY_SAME(B_Remainder, return m::remainder_(d1, d2);)
ND4J_BINARY_SAME(B_FMod, return m::fmod_(d1, d2);)
ND4J_BINARY(B_Atan2, return m::atan2_(d2, d1);, return m::atan2_(d2, d1);)
ND4J_BINARY_SAME(B_RelativeError, return m::re_(d1, d2);)
ND4J_BINARY(B_BinaryRelativeError, return m::re_(d1, d2) > p[0] ? (C)1 : (C)0;, return (C)0;)
ND4J_BINARY(B_BinaryMinimumAbsoluteRelativeError, {
    C thrRel = p[0];
    C thrAbs = p[1];
    return m::re_(d1, d2) > thrRel ? (m::abs_(d1 - d2) < thrAbs ? (C)0 : (C)1) : (C)0;
}, return (C)0;)
ND4J_BINARY_SAME(B_PowDerivative, return d2 * m::pow_(d1, d2 - (C)1);)
// LogPoisonLoss{,Full}: the unqualified exp / log resolve to the overload of the data type (ops.h:170-207)
ND4J_BINARY_SAME(B_LogPoisonLoss, return m::exp_(d2) - d1 * d2;)
ND4J_BINARY_SAME(B_LogPoisonLossFull, {
    const C twoPi = (C)(2.0 * 3.14159265358979323846);
    return m::exp_(d2) - d1 * d2 + (d1 * m::log_(d1) - d1 + (C)0.5 * m::log_(twoPi * d1));
})
#undef ND4J_BINARY
#undef ND4J_BINARY_SAME

// opNum -> functor kind for the two tables (legacy_ops.h:20-44 and 243-283).
__host__ __device__ constexpr int pairwiseKind(int opNum) {
    switch (opNum) {
        case 0: return B_Add;
        case 1: return B_Copy;
        case 2: return B_Divide;
        case 3: return B_EqualTo;
        case 4: return B_GreaterThan;
        case 5: return B_LessThan;
        case 6: return B_Multiply;
        case 7: return B_Pow;
        case 8: return B_ReverseSubtract;
        case 9: return B_Subtract;
        case 10: return B_Epsilon;
        case 11: return B_GreaterThanOrEqual;
        case 12: return B_LessThanOrEqual;
        case 13: return B_Max;
        case 14: return B_Min;
        case 15: return B_NotEqualTo;
        case 16: return B_Copy;  // Copy2
        case 17: return B_Axpy;
        case 18: return B_ReverseDivide;
        case 19: return B_TruncateDiv;
        case 20: return B_FloorDiv;
        case 21: return B_FloorMod;
        case 22: return B_SquaredSubtract;
        case 23: return B_ReverseMod;
        case 24: return B_SafeDivide;
        case 25: return B_Mod;
        case 26: return B_RelativeError;
        case 27: return B_BinaryRelativeError;
        case 28: return B_BinaryMinimumAbsoluteRelativeError;
        case 45: return B_CompareAndSet;
        case 46: return B_CompareAndReplace;
        case 56: return B_And;
        case 57: return B_Or;
        case 58: return B_Xor;
        case 59: return B_Remainder;
        case 60: return B_FMod;
        case 69: return B_Atan2;
        case 92: return B_PowDerivative;
        case 93: return B_LogPoisonLoss;
        case 94: return B_LogPoisonLossFull;
        default: return B_Invalid;
    }
}
static constexpr int kPairwiseOpCount = 95;

// SCALAR_OPS (include/loops/legacy_ops.h:165-189)
__host__ __device__ constexpr int scalarKind(int opNum) {
    switch (opNum) {
        case 0: return B_Add;
        case 1: return B_Subtract;
        case 2: return B_Multiply;
        case 3: return B_Divide;
        case 4: return B_ReverseDivide;
        case 5: return B_ReverseSubtract;
        case 6: return B_Max;
        case 7: return B_LessThan;
        case 8: return B_GreaterThan;
        case 9: return B_EqualTo;
        case 10: return B_LessThanOrEqual;
        case 11: return B_NotEqualTo;
        case 12: return B_Min;
        case 13: return B_Copy;
        case 14: return B_Mod;
        case 15: return B_ReverseMod;
        case 16: return B_GreaterThanOrEqual;
        case 17: return B_Remainder;
        case 18: return B_FMod;
        case 19: return B_TruncateDiv;
        case 20: return B_FloorDiv;
        case 21: return B_FloorMod;
        case 22: return B_SquaredSubtract;
        case 23: return B_SafeDivide;
        default: return B_Invalid;
    }
}

__host__ __device__ constexpr int broadcastKind(int opNum) {
    switch (opNum) {
        case 0: return B_Add;
        case 1: return B_Subtract;
        case 2: return B_Multiply;
        case 3: return B_Divide;
        case 4: return B_ReverseDivide;
        case 5: return B_ReverseSubtract;
        case 6: return B_Copy;
        case 7: return B_EqualTo;
        case 8: return B_GreaterThan;
        case 9: return B_GreaterThanOrEqual;
        case 10: return B_LessThan;
        case 11: return B_LessThanOrEqual;
        case 12: return B_NotEqualTo;
        case 13: return B_Min;
        case 14: return B_Max;
        case 15: return B_AMin;
        case 16: return B_AMax;
        case 17: return B_SquaredSubtract;
        case 18: return B_FloorMod;
        case 19: return B_FloorDiv;
        case 20: return B_ReverseMod;
        case 21: return B_SafeDivide;
        case 22: return B_Mod;
        case 23: return B_TruncateDiv;
        default: return B_Invalid;
    }
}
static constexpr int kBroadcastOpCount = 24;

}  // namespace nd4j_amd
