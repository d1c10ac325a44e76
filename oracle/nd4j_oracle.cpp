// TEST INFRASTRUCTURE ONLY - never linked into, loaded by or shipped with libnd4j_amd.so.
//
// CPU restatement ("port") of the reference's legacy op-execution loops, used as the parity checker of the
// HIP path and, when the compiled reference (oracle/_ref) is absent, as the timed CPU baseline.  It exports
// the same nd4j_cpu_* C interface as oracle/ref_driver.cpp.  Loop structure, branch conditions and OpenMP
// partitioning follow the reference files cited at each function; op functors follow include/ops/ops.h,
// include/ops/random_ops.h and include/ops/special_random_ops.h; math goes through the host libm exactly as
// include/templatemath.h does.  Compile with the reference's release flags (oracle/Makefile).
//
// Pinning (tests/test_oracle.py, no GPU needed): every family is checked against the golden vectors the
// reference's own tests hold (tests/golden/reference_fixtures.json), against closed forms (numpy libm /
// brute force on small inputs), and - where oracle/_ref was built - against the compiled reference on seeded
// inputs.  The RandomBuffer stream beyond the plain xoroshiro128+ fill has no golden vector in the
// reference's tests; it is pinned by vectors produced with the compiled reference
// (tests/golden/rng_stream.json, generator script beside it).
// The families added around the op loops are pinned the same way: scalar and reduce3 by vectors of and comparison
// with the compiled reference (reduce3 also by the reference's own known answers); the SoftMax family and IsMax by
// the compiled reference where its code is well defined and by float64 ground truth; flatten, concat, pullRows,
// tear, shuffle and the type conversions bit for bit by numpy and by the compiled reference; accumulate / average
// by the exact IEEE sequence in numpy (float, double) and by the reference's CPU loops within rounding.  No function
// of this file is "parity unpinned".
//
// shapeInfo / TAD decoding is shared with the product's host code (libnd4j_amd/csrc/shape_host.h, plain
// host C++ with no device dependency); that logic is pinned on its own against the reference's TadTests /
// ShapeTests fixtures and against the compiled reference (tests/test_shape_tad.py).

#include <omp.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../libnd4j_amd/csrc/shape_host.h"

using nd4j_amd::Long;
using namespace nd4j_amd;

namespace oracle {

static int gElementThreshold = 1024;  // blas/Environment.cpp:14-15
static int gTadThreshold = 8;

// ---------------------------------------------------------------------------------------------------
// fp16 storage type: every operator converts to float, computes, and rounds back (include/types/float16.h:
// 102-195 conversions, 333-476 operators).
static inline float halfToFloat(uint16_t h) {
    unsigned sign = (h >> 15) & 1, exponent = (h >> 10) & 0x1f, mantissa = (h & 0x3ff) << 13;
    if (exponent == 0x1f) {
        mantissa = mantissa ? (sign = 0, 0x7fffff) : 0;
        exponent = 0xff;
    } else if (!exponent) {
        if (mantissa) {
            unsigned msb;
            exponent = 0x71;
            do { msb = mantissa & 0x400000; mantissa <<= 1; --exponent; } while (!msb);
            mantissa &= 0x7fffff;
        }
    } else {
        exponent += 0x70;
    }
    unsigned bits = (sign << 31) | (exponent << 23) | mantissa;
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}
static inline uint16_t floatToHalf(float f) {
    unsigned x;
    std::memcpy(&x, &f, 4);
    unsigned u = x & 0x7fffffff;
    if (u > 0x7f800000) return 0x7fff;
    unsigned sign = (x >> 16) & 0x8000;
    if (u > 0x477fefff) return (uint16_t)(sign | 0x7c00);
    if (u < 0x33000001) return (uint16_t)sign;
    unsigned exponent = (u >> 23) & 0xff, mantissa = u & 0x7fffff, shift;
    if (exponent > 0x70) { shift = 13; exponent -= 0x70; }
    else { shift = 0x7e - exponent; exponent = 0; mantissa |= 0x800000; }
    unsigned lsb = 1u << shift, lsb_s1 = lsb >> 1, lsb_m1 = lsb - 1;
    unsigned remainder = mantissa & lsb_m1;
    mantissa >>= shift;
    if (remainder > lsb_s1 || (remainder == lsb_s1 && (mantissa & 1))) {
        ++mantissa;
        if (!(mantissa & 0x3ff)) { ++exponent; mantissa = 0; }
    }
    return (uint16_t)(sign | (exponent << 10) | mantissa);
}
struct half {
    uint16_t x;
    half() : x(0) {}
    half(float f) : x(floatToHalf(f)) {}
    half(double d) : x(floatToHalf((float)d)) {}
    half(int i) : x(floatToHalf((float)i)) {}
    half(long long i) : x(floatToHalf((float)i)) {}
    operator float() const { return halfToFloat(x); }
};
#define HALF_BIN(OP) \
    static inline half operator OP(half a, half b) { return half((float)a OP(float) b); }
HALF_BIN(+) HALF_BIN(-) HALF_BIN(*) HALF_BIN(/)
#undef HALF_BIN
static inline half operator-(half a) { return half(-(float)a); }
static inline half &operator+=(half &a, half b) { a = a + b; return a; }
#define HALF_CMP(OP) static inline bool operator OP(half a, half b) { return (float)a OP(float) b; }
HALF_CMP(<) HALF_CMP(>) HALF_CMP(<=) HALF_CMP(>=) HALF_CMP(==) HALF_CMP(!=)
#undef HALF_CMP

// ---------------------------------------------------------------------------------------------------
// math: include/templatemath.h - float goes to the float libm routine, double to the double one, half
// converts to float and back.
template <typename T> struct M;
template <> struct M<float> {
    typedef float C;
    static float up(float v) { return v; }
};
template <> struct M<double> {
    typedef double C;
    static double up(double v) { return v; }
};
template <> struct M<half> {
    typedef float C;
    static float up(half v) { return (float)v; }
};
#define UNARY(name, ff, fd)                                     \
    static inline float name(float v) { return ff(v); }         \
    static inline double name(double v) { return fd(v); }       \
    static inline half name(half v) { return half(ff((float)v)); }
UNARY(m_abs, fabsf, fabs) UNARY(m_ceil, ceilf, ceil) UNARY(m_cos, cosf, cos) UNARY(m_cosh, coshf, cosh)
UNARY(m_exp, expf, exp) UNARY(m_floor, floorf, floor) UNARY(m_log, logf, log) UNARY(m_round, roundf, round)
UNARY(m_sin, sinf, sin) UNARY(m_sinh, sinhf, sinh) UNARY(m_sqrt, sqrtf, sqrt) UNARY(m_tanh, tanhf, tanh)
UNARY(m_tan, tanf, tan) UNARY(m_acos, acosf, acos) UNARY(m_asin, asinf, asin) UNARY(m_atan, atanf, atan)
UNARY(m_acosh, acoshf, acosh) UNARY(m_atanh, atanhf, atanh) UNARY(m_erf, erff, erf) UNARY(m_erfc, erfcf, erfc)
UNARY(m_rint, rintf, rint)
#undef UNARY
#define BINARY(name, ff, fd)                                              \
    static inline float name(float a, float b) { return ff(a, b); }       \
    static inline double name(double a, double b) { return fd(a, b); }    \
    static inline half name(half a, half b) { return half(ff((float)a, (float)b)); }
BINARY(m_pow, powf, pow) BINARY(m_fmod, fmodf, fmod) BINARY(m_remainder, remainderf, remainder)
BINARY(m_atan2, atan2f, atan2)
#undef BINARY
template <typename T> static inline T m_max(T a, T b) { return a > b ? a : b; }
template <typename T> static inline T m_min(T a, T b) { return a < b ? a : b; }
static inline bool m_isnan(float v) { return v != v; }
static inline bool m_isnan(double v) { return v != v; }
static inline bool m_isnan(half v) { return v.x == 0x7fff; }
static inline bool m_isinf(float v) { return std::isinf(v); }
static inline bool m_isinf(double v) { return std::isinf(v); }
static inline bool m_isinf(half v) { return v < half(-65504.f) || v > half(65504.f); }
template <typename T> static inline T m_sigmoid(T v) { return (T)1.0 / ((T)1.0 + m_exp(-v)); }
template <typename T> static inline T m_sgn(T v) { return v < (T)0.0f ? (T)-1.0f : v > (T)0.0f ? (T)1.0f : (T)0.0f; }
template <typename T> static inline T m_re(T a, T b) {
    if (a == (T)0.0f && b == (T)0.0f) return (T)0.0f;
    return m_abs(a - b) / (m_abs(a) + m_abs(b));
}

// ---------------------------------------------------------------------------------------------------
// functors: include/ops/ops.h.  MatchCondition mode table: ops.h:1557-1594.
template <typename T> static inline T matchCondition(T d1, T *extra) {
    T compare = extra[0];
    T eps = extra[1];
    int mode = (int)(typename M<T>::C)M<T>::up(extra[2]);
    switch (mode) {
        case 0: return m_abs(d1 - compare) <= eps ? (T)1.0 : (T)0.0;
        case 1: return m_abs(d1 - compare) > eps ? (T)1.0 : (T)0.0;
        case 2: return d1 < compare ? (T)1.0 : (T)0.0;
        case 3: return d1 > compare ? (T)1.0 : (T)0.0;
        case 4: return d1 <= compare ? (T)1.0 : (T)0.0;
        case 5: return d1 >= compare ? (T)1.0 : (T)0.0;
        case 6: return m_abs(d1) < compare ? (T)1.0 : (T)0.0;
        case 7: return m_abs(d1) > compare ? (T)1.0 : (T)0.0;
        case 8: return m_isinf(d1) ? (T)1.0 : (T)0.0;
        case 9: return m_isnan(d1) ? (T)1.0 : (T)0.0;
        case 10: return d1 == compare ? (T)1.0 : (T)0.0;
        case 11: return d1 != compare ? (T)1.0 : (T)0.0;
        case 12: return m_abs(d1) >= compare ? (T)1.0 : (T)0.0;
        case 13: return m_abs(d1) <= compare ? (T)1.0 : (T)0.0;
        default: printf("Undefined match condition: [%i]\n", mode);
    }
    return d1;
}
// CompareAndSet / CompareAndReplace condition (ops.h:3563-3840): true when `probe` satisfies mode
template <typename T> static inline bool compareMode(int mode, T probe, T compare, T eps, bool &known) {
    known = true;
    switch (mode) {
        case 0: return m_abs(probe - compare) <= eps;
        case 1: return m_abs(probe - compare) > eps;
        case 2: return probe < compare;
        case 3: return probe > compare;
        case 4: return probe <= compare;
        case 5: return probe >= compare;
        case 6: return m_abs(probe) < compare;
        case 7: return m_abs(probe) > compare;
        case 8: return m_isinf(probe);
        case 9: return m_isnan(probe);
        case 10: return probe == compare;
        case 11: return probe != compare;
        case 12: return m_abs(probe) >= compare;
        case 13: return m_abs(probe) <= compare;
        default: known = false; printf("Undefined boolean operation: [%i]\n", mode); return false;
    }
}
template <typename T> static inline int toInt(T v) { return (int)M<T>::up(v); }

// TRANSFORM_OPS (include/loops/legacy_ops.h:49-141); returns false for ops without a scalar functor
template <typename T> static inline bool transformOp(int op, T d1, T *p, T &out) {
    switch (op) {
        case 0: out = m_abs(d1); break;
        case 1: out = m_ceil(d1); break;
        case 2: out = m_cos(d1); break;
        case 3: out = m_exp(d1); break;
        case 4: out = m_floor(d1); break;
        case 5: out = m_log(d1); break;
        case 6: out = -d1; break;
        case 7: out = m_pow(d1, p[0]); break;
        case 8: out = m_round(d1); break;
        case 9: {
            T mn = p[0], mx = p[1];
            if (d1 >= mn && d1 <= mx) { out = d1; break; }
            if (mn == (T)0.0f && mx == (T)1.0f) {
                T val = (T)1.0f / ((T)1.0f + m_exp(-d1));
                out = m_floor(val * (mx - mn)) + mn;
                break;
            }
            out = m_floor(d1 * (mx - mn)) + mn;
            break;
        }
        case 10: out = m_sigmoid(d1); break;
        case 11: out = (T)((d1 > (T)0.0f) - (d1 < (T)0.0f)); break;
        case 12: out = m_sin(d1); break;
        case 13: out = m_log((T)1.0f + m_exp(d1)); break;
        case 14: out = m_sqrt(d1); break;
        case 15: out = m_tanh(d1); break;
        case 16: out = m_acos(d1); break;
        case 17: out = m_asin(d1); break;
        case 18: out = m_atan(d1); break;
        case 19: out = d1 < (T)-1.0 ? (T)-1.0 : (d1 > (T)1.0 ? (T)1.0 : d1); break;
        case 20: out = d1 / ((T)1.0f + m_abs(d1)); break;
        case 21: out = d1 >= (T)0.0 ? d1 : m_exp(d1) - (T)1.0; break;
        case 22: out = d1 >= (T)0.0f ? (T)1.0f : m_exp(d1); break;
        case 23: { T t = m_tanh(d1); out = (T)1.0f - t * t; break; }
        case 24: out = d1 * ((T)1.0 - d1); break;
        case 25: out = (d1 >= (T)-1.0 && d1 <= (T)1.0) ? (T)1.0 : (T)0.0; break;
        case 26: out = (T)1.0f; break;
        case 27: out = d1; break;
        case 28: {
            T k = p[0];
            const T cut = (T)-3.79297773665f;
            if (d1 * k > -cut) out = -cut / k;
            else if (d1 * k < cut) out = cut / k;
            else out = d1;
            break;
        }
        case 29: { T s = m_sigmoid(d1); out = s * ((T)1.0f - s); break; }
        case 30: { T y = (T)1.0f + m_abs(d1); out = (T)1.0f / (y * y); break; }
        case 31: out = d1 < (T)0.0f ? p[0] * d1 : d1; break;
        case 32: out = d1 >= (T)0.0f ? (T)1.0f : p[0]; break;
        case 33: out = d1 < p[0] ? p[0] : d1; break;
        case 34: out = d1 > p[0] ? (T)1.0f : (T)0.0f; break;
        case 35: out = (T)1.0f - d1; break;
        // the whole-array ops' own op(): what the strided entry point runs for them (special_ops.h:361, 665, 885,
        // 1131, 1416: identity; 1567, 1724, 1938, 2446: softplus)
        case 36: case 37: case 48: case 70: case 71: out = d1; break;
        case 38: case 39: case 40: case 41: out = m_log((T)1.0f + m_exp(d1)); break;
        case 42: out = d1 * ((T)1.0 - d1); break;
        case 45: {
            bool known;
            bool r = compareMode<T>(toInt(p[3]), d1, p[0], p[2], known);
            out = (known && r) ? p[1] : d1;
            break;
        }
        case 46: out = m_isnan(d1) ? p[0] : d1; break;
        case 47: out = d1 <= (T)0. ? (T)0.001 : d1; break;
        case 49: out = d1 * d1 * d1; break;
        case 50: out = (T)3 * d1 * d1; break;
        case 51: out = m_min((T)1.0, m_max((T)0.0f, ((T)0.2f) * d1 + (T)0.5f)); break;
        case 52: out = (d1 < (T)-2.5f || d1 > (T)2.5f) ? (T)0.0f : (T)0.2f; break;
        case 53: {
            T dis = ((T)2.0f / (T)3.0f) * d1;
            T t = m_sgn(dis) * ((T)1.0f - ((T)1.0f / ((T)1.0f + m_abs(dis) + m_pow(dis, (T)2) + (T)1.41645f * m_pow(dis, (T)4))));
            out = (T)1.7159f * t;
            break;
        }
        case 54: {
            T dis = ((T)2.0f / (T)3.0f) * d1;
            T a = (T)1.0f + m_abs(dis) + m_pow(dis, (T)2) + (T)1.41645f * m_pow(dis, (T)4);
            T tD = ((T)1.0f + m_sgn(dis) * ((T)2.0f * dis + (T)4.0f * (T)1.41645f * m_pow(dis, (T)3))) / (a * a);
            out = (T)1.7159f * ((T)2.0f / (T)3.0f) * tD;
            break;
        }
        case 55: out = m_log(d1) / m_log(p[0]); break;
        case 59: out = d1 == p[0] ? (T)1.0f : (T)0.0f; break;
        case 61: out = m_max((T)0.0f, m_tanh(d1)); break;
        case 62: { if (d1 > (T)0.0f) { T t = m_tanh(d1); out = (T)1.0f - t * t; } else out = (T)0.0f; break; }
        case 63: out = m_sinh(d1); break;
        case 64: out = m_cosh(d1); break;
        case 65: out = m_tan(d1); break;
        case 66: out = (T)1.0f / m_pow(m_cos(d1), (T)2.0f); break;
        case 67: out = d1 > (T)0.0f ? (T)1.0507009873554804934193349852946 * d1
                                   : (T)1.0507009873554804934193349852946 * ((T)1.6732632423543772848170429916717 * m_exp(d1) - (T)1.6732632423543772848170429916717);
            break;
        case 68: out = d1 > (T)0.0f ? (T)1.0507009873554804934193349852946
                                   : (T)1.6732632423543772848170429916717 * (T)1.0507009873554804934193349852946 * m_exp(d1);
            break;
        case 72: out = matchCondition<T>(d1, p); break;
        case 73: out = d1 > p[1] ? p[1] : (d1 < p[0] ? p[0] : d1); break;
        case 74: out = d1 * m_sigmoid(d1); break;
        case 75: {
            T ex = m_pow((T)M_E, d1);
            out = (T)(((double)M<T>::up(ex) * ((double)M<T>::up(d1 + ex) + 1.)) /
                      (double)M<T>::up(m_pow((T)((double)M<T>::up(ex) + 1.), (T)2.0f)));
            break;
        }
        case 76: out = (T)1.0f / m_sqrt(d1); break;
        case 77: out = m_log((T)1 + d1); break;
        case 78: out = m_erf(d1); break;
        case 79: out = m_isinf(d1) ? (T)1.0f : (T)0.0f; break;
        case 80: out = m_isnan(d1) ? (T)1.0f : (T)0.0f; break;
        case 81: out = (!m_isnan(d1) && !m_isinf(d1)) ? (T)1.0f : (T)0.0f; break;
        case 82: out = m_acosh(d1); break;
        case 83: out = (T)1.f / (m_sqrt(d1 - (T)1.f) * m_sqrt(d1 + (T)1.f)); break;
        case 84: out = m_log(m_sqrt(m_pow(d1, (T)2) + (T)1) + d1); break;
        case 85: out = (T)1.f / (m_sqrt(m_pow(d1, (T)2) + (T)1)); break;
        case 86: out = m_cosh(d1); break;
        case 87: out = m_rint(d1); break;
        case 88: out = m_log(m_sigmoid(d1)); break;
        case 89: { T ex = m_pow((T)M_E, d1); out = (T)1. / (ex + (T)1.); break; }
        case 90: out = m_erfc(d1); break;
        case 91: out = m_exp(d1) - (T)1.0f; break;
        case 92: out = p[0] * m_pow(d1, p[0] - (T)1.); break;
        case 93: out = m_atanh(d1); break;
        case 94: out = (T)1.0f / d1; break;
        case 95: out = m_pow(d1, (T)2); break;
        case 96: { T r = d1 < p[0] ? p[0] : d1; out = r < (T)6. ? r : (T)6.; break; }
        default: return false;
    }
    return true;
}

// two-operand functors by name; `three` selects the (x, y, params) overload used by pairwise, otherwise the
// (x, y) overload used by broadcast
enum Bin {
    Add, Subtract, Multiply, Divide, ReverseDivide, ReverseSubtract, Copy, EqualTo, GreaterThan, GreaterThanOrEqual,
    LessThan, LessThanOrEqual, NotEqualTo, Min, Max, AMin, AMax, SquaredSubtract, FloorMod, FloorDiv, ReverseMod,
    SafeDivide, Mod, TruncateDiv, Pow, Epsilon, Axpy, CompareAndSet, CompareAndReplace, And, Or, Xor, Remainder, FMod,
    Atan2, RelativeError, BinaryRelativeError, BinaryMinimumAbsoluteRelativeError, PowDerivative, LogPoisonLoss,
    LogPoisonLossFull, Invalid
};
static Bin pairwiseBin(int op) {
    switch (op) {
        case 0: return Add; case 1: return Copy; case 2: return Divide; case 3: return EqualTo; case 4: return GreaterThan;
        case 5: return LessThan; case 6: return Multiply; case 7: return Pow; case 8: return ReverseSubtract;
        case 9: return Subtract; case 10: return Epsilon; case 11: return GreaterThanOrEqual; case 12: return LessThanOrEqual;
        case 13: return Max; case 14: return Min; case 15: return NotEqualTo; case 16: return Copy; case 17: return Axpy;
        case 18: return ReverseDivide; case 19: return TruncateDiv; case 20: return FloorDiv; case 21: return FloorMod;
        case 22: return SquaredSubtract; case 23: return ReverseMod; case 24: return SafeDivide; case 25: return Mod;
        case 26: return RelativeError; case 27: return BinaryRelativeError; case 28: return BinaryMinimumAbsoluteRelativeError;
        case 45: return CompareAndSet; case 46: return CompareAndReplace; case 56: return And; case 57: return Or;
        case 58: return Xor; case 59: return Remainder; case 60: return FMod; case 69: return Atan2;
        case 92: return PowDerivative; case 93: return LogPoisonLoss; case 94: return LogPoisonLossFull;
        default: return Invalid;
    }
}
static Bin broadcastBin(int op) {
    static const Bin table[24] = {Add, Subtract, Multiply, Divide, ReverseDivide, ReverseSubtract, Copy, EqualTo,
                                  GreaterThan, GreaterThanOrEqual, LessThan, LessThanOrEqual, NotEqualTo, Min, Max, AMin,
                                  AMax, SquaredSubtract, FloorMod, FloorDiv, ReverseMod, SafeDivide, Mod, TruncateDiv};
    return (op >= 0 && op < 24) ? table[op] : Invalid;
}
// SCALAR_OPS: include/loops/legacy_ops.h:165-189
static Bin scalarBin(int op) {
    static const Bin table[24] = {Add, Subtract, Multiply, Divide, ReverseDivide, ReverseSubtract, Max, LessThan,
                                  GreaterThan, EqualTo, LessThanOrEqual, NotEqualTo, Min, Copy, Mod, ReverseMod,
                                  GreaterThanOrEqual, Remainder, FMod, TruncateDiv, FloorDiv, FloorMod, SquaredSubtract,
                                  SafeDivide};
    return (op >= 0 && op < 24) ? table[op] : Invalid;
}
template <typename T, bool three> static inline T binaryOp(Bin b, T d1, T d2, T *p) {
    switch (b) {
        case Add: return d1 + d2;
        case Subtract: return d1 - d2;
        case Multiply: return d1 * d2;
        case Divide: return d1 / d2;
        case ReverseDivide: return d2 / d1;
        case ReverseSubtract: return d2 - d1;
        case Copy: return d2;
        case EqualTo: return (T)(d1 == d2);
        case GreaterThan: return (T)(d1 > d2);
        case GreaterThanOrEqual: return (T)(d1 >= d2);
        case LessThan: return (T)(d1 < d2);
        case LessThanOrEqual: return (T)(d1 <= d2);
        case NotEqualTo: return (T)(d1 != d2);
        case Min: return m_min(d1, d2);
        case Max: return m_max(d1, d2);
        case AMin: return three ? m_min(m_abs(d1), m_abs(d2)) : (m_abs(d1) < m_abs(d2) ? d1 : d2);
        case AMax: return three ? m_max(m_abs(d1), m_abs(d2)) : (m_abs(d1) > m_abs(d2) ? d1 : d2);
        case SquaredSubtract: return m_pow(d1 - d2, (T)2);
        case FloorMod: {
            T mm = m_fmod(d1, d2);
            return (d1 < (T)0.0f) == (d2 < (T)0.0f) ? mm : m_fmod(mm + d2, d2);
        }
        case FloorDiv: return m_floor(d1 / d2);
        case ReverseMod: return (T)(toInt(d2) % toInt(d1));
        case SafeDivide: return d2 == (T)0. ? (T)0. : d1 / d2;
        case Mod: return (T)(toInt(d1) % toInt(d2));
        case TruncateDiv: return (T)(toInt(d1) / toInt(d2));
        case Pow: return m_pow(d1, d2);
        case Epsilon: return three ? (m_abs(d1 - d2) <= (T)1e-12 ? (T)1.0f : (T)0.0f) : d1;
        case Axpy: return three ? p[0] * d1 + d2 : d2 + d1;
        case CompareAndSet: {
            if (!three) return d1;
            int mode = toInt(p[3]);
            bool known;
            bool r = compareMode<T>(mode, (mode == 12 || mode == 13) ? d1 : d2, p[0], p[2], known);
            return (known && r) ? d2 : d1;
        }
        case CompareAndReplace: {
            if (!three) return d1;
            bool known;
            bool r = compareMode<T>(toInt(p[3]), d1, p[0], p[2], known);
            return (known && r) ? d2 : d1;
        }
        case And: return three ? ((d1 != p[0] && d2 != p[0]) ? (T)1.0f : (T)0.0f) : d2 + d1;
        case Or: return three ? ((d1 != p[0] || d2 != p[0]) ? (T)1.0f : (T)0.0f) : d2 + d1;
        case Xor: return three ? (((d1 == p[0] && d2 != p[0]) || (d1 != p[0] && d2 == p[0])) ? (T)1.0f : (T)0.0f) : d2 + d1;
        case Remainder: return m_remainder(d1, d2);
        case FMod: return m_fmod(d1, d2);
        case Atan2: return m_atan2(d2, d1);
        case RelativeError: return m_re(d1, d2);
        case BinaryRelativeError: return three ? (m_re(d1, d2) > p[0] ? (T)1.0f : (T)0.0f) : (T)0.0f;
        case BinaryMinimumAbsoluteRelativeError:
            return three ? (m_re(d1, d2) > p[0] ? (m_abs(d1 - d2) < p[1] ? (T)0.0f : (T)1.0f) : (T)0.0f) : (T)0.0f;
        case PowDerivative: return d2 * m_pow(d1, d2 - (T)1.);
        // unqualified exp / log on a float argument resolve to the float overloads (ops.h:170-207)
        case LogPoisonLoss: return m_exp(d2) - d1 * d2;
        case LogPoisonLossFull: {
            const T twoPi = T(2.0 * 3.14159265358979323846);
            return m_exp(d2) - d1 * d2 + (d1 * m_log(d1) - d1 + (T)0.5 * m_log(twoPi * d1));
        }
        default: return d1;
    }
}

// ---------------------------------------------------------------------------------------------------
// shape helpers (include/helpers/shape.h:1799-1890, 3271-3300)
static inline void ind2subC(int rank, const Long *shape, int index, Long *out) {
    int denom = (int)prodOf(shape, rank);
    for (int i = 0; i < rank; i++) {
        denom /= (int)shape[i];
        if (denom > 0) { out[i] = index / denom; index %= denom; }
        else out[i] = 0;
    }
}
static inline void ind2subF(int rank, const Long *shape, int index, Long *out) {
    int denom = (int)prodOf(shape, rank);
    for (int i = rank - 1; i >= 0; i--) {
        denom /= (int)shape[i];
        out[i] = index / denom;
        index %= denom;
    }
}
static inline Long getOffset(Long base, const Long *shape, const Long *stride, const Long *idx, int rank) {
    Long off = base;
    for (int i = 0; i < rank; i++)
        if (shape[i] != 1) off += idx[i] * stride[i];
    return off;
}
// raw iteration with dimension 0 fastest (include/pairwise_util.h:58-74): calls f(offsets...) per element
template <typename F> static inline void rawIter(int rank, const Long *shape, F f) {
    Long coord[kMaxRank];
    std::memset(coord, 0, sizeof(coord));
    if (rank == 0) { f(coord); return; }
    while (true) {
        f(coord);
        int d = 0;
        for (; d < rank; d++) {
            if (++coord[d] == shape[d]) coord[d] = 0;
            else break;
        }
        if (d == rank) break;
    }
}
static inline int clampThreads(Long work, int threshold) {
    int per = (int)(work / threshold);
    int t = per > 1 ? per : 1;
    int mx = omp_get_max_threads();
    return t < mx ? t : mx;
}
// BlockInformation (include/pairwise_util.h:236-259)
struct BlockInfo {
    Long items, chunks;
    int threads;
    BlockInfo(Long length, int threshold) {
        threads = clampThreads(length, threshold);
        items = length / threads;
        if (items < 1) items = 1;
        chunks = length / items;
        if (length % items > 0) chunks++;
    }
};

// ---------------------------------------------------------------------------------------------------
// transform: include/loops/cpu/transform.cpp:28-135
template <typename T> static void transformStrided(int op, T *x, Long xs, T *z, Long zs, T *extra, Long n) {
    T probe;
    if (n > 0 && !transformOp<T>(op, x[0], extra, probe)) { printf("[ERROR] Unknown opNum=%d (oracle transform)\n", op); return; }
    int threads = clampThreads(n, gElementThreshold);
    int span = (int)(n / threads) + 8;
#pragma omp parallel num_threads(threads) if (threads > 1)
    {
        Long tid = omp_get_thread_num();
        Long start = span * tid, end = span * (tid + 1);
        if (end > n) end = n;
        for (Long i = start; i < end; i++) transformOp<T>(op, x[i * xs], extra, z[i * zs]);
    }
}
// Whole-array special transforms (include/ops/special_ops.h): SoftMax 38 (1483-1568), SoftMaxDerivative 39
// (1806-1937), LogSoftMax 40 (1635-1726) over each row of a matrix or over a vector; IsMax 41 (1951-2260): one-hot of
// the first maximum of the whole array, or of every TAD along the dimensions listed in extraParams
// ([0] = count, [1..] = dimensions).  Restated as what the routines compute when called in place (x == z), which is
// how the reference's vector branches of 39 / 40 and the matrix branch of 39 read their input.
template <typename T> static void specialTransform(int op, T *x, Long *xi, T *z, Long *zi, T *extra) {
    const int rank = siRank(xi);
    const Long n = siNumel(xi);
    if (n <= 0) return;
    if (op != 41) {
        const bool vector = rank <= 1 || (rank == 2 && (siShape(xi)[0] == 1 || siShape(xi)[1] == 1));
        Long rows, len, xRow, xEl, zRow, zEl;
        if (vector) {
            const int xd = (rank == 2 && siShape(xi)[0] != 1) ? 0 : rank - 1;
            const int zd = (siRank(zi) == 2 && siShape(zi)[0] != 1) ? 0 : siRank(zi) - 1;
            rows = 1; len = n; xRow = zRow = 0;
            xEl = siStride(xi)[xd];
            zEl = siStride(zi)[zd];
        } else if (rank == 2) {
            rows = siShape(xi)[0]; len = siShape(xi)[1];
            xRow = siStride(xi)[0]; xEl = siStride(xi)[1];
            zRow = siStride(zi)[0]; zEl = siStride(zi)[1];
        } else {
            return;
        }
        for (Long r = 0; r < rows; r++) {
            T *xr = x + r * xRow, *zr = z + r * zRow;
            T mx = xr[0];
            for (Long c = 1; c < len; c++) mx = m_max(mx, xr[c * xEl]);
            T sum = (T)0.0f;
            for (Long c = 0; c < len; c++) { T e = m_exp(xr[c * xEl] - mx); zr[c * zEl] = e; sum += e; }
            for (Long c = 0; c < len; c++) {
                T v = zr[c * zEl] / sum;
                if (op == 39) v = v * ((T)1.0f - v);
                else if (op == 40) v = m_log(v);
                zr[c * zEl] = v;
            }
        }
        return;
    }
    int dimLen = extra == nullptr ? 0 : toInt(extra[0]);
    if (dimLen == 1 && toInt(extra[1]) == 0x7fffffff) dimLen = 0;
    if (dimLen <= 0 || dimLen >= rank) {
        // first maximum in the element order of the index reductions: memory-linear with an element-wise stride,
        // C-order coordinates otherwise
        const Long xe = siEws(xi), ze = siEws(zi);
        Long best = 0;
        T bestV = x[0];
        Long cx[kMaxRank];
        for (Long i = 0; i < n; i++) {
            Long ox;
            if (xe >= 1) ox = i * xe;
            else { ind2subC(rank, siShape(xi), (int)i, cx); ox = getOffset(0, siShape(xi), siStride(xi), cx, rank); }
            if (x[ox] > bestV) { bestV = x[ox]; best = i; }
        }
        for (Long i = 0; i < n; i++) {
            Long oz;
            if (ze >= 1) oz = i * ze;
            else { ind2subC(siRank(zi), siShape(zi), (int)i, cx); oz = getOffset(0, siShape(zi), siStride(zi), cx, siRank(zi)); }
            z[oz] = i == best ? (T)1.0f : (T)0.0f;
        }
        return;
    }
    int dims[kMaxRank];
    for (int i = 0; i < dimLen; i++) dims[i] = toInt(extra[i + 1]);
    TadPack tx, tz;
    computeTad(xi, dims, dimLen, tx, true);
    computeTad(zi, dims, dimLen, tz, true);
    const Long *xt = tx.shapeInfo.data(), *zt = tz.shapeInfo.data();
    const Long len = siNumel(xt);
    Long c[kMaxRank];
    for (Long r = 0; r < tx.numTads; r++) {
        Long best = 0;
        T bestV = (T)0.0f;
        for (Long f = 0; f < len; f++) {
            Long ox;
            if (siEws(xt) >= 1) ox = f * siEws(xt);
            else { ind2subC(siRank(xt), siShape(xt), (int)f, c); ox = getOffset(0, siShape(xt), siStride(xt), c, siRank(xt)); }
            T v = x[tx.offsets[r] + ox];
            if (f == 0 || v > bestV) { bestV = v; best = f; }
        }
        for (Long f = 0; f < len; f++) {
            Long oz;
            if (siEws(zt) >= 1) oz = f * siEws(zt);
            else { ind2subC(siRank(zt), siShape(zt), (int)f, c); oz = getOffset(0, siShape(zt), siStride(zt), c, siRank(zt)); }
            z[tz.offsets[r] + oz] = f == best ? (T)1.0f : (T)0.0f;
        }
    }
}


// ---- the other whole-array transforms (include/ops/special_ops.h) ------------------------------------------------
static inline bool inRange(int a, int b) { return (unsigned)a < (unsigned)b; }   // special_ops.h:409-411
static bool stridesDescend(const Long *info) {                                    // shape::strideDescendingCAscendingF
    const int rank = siRank(info);
    const Long *st = siStride(info);
    if (siOrder(info) == 'c') { for (int i = 1; i < rank; i++) if (st[i - 1] <= st[i]) return false; return true; }
    for (int i = 1; i < rank; i++) if (st[i - 1] >= st[i]) return false;
    return true;
}

// Reverse 70 (special_ops.h:1317-1414): the array read in its own order lands back to front.  In place: swaps for an
// element-wise stride; without one only the first half is copied onto the mirrored positions.
template <typename T> static void reverseWhole(T *x, Long *xi, T *z, Long *zi) {
    const Long n = siNumel(xi), last = n - 1;
    const Long xe = siEws(xi);
    const char xo = siOrder(xi);
    const int xr = siRank(xi);
    Long cx[kMaxRank], cz[kMaxRank];
    auto coords = [](char order, int rank, const Long *shape, Long idx, Long *c) {
        if (order == 'c') { for (int d = rank - 1; d >= 0; d--) { c[d] = idx % shape[d]; idx /= shape[d]; } }
        else { for (int d = 0; d < rank; d++) { c[d] = idx % shape[d]; idx /= shape[d]; } }
    };
    if (x == z) {
        if (xe >= 1) {
            for (Long e = 0; e < n / 2; e++) { T t = x[e * xe]; x[e * xe] = x[(last - e) * xe]; x[(last - e) * xe] = t; }
        } else {
            for (Long e = 0; e < n / 2; e++) {
                coords(xo, xr, siShape(xi), e, cx);
                coords(xo, xr, siShape(xi), last - e, cz);
                z[getOffset(0, siShape(xi), siStride(xi), cz, xr)] = x[getOffset(0, siShape(xi), siStride(xi), cx, xr)];
            }
        }
        return;
    }
    const Long ze = siEws(zi);
    const char zo = siOrder(zi);
    if (xe >= 1 && ze >= 1 && xo == zo) {
        for (Long e = 0; e < n; e++) z[(last - e) * ze] = x[e * xe];
        return;
    }
    for (Long e = 0; e < n; e++) {
        coords(xo, xr, siShape(xi), e, cx);
        coords(zo, siRank(zi), siShape(zi), last - e, cz);
        z[getOffset(0, siShape(zi), siStride(zi), cz, siRank(zi))] = x[getOffset(0, siShape(xi), siStride(xi), cx, xr)];
    }
}

// Histogram 48 (special_ops.h:811-882): extra = [numBins, min, max]; the first length(x) elements of the buffer are
// binned by (x - min) / binSize, clamped to the outer bins, and the counts are ADDED to z.  The divisor is invariant in
// the loop and the reference's release flags allow reciprocals: the compiled loop multiplies by 1 / binSize (and does
// not fold the bin count into that reciprocal, hence the barrier: this file is built with the same flags).
template <typename T> static inline T opaqueValue(T v) { asm volatile("" : "+m"(v)); return v; }
template <typename T> static void histogramWhole(T *x, Long *xi, T *z, T *extra) {
    const int length = (int)siNumel(xi);
    const int numBins = toInt(extra[0]);
    const T lo = extra[1], hi = extra[2];
    const T binSize = opaqueValue<T>((hi - lo) / (T)numBins);
    // for half the reciprocal stays in float: float16's operator/ divides two floats and rounds the quotient
    typedef typename M<T>::C C;
    const C perBin = opaqueValue<C>((C)1.0f / M<T>::up(binSize));
    std::vector<int> bins(numBins > 0 ? numBins : 0, 0);
    for (int i = 0; i < length; i++) {
        int idx = toInt((T)(M<T>::up(x[i] - lo) * perBin));
        if (idx < 0) idx = 0;
        else if (idx >= numBins) idx = numBins - 1;
        bins[idx]++;
    }
    for (int b = 0; b < numBins; b++) z[b] = (T)(M<T>::up(z[b]) + (C)bins[b]);  // T += int: the count is not rounded to T first
}

// Im2col 37 (special_ops.h:530-663): x [bS, iC, iH, iW] -> z [bS, iC, kH, kW, oH, oW]; extra = [kH, kW, sH, sW, pH, pW,
// dH, dW]; positions outside the image are zero.  When both arrays are c-order with descending strides a batch entry
// of the result is written as one dense run, whatever its inner strides say.
template <typename T> static void im2colWhole(T *x, Long *xi, T *z, Long *zi, T *extra) {
    const int kH = toInt(extra[0]), kW = toInt(extra[1]), sH = toInt(extra[2]), sW = toInt(extra[3]);
    const int pH = toInt(extra[4]), pW = toInt(extra[5]), dH = toInt(extra[6]), dW = toInt(extra[7]);
    const Long *is = siShape(xi), *ist = siStride(xi), *os = siShape(zi), *ost = siStride(zi);
    const int bS = (int)is[0], iC = (int)is[1], iH = (int)is[2], iW = (int)is[3], oH = (int)os[4], oW = (int)os[5];
    const bool dense = siOrder(xi) == 'c' && siOrder(zi) == 'c' && stridesDescend(xi) && stridesDescend(zi);
    Long zs[6] = {ost[0], ost[1], ost[2], ost[3], ost[4], ost[5]};
    if (dense) { zs[5] = 1; zs[4] = oW; zs[3] = (Long)oH * oW; zs[2] = zs[3] * kW; zs[1] = zs[2] * kH; }
    for (int b = 0; b < bS; b++)
        for (int c = 0; c < iC; c++)
            for (int kr = 0; kr < kH; kr++)
                for (int kc = 0; kc < kW; kc++)
                    for (int orow = 0; orow < oH; orow++)
                        for (int ocol = 0; ocol < oW; ocol++) {
                            const int r = -pH + kr * dH + orow * sH, q = -pW + kc * dW + ocol * sW;
                            T v = (T)0.0f;
                            if (inRange(r, iH) && inRange(q, iW)) v = x[b * (int)ist[0] + c * (int)ist[1] + r * (int)ist[2] + q * (int)ist[3]];
                            z[b * (int)zs[0] + c * zs[1] + kr * zs[2] + kc * zs[3] + orow * zs[4] + ocol * zs[5]] = v;
                        }
}

// Col2Im 36 (special_ops.h:997-1129): x [bS, iC, kH, kW, oH, oW] -> z [bS, iC, iH, iW]; extra = [sH, sW, pH, pW, iH, iW,
// dH, dW].  The first length(z) elements of z's buffer are cleared, then every column entry is added onto its pixel in
// the order (kRow, kCol, oRow, oCol).  With c-order arrays of descending strides a batch entry of x is read as one run
// of stride inStride[5].
template <typename T> static void col2imWhole(T *x, Long *xi, T *z, Long *zi, T *extra) {
    const Long *is = siShape(xi), *ist = siStride(xi), *ost = siStride(zi);
    const int kH = (int)is[2], kW = (int)is[3], bS = (int)is[0], iC = (int)is[1], oH = (int)is[4], oW = (int)is[5];
    const int sH = toInt(extra[0]), sW = toInt(extra[1]), pH = toInt(extra[2]), pW = toInt(extra[3]);
    const int iH = toInt(extra[4]), iW = toInt(extra[5]), dH = toInt(extra[6]), dW = toInt(extra[7]);
    const bool dense = siOrder(xi) == 'c' && siOrder(zi) == 'c' && stridesDescend(xi) && stridesDescend(zi);
    Long xs[6] = {ist[0], ist[1], ist[2], ist[3], ist[4], ist[5]};
    if (dense) { xs[4] = oW * xs[5]; xs[3] = oH * xs[4]; xs[2] = kW * xs[3]; xs[1] = kH * xs[2]; }
    const Long zn = siNumel(zi);
    for (Long i = 0; i < zn; i++) z[i] = (T)0.0f;
    for (int b = 0; b < bS; b++)
        for (int c = 0; c < iC; c++)
            for (int kr = 0; kr < kH; kr++)
                for (int kc = 0; kc < kW; kc++)
                    for (int orow = 0; orow < oH; orow++) {
                        const int r = -pH + kr * dH + orow * sH;
                        if (!inRange(r, iH)) continue;
                        for (int ocol = 0; ocol < oW; ocol++) {
                            const int q = -pW + kc * dW + ocol * sW;
                            if (!inRange(q, iW)) continue;
                            T &o = z[b * (int)ost[0] + c * (int)ost[1] + r * (int)ost[2] + q * (int)ost[3]];
                            o = o + x[b * (int)xs[0] + c * xs[1] + kr * xs[2] + kc * xs[3] + orow * xs[4] + ocol * xs[5]];
                        }
                    }
}

// Pooling2D 71 (special_ops.h:227-359): x [bS, iC, iH, iW] -> z [bS, iC, oH, oW]; extra = [kH, kW, sH, sW, pH, pW, dH, dW,
// -, mode, p]: mode 0 max, 1 average (p == 0: divide by the cells inside the image, p == 1: by kH * kW), 2 p-norm.
// A c-order result is written densely behind each (batch, channel) start; an f-order one through its strides.
template <typename T> static void pooling2dWhole(T *x, Long *xi, T *z, Long *zi, T *extra) {
    const int kH = toInt(extra[0]), kW = toInt(extra[1]), sH = toInt(extra[2]), sW = toInt(extra[3]);
    const int pH = toInt(extra[4]), pW = toInt(extra[5]), dH = toInt(extra[6]), dW = toInt(extra[7]);
    const int mode = toInt(extra[9]);
    const T p0 = extra[10];
    const int kHEff = kH + (kH - 1) * (dH - 1), kWEff = kW + (kW - 1) * (dW - 1);
    const Long *is = siShape(xi), *ist = siStride(xi), *os = siShape(zi), *ost = siStride(zi);
    const int bS = (int)is[0], iC = (int)is[1], iH = (int)is[2], iW = (int)is[3], oH = (int)os[2], oW = (int)os[3];
    const bool fOrder = siOrder(zi) == 'f';
    auto ceilDiv = [](int a, int b) { return toInt(m_ceil((T)a / (T)b)); };
    for (int c = 0; c < iC; c++)
        for (int b = 0; b < bS; b++) {
            const int zb = b * (int)ost[0] + c * (int)ost[1];
            const T *in = x + b * ist[0] + c * ist[1];
            for (int yy = 0; yy < oH; yy++)
                for (int xx = 0; xx < oW; xx++) {
                    int hs = yy * sH - pH, ws = xx * sW - pW, he = hs + kHEff, we = ws + kWEff;
                    if (hs < 0) hs += ceilDiv(-hs, dH) * dH;
                    if (ws < 0) ws += ceilDiv(-ws, dW) * dW;
                    if (he > iH) he -= ceilDiv(he - iH, dH) * dH;
                    if (we > iW) we -= ceilDiv(we - iW, dW) * dW;
                    const int poolSize = toInt(m_ceil((T)(he - hs) / (T)dH) * (T)toInt(m_ceil((T)(we - ws) / (T)dW)));
                    T acc = mode == 0 ? (T)-1e37 : (T)0.0f;  // MAX_FLOAT is 1e37 (ops.h:12)
                    for (long ky = hs; ky < he; ky += dH)
                        for (long kx = ws; kx < we; kx += dW) {
                            const T v = in[ky * ist[2] + kx * ist[3]];
                            if (mode == 0) { if (v > acc) acc = v; }
                            else if (mode == 1) acc = acc + v;
                            else if (mode == 2) acc = acc + m_pow(m_abs(v), p0);
                        }
                    if (mode == 1) {
                        int div = 0;
                        if (toInt(p0) == 0) div = poolSize;
                        else if (toInt(p0) == 1) div = kH * kW;
                        acc = acc / (T)div;
                    } else if (mode == 2) {
                        acc = m_pow(acc, (T)1.0f / p0);
                    }
                    if (!fOrder) z[zb + yy * oW + xx] = acc;
                    else z[zb + yy * (int)ost[2] + xx * (int)ost[3]] = acc;
                }
        }
}

template <typename T> static bool wholeArrayTransform(int op, T *x, Long *xi, T *z, Long *zi, T *extra) {
    switch (op) {
        case 36: col2imWhole<T>(x, xi, z, zi, extra); return true;
        case 37: im2colWhole<T>(x, xi, z, zi, extra); return true;
        case 48: histogramWhole<T>(x, xi, z, extra); return true;
        case 70: reverseWhole<T>(x, xi, z, zi); return true;
        case 71: pooling2dWhole<T>(x, xi, z, zi, extra); return true;
        default: return false;
    }
}

template <typename T> static void transformShaped(int op, T *x, Long *xi, T *z, Long *zi, T *extra) {
    if (op >= 38 && op <= 41) { specialTransform<T>(op, x, xi, z, zi, extra); return; }
    if (wholeArrayTransform<T>(op, x, xi, z, zi, extra)) return;
    Long n = siNumel(xi);
    Long xe = siEws(xi), ze = siEws(zi);
    if (xe >= 1 && ze >= 1 && siOrder(xi) == siOrder(zi)) { transformStrided<T>(op, x, xe, z, ze, extra, n); return; }
    T probe;
    if (n > 0 && !transformOp<T>(op, x[0], extra, probe)) { printf("[ERROR] Unknown opNum=%d (oracle transform)\n", op); return; }
    int rank = siRank(xi);
    const Long *xst = siStride(xi), *zst = siStride(zi);
    rawIter(rank, siShape(xi), [&](const Long *c) {
        Long ox = 0, oz = 0;
        for (int d = 0; d < rank; d++) { ox += c[d] * xst[d]; oz += c[d] * zst[d]; }
        transformOp<T>(op, x[ox], extra, z[oz]);
    });
}

// scalar: include/loops/cpu/scalar.cpp.  Strided 218-285 (one thread: num_threads is pinned to 1 there), shaped
// 121-215 (EWS pair of equal order -> strided, otherwise raw iteration over x's shape with both stride sets),
// per-TAD scalars 14-62 (z is walked with the x TAD's element-wise stride, lines 22-23; TADs without an
// element-wise stride only print a message).
// The scalar is invariant in these loops and the reference's release flags include -freciprocal-math, so the
// compiled reference divides by it as a multiplication by 1 / scalar (checked on 200000 random operands: Divide,
// SafeDivide and FloorDiv agree with x * (1 / s) everywhere, with x / s only on 60 %).  Written out here so that
// the result does not depend on what the optimiser makes of this file.
template <typename T> static inline T scalarBinary(Bin b, T d1, T s, T *extra) {
    if (b == Divide) return d1 * ((T)1.0f / s);
    if (b == SafeDivide) return s == (T)0.0f ? (T)0.0f : d1 * ((T)1.0f / s);
    if (b == FloorDiv) return m_floor(d1 * ((T)1.0f / s));
    return binaryOp<T, true>(b, d1, s, extra);
}
template <typename T> static void scalarStrided(Bin b, T *x, Long xs, T *z, Long zs, T scalar, T *extra, Long n) {
    for (Long i = 0; i < n; i++) z[i * zs] = scalarBinary<T>(b, x[i * xs], scalar, extra);
}
template <typename T> static void scalarShaped(int op, T *x, Long *xi, T *z, Long *zi, T scalar, T *extra) {
    Bin b = scalarBin(op);
    if (b == Invalid) { printf("[ERROR] Unknown opNum=%d (oracle scalar)\n", op); return; }
    Long n = siNumel(xi);
    Long xe = siEws(xi), ze = siEws(zi);
    if (xe >= 1 && ze >= 1 && siOrder(xi) == siOrder(zi)) { scalarStrided<T>(b, x, xe, z, ze, scalar, extra, n); return; }
    int rank = siRank(xi);
    const Long *xst = siStride(xi), *zst = siStride(zi);
    rawIter(rank, siShape(xi), [&](const Long *c) {
        Long ox = 0, oz = 0;
        for (int d = 0; d < rank; d++) { ox += c[d] * xst[d]; oz += c[d] * zst[d]; }
        z[oz] = scalarBinary<T>(b, x[ox], scalar, extra);
    });
}
template <typename T>
static void scalarTad(int op, T *x, Long *xi, T *z, Long *zi, T *scalars, T *extra, int *dim, int dimLen) {
    (void)zi;
    Bin b = scalarBin(op);
    if (b == Invalid) { printf("[ERROR] Unknown opNum=%d (oracle scalar)\n", op); return; }
    TadPack tp;
    computeTad(xi, dim, dimLen, tp, true);
    const Long tadEws = siEws(tp.shapeInfo.data());
    const Long tadLength = siNumel(tp.shapeInfo.data());
    if (tadEws < 1) { printf("Super-bad loop visited. Shouldn't ever happen\n"); return; }
#pragma omp parallel for schedule(guided) if (tp.numTads / gTadThreshold > 1)
    for (Long r = 0; r < tp.numTads; r++) {
        T *ox = x + tp.offsets[r], *oz = z + tp.offsets[r];
        const T scalar = scalars[r];
        for (Long f = 0; f < tadLength; f++) oz[f * tadEws] = scalarBinary<T>(b, ox[f * tadEws], scalar, extra);
    }
}

// reduce3: include/loops/reduce3.h.  Functors ops.h:2567-2990: the reduction value plus the two running values
// the reference keeps in extraParams[0..1]; EqualsWithEps reads its epsilon from extraParams[2], which
// execScalar fills from the caller's extraParams[0] (reduce3.h:854-858).
template <typename T> struct R3 { T r, e0, e1; };
template <typename T> static inline void r3Op(int op, R3<T> &a, T d1, T d2, T eps) {
    switch (op) {
        case 0: a.r = a.r + m_abs(d1 - d2); break;
        case 1: { T d = d1 - d2; a.r = d * d + a.r; break; }
        case 2: a.e0 += d1 * d1; a.e1 += d2 * d2; a.r = a.r + d1 * d2; break;
        case 3: a.r = d1 * d2 + a.r; break;
        case 4: {
            T diff = m_abs(d1 - d2);
            T v = (T)1.0f;
            if (diff <= eps) v = (T)0.0f;
            else if (diff <= m_max(m_abs(d1), m_abs(d2)) * eps) v = (T)0.0f;
            a.r = v + a.r;
            break;
        }
        case 5: a.e0 += m_abs(d1) * m_abs(d1); a.e1 += m_abs(d2) * m_abs(d2); a.r = a.r + d1 * d2; break;
        case 6: a.e0 += m_min(d1, d2); a.e1 += m_max(d1, d2); break;
        default: a.r = a.r + ((d1 == d2) ? (T)0.0f : (T)1.0f); break;
    }
}
template <typename T> static inline T r3Post(int op, const R3<T> &a, Long n) {
    switch (op) {
        case 1: return m_sqrt(a.r);
        case 2: return a.r / (m_sqrt(a.e0) * m_sqrt(a.e1));
        case 5: return (T)1.0f - (a.r / (m_sqrt(a.e0) * m_sqrt(a.e1)));
        case 6: return (T)1.0f - (a.e0 / a.e1);
        case 7: return (T)(a.r / (T)(float)n);
        default: return a.r;
    }
}
// whole arrays (reduce3.h:838-916): memory-linear pairing when both arrays have an element-wise stride and the
// same order, C-order logical pairing otherwise; one sequential pass
template <typename T> static T reduce3Scalar(int op, T *x, Long *xi, T *extra, T *y, Long *yi) {
    if (op < 0 || op > 7) { printf("[ERROR] Unknown opNum=%d (oracle reduce3)\n", op); return (T)0.0f; }
    const T eps = extra != nullptr ? extra[0] : (T)0.0f;
    const Long n = siNumel(xi);
    const Long xe = siEws(xi), ye = siEws(yi);
    R3<T> a;
    a.r = a.e0 = a.e1 = (T)0.0f;
    if (siOrder(xi) == siOrder(yi) && xe >= 1 && ye >= 1) {
        for (Long i = 0; i < n; i++) r3Op<T>(op, a, x[i * xe], y[i * ye], eps);
    } else {
        Long cx[kMaxRank], cy[kMaxRank];
        for (Long i = 0; i < n; i++) {
            ind2subC(siRank(xi), siShape(xi), (int)i, cx);
            ind2subC(siRank(yi), siShape(yi), (int)i, cy);
            r3Op<T>(op, a, x[getOffset(0, siShape(xi), siStride(xi), cx, siRank(xi))],
                    y[getOffset(0, siShape(yi), siStride(yi), cy, siRank(yi))], eps);
        }
    }
    return r3Post<T>(op, a, n);
}
// one run of `n` pairs: element f of each operand is found from its linear index in the given order
template <typename T>
static T reduce3Run(int op, T *x, const Long *xInfo, T *y, const Long *yInfo, char order, Long n, T eps) {
    R3<T> a;
    a.r = a.e0 = a.e1 = (T)0.0f;
    Long cx[kMaxRank], cy[kMaxRank];
    for (Long f = 0; f < n; f++) {
        if (order == 'f') { ind2subF(siRank(xInfo), siShape(xInfo), (int)f, cx); ind2subF(siRank(yInfo), siShape(yInfo), (int)f, cy); }
        else { ind2subC(siRank(xInfo), siShape(xInfo), (int)f, cx); ind2subC(siRank(yInfo), siShape(yInfo), (int)f, cy); }
        r3Op<T>(op, a, x[getOffset(0, siShape(xInfo), siStride(xInfo), cx, siRank(xInfo))],
                y[getOffset(0, siShape(yInfo), siStride(yInfo), cy, siRank(yInfo))], eps);
    }
    return r3Post<T>(op, a, n);
}
// along `dimension` (reduce3.h:998-1081, 1083-1346): TAD r of x against TAD r of y (equally long arrays) or against
// all of y (y as long as one TAD); pairs by linear index inside the TAD, in the x TAD's order
template <typename T>
static void reduce3Dims(int op, T *x, Long *xi, T *extra, T *y, Long *yi, T *z, Long *zi, int *dim, int dimLen) {
    if (op < 0 || op > 7) { printf("[ERROR] Unknown opNum=%d (oracle reduce3)\n", op); return; }
    if (siIsScalar(zi)) { z[0] = reduce3Scalar<T>(op, x, xi, extra, y, yi); return; }
    const T eps = extra != nullptr ? extra[0] : (T)0.0f;
    if (siNumel(xi) < siNumel(yi)) {
        // x is the single run, y has the TADs (reduce3.h:1186-1215 iterates over the longer operand)
        TadPack ty;
        computeTad(yi, dim, dimLen, ty, true);
        const Long n = siNumel(ty.shapeInfo.data());
        const char order = siOrder(ty.shapeInfo.data()) == 'f' ? 'f' : 'c';
        for (Long r = 0; r < ty.numTads; r++) z[r] = reduce3Run<T>(op, x, xi, y + ty.offsets[r], ty.shapeInfo.data(), order, n, eps);
        return;
    }
    TadPack tx;
    computeTad(xi, dim, dimLen, tx, true);
    const Long n = siNumel(tx.shapeInfo.data());
    const char order = siOrder(tx.shapeInfo.data()) == 'f' ? 'f' : 'c';
    if (siNumel(yi) == siNumel(xi)) {
        TadPack ty;
        computeTad(yi, dim, dimLen, ty, true);
        for (Long r = 0; r < tx.numTads; r++)
            z[r] = reduce3Run<T>(op, x + tx.offsets[r], tx.shapeInfo.data(), y + ty.offsets[r], ty.shapeInfo.data(), order, n, eps);
    } else {
        for (Long r = 0; r < tx.numTads; r++) z[r] = reduce3Run<T>(op, x + tx.offsets[r], tx.shapeInfo.data(), y, yi, order, n, eps);
    }
}
// every TAD of x against every TAD of y (reduce3.h:918-995)
template <typename T>
static void reduce3All(int op, T *x, Long *xi, T *extra, T *y, Long *yi, T *z, int *dim, int dimLen) {
    if (op < 0 || op > 7) { printf("[ERROR] Unknown opNum=%d (oracle reduce3)\n", op); return; }
    const T eps = extra != nullptr ? extra[0] : (T)0.0f;
    TadPack tx, ty;
    computeTad(xi, dim, dimLen, tx, true);
    computeTad(yi, dim, dimLen, ty, true);
    const Long n = siNumel(tx.shapeInfo.data());
    for (Long r = 0; r < tx.numTads; r++)
        for (Long g = 0; g < ty.numTads; g++) {
            R3<T> a;
            a.r = a.e0 = a.e1 = (T)0.0f;
            Long cx[kMaxRank], cy[kMaxRank];
            const Long *xt = tx.shapeInfo.data(), *yt = ty.shapeInfo.data();
            for (Long f = 0; f < n; f++) {
                if (siOrder(yt) == 'c') ind2subC(siRank(yt), siShape(yt), (int)f, cy); else ind2subF(siRank(yt), siShape(yt), (int)f, cy);
                if (siOrder(xt) == 'c') ind2subC(siRank(xt), siShape(xt), (int)f, cx); else ind2subF(siRank(xt), siShape(xt), (int)f, cx);
                r3Op<T>(op, a, x[tx.offsets[r] + getOffset(0, siShape(xt), siStride(xt), cx, siRank(xt))],
                        y[ty.offsets[g] + getOffset(0, siShape(yt), siStride(yt), cy, siRank(yt))], eps);
            }
            z[r * ty.numTads + g] = r3Post<T>(op, a, n);
        }
}

// pairwise: include/loops/pairwise_transform.h:154-424
template <typename T> static void pairwiseStrided(Bin b, T *x, Long xs, T *y, Long ys, T *z, Long zs, T *extra, Long n) {
    int threads = clampThreads(n, gElementThreshold);
    int span = (int)(n / threads) + 8;
#pragma omp parallel num_threads(threads) if (threads > 1)
    {
        Long tid = omp_get_thread_num();
        Long start = span * tid, end = span * (tid + 1);
        if (end > n) end = n;
        if (threads == 1) { start = 0; end = n; }
        for (Long i = start; i < end; i++) z[i * zs] = binaryOp<T, true>(b, x[i * xs], y[i * ys], extra);
    }
}
template <typename T> static void pairwiseShaped(int op, T *x, Long *xi, T *y, Long *yi, T *z, Long *zi, T *extra) {
    Bin b = pairwiseBin(op);
    if (b == Invalid) { printf("[ERROR] Unknown opNum=%d (oracle pairwise)\n", op); return; }
    Long n = siNumel(xi);
    Long xe = siEws(xi), ye = siEws(yi), ze = siEws(zi);
    int xr = siRank(xi), yr = siRank(yi), zr = siRank(zi);
    if (siIsScalar(yi)) {
        if (xe == 1 && ze == 1) {
            for (Long e = 0; e < n; e++) z[e] = binaryOp<T, true>(b, x[e], y[0], extra);
        } else {
#pragma omp parallel for schedule(guided)
            for (Long i = 0; i < n; i++) {
                Long xc[kMaxRank], zc[kMaxRank];
                ind2subC(xr, siShape(xi), (int)i, xc);
                ind2subC(zr, siShape(zi), (int)i, zc);
                z[getOffset(0, siShape(zi), siStride(zi), zc, zr)] =
                    binaryOp<T, true>(b, x[getOffset(0, siShape(xi), siStride(xi), xc, xr)], y[0], extra);
            }
        }
        return;
    }
    bool same = xr == yr;
    for (int i = 0; same && i < xr; i++) same = siShape(xi)[i] == siShape(yi)[i];
    bool orders = siOrder(xi) == siOrder(yi) && siOrder(zi) == siOrder(xi);
    bool ews = xe >= 1 && ye >= 1 && ze >= 1 && xe == ye;
    if (ews && orders) {
        pairwiseStrided<T>(b, x, xe, y, ye, z, ze, extra, same ? n : siNumel(yi));
    } else if (same) {
        const Long *shp = siShape(xi), *xst = siStride(xi), *yst = siStride(yi), *zst = siStride(zi);
#pragma omp parallel for schedule(guided)
        for (Long i = 0; i < shp[0]; i++) {
            T *xl = x + xst[0] * i, *yl = y + yst[0] * i, *zl = z + zst[0] * i;
            rawIter(xr - 1, shp + 1, [&](const Long *c) {
                Long ox = 0, oy = 0, oz = 0;
                for (int d = 0; d < xr - 1; d++) { ox += c[d] * xst[d + 1]; oy += c[d] * yst[d + 1]; oz += c[d] * zst[d + 1]; }
                zl[oz] = binaryOp<T, true>(b, xl[ox], yl[oy], extra);
            });
        }
    } else {
#pragma omp parallel for schedule(guided)
        for (Long i = 0; i < n; i++) {
            Long xc[kMaxRank], yc[kMaxRank], zc[kMaxRank];
            ind2subC(xr, siShape(xi), (int)i, xc);
            ind2subC(yr, siShape(yi), (int)i, yc);
            Long ox = getOffset(0, siShape(xi), siStride(xi), xc, xr);
            Long oy = getOffset(0, siShape(yi), siStride(yi), yc, yr);
            Long oz = ox;
            if (x != z) { ind2subC(zr, siShape(zi), (int)i, zc); oz = getOffset(0, siShape(zi), siStride(zi), zc, zr); }
            z[oz] = binaryOp<T, true>(b, x[ox], y[oy], extra);
        }
    }
}

// broadcast: include/loops/cpu/broadcasting.cpp:42-156
template <typename T> static void broadcast(int op, T *x, Long *xi, T *y, Long *yi, T *z, Long *zi, int *dim, int dimLen) {
    Bin b = broadcastBin(op);
    if (b == Invalid) { printf("[ERROR] Unknown opNum=%d (oracle broadcast)\n", op); return; }
    TadPack tp;
    computeTad(xi, dim, dimLen, tp, true);
    const Long *ti = tp.shapeInfo.data();
    Long tadEws = siEws(ti), yEws = siEws(yi), zEws = tadEws;
    Long tadLength = tadLengthOf(xi, dim, dimLen);
    Long tads = siNumel(xi) / tadLength;
    int threads = clampThreads(tads, gTadThreshold);
#pragma omp parallel for schedule(guided) num_threads(threads) if (threads > 1)
    for (Long i = 0; i < tads; i++) {
        Long off = tp.offsets[i];
        if (tadEws > 0 && yEws > 0 && zEws > 0 && dimLen == 1) {
            T *oz = z + off, *ox = x + off;
            for (Long f = 0; f < tadLength; f++) oz[f * zEws] = binaryOp<T, false>(b, ox[f * tadEws], y[f * yEws], nullptr);
        } else {
            int tr = siRank(ti), yr = siRank(yi);
            Long xc[kMaxRank], yc[kMaxRank];
            for (Long f = 0; f < tadLength; f++) {
                if (siOrder(ti) == 'c') { ind2subC(tr, siShape(ti), (int)f, xc); ind2subC(yr, siShape(yi), (int)f, yc); }
                else { ind2subF(tr, siShape(ti), (int)f, xc); ind2subF(yr, siShape(yi), (int)f, yc); }
                Long o = getOffset(off, siShape(ti), siStride(ti), xc, tr);
                Long oy = getOffset(0, siShape(yi), siStride(yi), yc, yr);
                z[o] = binaryOp<T, false>(b, x[o], y[oy], nullptr);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// reduce functors (ops.h:1534-2560, special_accumulation_ops.h:16-45)
template <typename T> struct ReduceFn {
    int op;
    T *extra;
    bool valid() const { return (op >= 0 && op <= 26 && op != 2); }
    T start(const T *in) const {
        switch (op) {
            case 3: case 4: case 13: case 14: return in[0];
            case 8: case 21: return (T)1.0f;
            default: return (T)0.0f;
        }
    }
    T opf(T d1) const {
        switch (op) {
            case 5: case 11: case 13: case 14: case 15: return m_abs(d1);
            case 6: case 25: return d1 * d1;
            case 9: case 10: { T r = d1 - extra[0]; return r * r; }
            case 12: return matchCondition<T>(d1, extra);
            case 16: return d1 * m_log(d1);
            case 17: return m_log(m_pow(d1, (T)2.0f));
            case 18: return m_pow(d1, (T)2.0f) * m_log(m_pow(d1, (T)2.0f));
            case 19: return m_exp(d1 - extra[0]);
            case 22: return d1 == (T)0.0f ? (T)0.0f : (T)1.0f;
            case 23: { T v = m_abs(d1); return v * v; }
            case 24: return m_pow(m_abs(d1), extra[0]);
            case 26: return d1 == (T)0.0f ? (T)1.0f : (T)0.0f;
            default: return d1;
        }
    }
    T update(T old, T v) const {
        switch (op) {
            case 3: return m_max(v, old);
            case 4: return m_min(v, old);
            case 7: return m_max(m_abs(old), m_abs(v));
            case 8: case 21: return v * old;
            case 9: case 10: case 12: return old + v;
            case 11: case 15: return m_abs(v) + m_abs(old);
            case 13: return m_max(m_abs(v), m_abs(old));
            case 14: return m_min(m_abs(v), m_abs(old));
            default: return v + old;
        }
    }
    T post(T r, Long n) const {
        switch (op) {
            case 0: return r / (T)(int)n;
            case 6: case 23: return m_sqrt(r);
            case 7: return m_max(m_abs(r), m_abs(r));
            case 9: { T v = (r - (m_pow(extra[1], (T)2.0f) / (T)(int)n)) / (T)(n - (int)1); return m_sqrt(v); }
            case 10: return (r - (m_pow(extra[1], (T)2.0f) / (T)(int)n)) / (T)(n - (int)1);
            case 11: case 13: case 14: return m_abs(r);
            case 15: return m_abs(r) / (T)(int)n;
            case 18: return -r;
            case 19: return extra[0] + m_log(r);
            case 20: case 21: return r > (T)0.0f ? (T)1.0f : (T)0.0f;
            case 24: return m_pow(r, (T)1.0 / extra[0]);
            default: return r;
        }
    }
};

// include/loops/cpu/reduce.cpp:14-64 and 206-323
template <typename T> static T reduceScalar(int op, T *x, Long *xi, T *extra) {
    ReduceFn<T> fn{op, extra};
    if (!fn.valid()) { printf("[ERROR] Unknown opNum=%d (oracle reduce)\n", op); return (T)0.0f; }
    Long length = siNumel(xi);
    int ews = (int)siEws(xi);
    if (ews >= 1) {
        if (length < gElementThreshold) {
            T local = fn.start(x);
            for (Long i = 0; i < length; i++) local = fn.update(local, fn.opf(x[i * ews]));
            return fn.post(local, length);
        }
        T finalVal = fn.start(x);
        BlockInfo info(length, gElementThreshold);
        std::vector<T> blocks(info.threads);
#pragma omp parallel num_threads(info.threads) if (info.threads > 1)
        {
            T local = fn.start(x);
            for (Long i = omp_get_thread_num(); i < info.chunks; i += info.threads) {
                Long newOffset = i * info.items;
                if (newOffset >= length) break;
                const T *chunk = x + newOffset * ews;
                for (Long j = 0; j < info.items && newOffset + j < length; j++) local = fn.update(local, fn.opf(chunk[j * ews]));
            }
            blocks[omp_get_thread_num()] = local;
        }
        for (int i = 0; i < info.threads; i++) finalVal = fn.update(finalVal, blocks[i]);
        return fn.post(finalVal, length);
    }
    T start = fn.start(x);
    int rank = siRank(xi);
    const Long *st = siStride(xi);
    rawIter(rank, siShape(xi), [&](const Long *c) {
        Long o = 0;
        for (int d = 0; d < rank; d++) o += c[d] * st[d];
        start = fn.update(start, fn.opf(x[o]));
    });
    return fn.post(start, length);
}

// include/loops/cpu/reduce.cpp:91-193; LogSumExp special accumulation: special_accumulation_ops.h:113-175
template <typename T> static void reduceDims(int op, T *x, Long *xi, T *extra, T *z, Long *zi, int *dim, int dimLen) {
    ReduceFn<T> fn{op, extra};
    if (!fn.valid()) { printf("[ERROR] Unknown opNum=%d (oracle reduce)\n", op); return; }
    Long resultLength = siNumel(zi);
    if (resultLength == 1 || dim == nullptr || dimLen == siRank(xi)) { z[0] = reduceScalar<T>(op, x, xi, extra); return; }
    TadPack tp;
    computeTad(xi, dim, dimLen, tp, true);
    const Long *ti = tp.shapeInfo.data();
    Long tadLength = tadLengthOf(xi, dim, dimLen);
    Long numTads = siNumel(xi) / tadLength;
    Long tadEws = siEws(ti);
    int threads = clampThreads(resultLength, gTadThreshold);
    bool ewsPath = tadEws > 0 && (numTads == 1 || siIsVector(ti) || siIsScalar(ti));
#pragma omp parallel for schedule(guided) num_threads(threads) if (threads > 1)
    for (Long i = 0; i < resultLength; i++) {
        ReduceFn<T> f = fn;
        T shift = z[i];
        if (op == 19) f.extra = &shift;  // the result array holds the maxima of the pre-pass
        T *iter = x + tp.offsets[i];
        T acc = f.start(iter);
        if (ewsPath) {
            for (Long j = 0; j < tadLength; j++) acc = f.update(acc, f.opf(iter[j * tadEws]));
        } else {
            int tr = siRank(ti);
            Long c[kMaxRank];
            for (Long j = 0; j < tadLength; j++) {
                ind2subC(tr, siShape(ti), (int)j, c);
                acc = f.update(acc, f.opf(x[getOffset(tp.offsets[i], siShape(ti), siStride(ti), c, tr)]));
            }
        }
        z[i] = f.post(acc, tadLength);
    }
}

// ---------------------------------------------------------------------------------------------------
// index reduce (ops.h:2992-3466); lower index wins ties, which is what sequential scans produce
template <typename T> struct IndexFn {
    int op;
    T *extra;
    struct IV { T value; Long index; };
    IV start() const {
        IV v;
        v.index = (op == 4 || op == 5) ? -1 : 0;
        switch (op) {
            case 0: v.value = (T)-1e37; break;
            case 1: case 3: v.value = (T)1e37; break;
            case 2: v.value = (T)1e-37; break;
            default: v.value = (T)-1e37; break;
        }
        return v;
    }
    IV update(IV old, IV nw) const {
        switch (op) {
            case 0:
                if (nw.value > old.value) return nw;
                if (nw.value == old.value && nw.index < old.index) return nw;
                return old;
            case 1:
                if (nw.value < old.value) return nw;
                if (nw.value == old.value && nw.index < old.index) return nw;
                return old;
            case 2:
                nw.value = m_abs(nw.value); old.value = m_abs(old.value);
                if (nw.value > old.value) return nw;
                if (nw.value == old.value && nw.index < old.index) return nw;
                return old;
            case 3:
                nw.value = m_abs(nw.value); old.value = m_abs(old.value);
                if (nw.value < old.value) return nw;
                if (nw.value == old.value && nw.index < old.index) return nw;
                return old;
            case 4:
                if (nw.index < 0) return old;
                if (matchCondition<T>(nw.value, extra) == (T)0.0f) return old;
                if (old.index < 0) return nw;
                return old.index > nw.index ? nw : old;
            default:
                if (nw.index < 0) return old;
                if (matchCondition<T>(nw.value, extra) == (T)0.0f) return old;
                if (old.index < 0) return nw;
                return old.index < nw.index ? nw : old;
        }
    }
};
// include/loops/cpu/indexreduce.cpp:36-129
template <typename T> static T indexScalar(int op, T *x, Long *xi, T *extra) {
    if (op < 0 || op > 5) { printf("[ERROR] Unknown opNum=%d (oracle indexreduce)\n", op); return (T)0.0f; }
    IndexFn<T> fn{op, extra};
    typename IndexFn<T>::IV acc = fn.start();
    Long length = siNumel(xi);
    int ews = (int)siEws(xi);
    if (ews < 1) {
        int rank = siRank(xi);
        Long c[kMaxRank];
        for (Long i = 0; i < length; i++) {
            ind2subC(rank, siShape(xi), (int)i, c);
            typename IndexFn<T>::IV cur{x[getOffset(0, siShape(xi), siStride(xi), c, rank)], i};
            acc = fn.update(acc, cur);
        }
        return (T)acc.index;
    }
    if (ews == 1 && length >= gElementThreshold) {
        BlockInfo info(length, gElementThreshold);
        // the reference merges thread results in arrival order under `omp critical`; merging them in chunk
        // order gives the same winner whenever the maximum is unique and the lowest index otherwise
        std::vector<typename IndexFn<T>::IV> locals(info.threads, fn.start());
#pragma omp parallel num_threads(info.threads) if (info.threads > 1)
        {
            typename IndexFn<T>::IV local = fn.start();
            for (Long i = omp_get_thread_num(); i < info.chunks; i += info.threads) {
                Long newOffset = i * info.items;
                if (newOffset >= length) break;
                Long items = info.items;
                if (newOffset + items >= length) items = length - newOffset;
                for (Long j = 0; j < items; j++) {
                    typename IndexFn<T>::IV cur{x[newOffset + j], newOffset + j};
                    local = fn.update(local, cur);
                }
            }
            locals[omp_get_thread_num()] = local;
        }
        for (int t = 0; t < info.threads; t++) acc = fn.update(acc, locals[t]);
        return (T)acc.index;
    }
    for (Long i = 0; i < length; i++) {
        typename IndexFn<T>::IV cur{x[i * ews], i};
        acc = fn.update(acc, cur);
    }
    return (T)acc.index;
}
// include/loops/cpu/indexreduce.cpp:131-228
template <typename T> static void indexDims(int op, T *x, Long *xi, T *extra, T *z, Long *zi, int *dim, int dimLen) {
    if (op < 0 || op > 5) { printf("[ERROR] Unknown opNum=%d (oracle indexreduce)\n", op); return; }
    if (siIsScalar(zi)) { z[0] = indexScalar<T>(op, x, xi, extra); return; }
    IndexFn<T> fn{op, extra};
    Long resultLength = siNumel(zi);
    TadPack tp;
    computeTad(xi, dim, dimLen, tp, true);
    const Long *ti = tp.shapeInfo.data();
    int tadLength = (int)tadLengthOf(xi, dim, dimLen);
    int numTads = (int)(siNumel(xi) / tadLength);
    bool ewsPath = siEws(ti) > 0 && (numTads == 1 || siIsVector(ti) || siIsScalar(ti));
#pragma omp parallel for schedule(guided) if (resultLength > gTadThreshold)
    for (Long i = 0; i < resultLength; i++) {
        typename IndexFn<T>::IV acc = fn.start();
        Long off = tp.offsets[i];
        if (ewsPath) {
            Long ews = siEws(ti);
            for (int j = 0; j < tadLength; j++) {
                typename IndexFn<T>::IV cur{x[off + ews * j], (Long)j};
                acc = fn.update(acc, cur);
            }
        } else {
            int tr = siRank(ti);
            Long c[kMaxRank];
            for (int j = 0; j < tadLength; j++) {
                ind2subC(tr, siShape(ti), j, c);
                typename IndexFn<T>::IV cur{x[getOffset(off, siShape(ti), siStride(ti), c, tr)], (Long)j};
                acc = fn.update(acc, cur);
            }
        }
        z[i] = (T)acc.index;
    }
}

// ---------------------------------------------------------------------------------------------------
// summary stats (include/loops/summarystatsreduce.h:51-257, cpu/summarystatsreduce.cpp:24-196); only the
// moments that reach variance / standard deviation are carried
struct Stats {
    double n, mean, M2;
    void init() { n = mean = M2 = 0; }
    void initWith(double v) { n = 1; mean = v; M2 = 0; }
};
static inline Stats statsUpdate(Stats x, Stats y) {
    if ((long)x.n == 0 && (long)y.n > 0) return y;
    if ((long)x.n > 0 && (long)y.n == 0) return x;
    Stats r;
    double n = x.n + y.n;
    double delta = y.mean - x.mean;
    double delta2 = delta * delta;
    r.n = n;
    r.mean = x.mean + delta * y.n / n;
    r.M2 = x.M2 + y.M2;
    r.M2 += delta2 * x.n * y.n / n;
    return r;
}
template <typename T> static inline T statsValue(int op, bool bias, Stats s) {
    double var = s.n <= 1.0 ? 0.0 : s.M2 / s.n;
    double varB = s.n <= 1.0 ? 0.0 : s.M2 / (s.n - 1.0);
    if (op == 0) {
        if (bias) { T ret = (T)varB; if (ret < (T)0.0f) return (T)var; return ret; }
        return (T)var;
    }
    if (bias) { T ret = (T)varB; if (ret < (T)0.0f) return (T)sqrt(var); return m_sqrt(ret); }
    return (T)sqrt(var);
}
template <typename T> static T statsScalar(int op, bool bias, T *x, Long *xi) {
    if (op < 0 || op > 1) { printf("[ERROR] Unknown opNum=%d (oracle summarystats)\n", op); return (T)0.0f; }
    Stats acc;
    acc.init();
    Long length = siNumel(xi);
    if (siEws(xi) == 1) {
        for (Long i = 0; i < length; i++) { Stats c; c.initWith(M<T>::up(x[i])); acc = statsUpdate(acc, c); }
    } else {
        int rank = siRank(xi);
        Long c[kMaxRank];
        for (Long i = 0; i < length; i++) {
            ind2subC(rank, siShape(xi), (int)i, c);
            Stats s; s.initWith(M<T>::up(x[getOffset(0, siShape(xi), siStride(xi), c, rank)]));
            acc = statsUpdate(acc, s);
        }
    }
    return statsValue<T>(op, bias, acc);
}
template <typename T> static void statsDims(int op, bool bias, T *x, Long *xi, T *z, Long *zi, int *dim, int dimLen) {
    if (op < 0 || op > 1) { printf("[ERROR] Unknown opNum=%d (oracle summarystats)\n", op); return; }
    if (siIsScalar(zi)) { z[0] = statsScalar<T>(op, bias, x, xi); return; }
    TadPack tp;
    computeTad(xi, dim, dimLen, tp, true);
    const Long *ti = tp.shapeInfo.data();
    int resultLength = (int)siNumel(zi);
    if (resultLength == 1 || dimLen == siRank(xi) || tp.wholeThing) { z[0] = statsScalar<T>(op, bias, x, xi); return; }
    bool ewsOk = siEws(ti) > 0 && (tp.numTads == 1 || siIsVector(ti) || siIsScalar(ti) || tp.wholeThing);
    if (!ewsOk && !(dimLen > 1)) {
        // raw iteration over the TAD starting from a zero sample (cpu/summarystatsreduce.cpp:92-146)
        int tr = siRank(ti);
#pragma omp parallel for schedule(guided)
        for (int i = 0; i < resultLength; i++) {
            Stats comp;
            comp.initWith(0.0);
            T *xp = x + tp.offsets[i];
            const Long *st = siStride(ti);
            rawIter(tr, siShape(ti), [&](const Long *c) {
                Long o = 0;
                for (int d = 0; d < tr; d++) o += c[d] * st[d];
                Stats s; s.initWith(M<T>::up(xp[o]));
                comp = statsUpdate(comp, s);
            });
            z[i] = statsValue<T>(op, bias, comp);
        }
    } else if (dimLen == 1) {
        Long ews = siEws(ti);
        Long tadLength = siNumel(ti);
#pragma omp parallel for schedule(guided)
        for (int i = 0; i < resultLength; i++) {
            Long base = tp.offsets[i];
            Stats comp;
            comp.initWith(M<T>::up(x[base]));
            for (Long j = 1; j < tadLength; j++) { Stats s; s.initWith(M<T>::up(x[base + ews * j])); comp = statsUpdate(comp, s); }
            z[i] = statsValue<T>(op, bias, comp);
        }
    } else {
        int tr = siRank(ti);
        Long tadLength = siNumel(ti);
#pragma omp parallel for schedule(guided)
        for (int r = 0; r < resultLength; r++) {
            Long c[kMaxRank];
            Long base = tp.offsets[r];
            Stats comp;
            comp.initWith(M<T>::up(x[base]));
            for (Long i = 1; i < tadLength; i++) {
                ind2subC(tr, siShape(ti), (int)i, c);
                Stats s; s.initWith(M<T>::up(x[getOffset(base, siShape(ti), siStride(ti), c, tr)]));
                comp = statsUpdate(comp, s);
            }
            z[r] = statsValue<T>(op, bias, comp);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// generator: include/helpers/helper_generator.h:61-334, 569-621
struct Rng {
    Long size;
    uint64_t *buffer;
    Long seed, generation, currentPosition, amplifier;
    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    static uint64_t seedConv(Long s) {
        uint64_t x = (uint64_t)s;
        uint64_t z = (x += UINT64_C(0x9E3779B97F4A7C15));
        z = (z ^ (z >> 30)) * UINT64_C(0xBF58476D1CE4E5B9);
        z = (z ^ (z >> 27)) * UINT64_C(0x94D049BB133111EB);
        return z ^ (z >> 31);
    }
    static uint64_t next64(uint64_t s0) {
        uint64_t s1 = s0 % 2147483647 + 11;
        s1 ^= s0;
        uint64_t r0 = rotl(s0, 55) ^ s1 ^ (s1 << 14);
        uint64_t r1 = rotl(s1, 36);
        return r0 + r1;
    }
    static uint64_t safeShift(uint64_t x, uint64_t y) {
        if (y != 0 && x > UINT64_MAX / y) return x / y + 11;
        return x * y + 11;
    }
    void fill() {
        uint64_t s0 = seedConv(seed), s1 = seedConv(seed * 119 + 3);
        for (Long i = 0; i < size; i++) {
            buffer[i] = s0 + s1;
            s1 ^= s0;
            s0 = rotl(s0, 55) ^ s1 ^ (s1 << 14);
            s1 = rotl(s1, 36);
        }
    }
    uint64_t element(Long position) const {
        Long actual = currentPosition + position;
        Long tempGen = generation;
        if (actual >= size) { tempGen += actual / size; actual = actual % size; }
        uint64_t ret = buffer[actual];
        if (tempGen != generation) ret = safeShift(ret, (uint64_t)tempGen);
        if (generation > 1) ret = safeShift(ret, (uint64_t)generation);
        if (amplifier != seed) ret = safeShift(ret, (uint64_t)amplifier);
        if (amplifier != seed || generation > 1 || tempGen != generation) ret = next64(seedConv((Long)ret));
        return ret;
    }
    void rewind(Long n) {
        Long newPos = currentPosition + n;
        if (newPos > size) { generation += newPos / size; newPos = newPos % size; }
        else if (newPos == size) { generation++; newPos = 0; }
        currentPosition = newPos;
    }
    template <typename T> T unit(Long i) const;
    template <typename T> T unit(Long i, T from, T to) const { return from + (unit<T>(i) * (to - from)); }
};
template <> float Rng::unit<float>(Long i) const { return (float)element(i) / (float)18446744073709551615LLU; }
template <> double Rng::unit<double>(Long i) const { return (double)element(i) / (double)18446744073709551615LLU; }
template <> half Rng::unit<half>(Long i) const { return (half)((float)element(i) / (float)18446744073709551615LLU); }

// plain ops (include/ops/random_ops.h); returns the reference's marker values for undefined overloads
template <typename T> static inline T randomOp(int op, int operands, T x, T y, Long i, Long length, const Rng &g, T *a) {
    T undef = operands == 1 ? (T)-1.0f : (operands == 2 ? (T)-2.0f : (T)-3.0f);
    switch (op) {
        case 0: return operands == 1 ? g.unit<T>(i, a[0], a[1]) : undef;
        case 1: return operands == 2 ? (g.unit<T>(i) >= a[0] ? (T)0.0f : x) : undef;
        case 2: return operands == 2 ? (g.unit<T>(i) >= a[0] ? (T)0.0f : x / a[0]) : undef;
        case 3: return operands == 3 ? (g.unit<T>(i) <= a[0] ? y : x) : undef;
        case 4: {
            if (operands != 1) return undef;
            T step = (T)i / ((T)length - (T)1.0f);
            return a[0] * ((T)1.0f - step) + step * a[1];
        }
        case 7:
            if (operands == 1) return a[0] >= g.unit<T>(i) ? (T)1.0f : (T)0.0f;
            if (operands == 2) return x >= g.unit<T>(i) ? (T)1.0f : (T)0.0f;
            return undef;
        case 12: {
            if (operands != 2) return undef;
            T r = g.unit<T>(i);
            return r >= a[0] ? (T)a[1] * a[3] + a[2] : a[1] * x + a[2];
        }
        case 13: {
            T lambda = a[0];
            if (operands == 1) {
                T lo = sizeof(T) == 8 ? (T)2.2250738585072014e-308 : (sizeof(T) == 4 ? (T)1.175494e-38 : (T)6.1035e-05);
                T v = g.unit<T>(i, lo, (T)1.0f);
                return (T)1.f - m_pow((T)M_E, -(lambda * v));
            }
            if (operands == 2) return x <= (T)0.f ? (T)0.f : (T)1.f - m_pow((T)M_E, -(lambda * x));
            return undef;
        }
        default: return undef;
    }
}
// include/loops/cpu/random.cpp:11-199 and the special ops of include/ops/special_random_ops.h
template <typename T>
static void randomExec(int op, Rng *g, int operands, T *x, Long *xi, T *y, Long *yi, T *z, Long *zi, T *a) {
    if (op < 0 || op > 13) { printf("[ERROR] Unknown opNum=%d (oracle random)\n", op); return; }
    Long length = siNumel(zi);
    bool special = op == 5 || op == 6 || (op >= 8 && op <= 11);
    if (special && operands == 3) {
        Long yEws = siEws(yi), zEws = siEws(zi), xEws = siEws(xi);
        const T two_pi = (T)(2.0 * 3.14159265358979323846);
        if (op == 6 || op == 10) {
            T mean = a[0], stddev = a[1];
#pragma omp parallel for schedule(static)
            for (Long k = 0; k < (length + 1) / 2; k++) {
                Long e = 2 * k;
                T u0 = g->unit<T>(e, (T)1e-5f, (T)1.0f), u1 = g->unit<T>(e + 1, (T)1e-5f, (T)1.0f);
                T l = m_sqrt((T)-2.0f * m_log(u0));
                T z0 = l * m_cos(two_pi * u1), z1 = l * m_sin(two_pi * u1);
                T m0 = y == z ? mean : y[e * yEws];
                T v0 = z0 * stddev + m0;
                z[e * zEws] = op == 10 ? m_exp(v0) : v0;
                if (e + 1 < length) {
                    T m1 = y == z ? mean : y[(e + 1) * yEws];
                    T v1 = z1 * stddev + m1;
                    z[(e + 1) * zEws] = op == 10 ? m_exp(v1) : v1;
                }
            }
            g->rewind(length);
        } else if (op == 8 || op == 9) {
            int trials = toInt(a[0]);
#pragma omp parallel for schedule(static)
            for (Long e = 0; e < length; e++) {
                T prob = a[1];
                int success = 0;
                for (int t = 1; t <= trials; t++) {
                    T r = g->unit<T>((e + 1) * t);
                    if (y != z) prob = op == 8 ? y[(t - 1) * yEws] : y[e * yEws];
                    if (r < prob) success++;
                }
                z[e * zEws] = (T)success;
            }
            if (trials > 0) g->rewind(length * trials);
        } else if (op == 11) {
            T mean = a[0], stddev = a[1];
            Long middle = length % 2 == 0 ? length / 2 : length / 2 + 1;
            T ds = m_abs(stddev) * (T)2.0f;
#pragma omp parallel for schedule(static)
            for (Long e = 0; e < middle; e++) {
                Long gen0 = 0;
                T m0 = y == z ? mean : y[e * yEws];
                T m1 = y == z ? mean : (e + middle < length ? y[(e + middle) * yEws] : (T)0.0f);
                T r0, r1;
                do {
                    T u0 = g->unit<T>(e + gen0, (T)1e-6f, (T)1.0f), u1 = g->unit<T>(e + middle + gen0, (T)1e-6f, (T)1.0f);
                    T l = m_sqrt((T)-2.0f * m_log(u0));
                    r0 = (l * m_cos(two_pi * u1)) * stddev + m0;
                    r1 = (l * m_sin(two_pi * u1)) * stddev + m1;
                    gen0 += length;
                } while (m_abs(m0) + m_abs(r0) > ds || m_abs(m1) + m_abs(r1) > ds);
                z[e * zEws] = r0;
                if (e + middle < length) z[(e + middle) * zEws] = r1;
            }
            g->rewind(length);
        } else {  // Choice
            Long yLength = siNumel(yi);
            if (zEws >= 1 && xEws >= 1 && yEws >= 1) {
#pragma omp parallel for schedule(static)
                for (Long e = 0; e < length; e++) {
                    T prob = g->unit<T>(e);
                    T cum = (T)0.0f;
                    for (Long f = 0; f < yLength; f++) {
                        cum += y[f * yEws];
                        if (prob <= cum || f == yLength - 1) { z[e * zEws] = x[f * xEws]; break; }
                    }
                }
            } else {
                int xr = siRank(xi), yr = siRank(yi), zr = siRank(zi);
                for (Long i = 0; i < length; i++) {
                    Long c[kMaxRank];
                    ind2subF(zr, siShape(zi), (int)i, c);
                    Long oz = getOffset(0, siShape(zi), siStride(zi), c, zr);
                    T prob = g->unit<T>(i);
                    T cum = (T)0.0f;
                    for (Long f = 0; f < yLength; f++) {
                        ind2subF(yr, siShape(yi), (int)i, c);
                        cum += y[getOffset(0, siShape(yi), siStride(yi), c, yr)];
                        if (prob <= cum || f == yLength - 1) {
                            ind2subF(xr, siShape(xi), (int)f, c);
                            z[oz] = x[getOffset(0, siShape(xi), siStride(xi), c, xr)];
                            break;
                        }
                    }
                }
            }
            g->rewind(length);
        }
        return;
    }
    Long xe = operands >= 2 ? siEws(xi) : 1, ye = operands >= 3 ? siEws(yi) : 1, ze = siEws(zi);
    int threads = clampThreads(length, gElementThreshold);
    if (xe >= 1 && ye >= 1 && ze >= 1) {
#pragma omp parallel for num_threads(threads) if (threads > 1) schedule(guided)
        for (Long e = 0; e < length; e++)
            z[e * ze] = randomOp<T>(op, operands, operands >= 2 ? x[e * xe] : (T)0.0f, operands >= 3 ? y[e * ye] : (T)0.0f, e,
                                    length, *g, a);
    } else {
#pragma omp parallel for num_threads(threads) if (threads > 1) schedule(guided)
        for (Long i = 0; i < length; i++) {
            Long c[kMaxRank];
            T xv = (T)0.0f, yv = (T)0.0f;
            if (operands >= 2) { ind2subF(siRank(xi), siShape(xi), (int)i, c); xv = x[getOffset(0, siShape(xi), siStride(xi), c, siRank(xi))]; }
            if (operands >= 3) { ind2subF(siRank(yi), siShape(yi), (int)i, c); yv = y[getOffset(0, siShape(yi), siStride(yi), c, siRank(yi))]; }
            ind2subF(siRank(zi), siShape(zi), (int)i, c);
            z[getOffset(0, siShape(zi), siStride(zi), c, siRank(zi))] = randomOp<T>(op, operands, xv, yv, i, length, *g, a);
        }
    }
    g->rewind(length);
}


// ---- data-movement specials ---------------------------------------------------------------------------------
// flatten: blas/cpu/NativeOps.cpp:1529-1664.  The input's elements in `order`, written from result + offset on;
// only the same-order branch with element-wise strides honours the result's stride (1566-1579), the others write
// densely (1586-1598, 1608-1660).
template <typename T>
void flatten(int offset, char order, T *result, const Long *zi, const T *input, const Long *xi) {
    result += offset;
    const Long len = siNumel(xi);
    const int rank = siRank(xi);
    const Long xe = siEws(xi), ze = siEws(zi);
    if (siOrder(xi) == order && xe >= 1 && ze >= 1) {
        for (Long i = 0; i < len; i++) result[i * ze] = input[i * xe];
        return;
    }
    Long c[kMaxRank];
    for (Long i = 0; i < len; i++) {
        if (order == 'f') ind2subF(rank, siShape(xi), (int)i, c);
        else ind2subC(rank, siShape(xi), (int)i, c);
        result[i] = input[getOffset(0, siShape(xi), siStride(xi), c, rank)];
    }
}

// concat: include/ops/impl/specials.cpp:17-200 - the inputs one after the other along `dimension` of the result.
// Restated by coordinates (what every branch there computes for inputs that agree in the other dimensions);
// all-scalar inputs fill result[i] = data[i][0] (47-52).
template <typename T>
void concat(int dimension, int numArrays, T **data, Long **infos, T *result, const Long *zi) {
    bool allScalar = true;
    for (int r = 0; r < numArrays; r++) allScalar = allScalar && siNumel(infos[r]) == 1;
    if (allScalar) {
        for (int r = 0; r < numArrays; r++) result[r * (siEws(zi) >= 1 ? siEws(zi) : 1)] = data[r][0];
        return;
    }
    const int rank = siRank(zi);
    Long start = 0;
    Long c[kMaxRank];
    for (int r = 0; r < numArrays; r++) {
        const Long *xi = infos[r];
        const Long len = siNumel(xi);
        for (Long i = 0; i < len; i++) {
            ind2subC(rank, siShape(xi), (int)i, c);
            const Long xo = getOffset(0, siShape(xi), siStride(xi), c, rank);
            c[dimension] += start;
            result[getOffset(0, siShape(zi), siStride(zi), c, rank)] = data[r][xo];
        }
        start += siShape(xi)[dimension];
    }
}

// pullRows: blas/cpu/NativeOps.cpp:2044-2104
template <typename T>
void pullRows(const T *x, T *z, Long n, const Long *indexes, const Long *ti, const Long *tadOffsets, const Long *zti,
              const Long *zTadOffsets) {
    const Long xe = siEws(ti), ze = siEws(zti), tadLength = siNumel(ti);
    Long cx[kMaxRank], cz[kMaxRank];
    for (Long idx = 0; idx < n; idx++) {
        const T *rx = x + tadOffsets[indexes[idx]];
        T *rz = z + zTadOffsets[idx];
        if (xe >= 1 && ze >= 1) {
            for (Long i = 0; i < tadLength; i++) rz[i * ze] = rx[i * xe];
        } else {
            for (Long i = 0; i < tadLength; i++) {
                ind2subC(siRank(ti), siShape(ti), (int)i, cx);
                ind2subC(siRank(zti), siShape(zti), (int)i, cz);
                rz[getOffset(0, siShape(zti), siStride(zti), cz, siRank(zti))] =
                    rx[getOffset(0, siShape(ti), siStride(ti), cx, siRank(ti))];
            }
        }
    }
}

// tear: blas/cpu/NativeOps.cpp:2118-2160 (the stride-less branch decomposes with ind2sub, i.e. in F order)
template <typename T>
void tear(const T *x, const Long *xi, T **targets, const Long *zi, const Long *ti, const Long *tadOffsets) {
    const Long tadLength = siNumel(ti), te = siEws(ti), ze = siEws(zi);
    const Long numTads = siNumel(xi) / tadLength;
    Long cx[kMaxRank], cz[kMaxRank];
    for (Long r = 0; r < numTads; r++) {
        T *z = targets[r];
        const T *src = x + tadOffsets[r];
        if (ze > 0 && te > 0) {
            for (Long j = 0; j < tadLength; j++) z[j * ze] = src[j * te];
        } else {
            for (Long j = 0; j < tadLength; j++) {
                ind2subF(siRank(ti), siShape(ti), (int)j, cx);
                ind2subF(siRank(zi), siShape(zi), (int)j, cz);
                z[getOffset(0, siShape(zi), siStride(zi), cz, siRank(zi))] = src[getOffset(0, siShape(ti), siStride(ti), cx, siRank(ti))];
            }
        }
    }
}

// shuffle: blas/cpu/NativeOps.cpp:2265-2325 - in place on x, TAD r swapped with TAD map[r], r ascending
template <typename T>
void shuffle(T **xs, Long **xInfos, int N, const int *map, Long **tadInfos, Long **tadOffsets) {
    Long c[kMaxRank];
    for (int f = 0; f < N; f++) {
        T *x = xs[f];
        const Long *ti = tadInfos[f], *off = tadOffsets[f];
        const Long tadLength = siNumel(ti), ews = siEws(ti);
        const Long numTads = siNumel(xInfos[f]) / tadLength;
        for (Long r = 0; r < numTads; r++) {
            if (map[r] < 0) continue;
            const Long oa = off[r], ob = off[map[r]];
            for (Long i = 0; i < tadLength; i++) {
                Long o;
                if (ews == 1) o = i;
                else { ind2subC(siRank(ti), siShape(ti), (int)i, c); o = getOffset(0, siShape(ti), siStride(ti), c, siRank(ti)); }
                T t = x[oa + o];
                x[oa + o] = x[ob + o];
                x[ob + o] = t;
            }
        }
    }
}

// accumulate / average of n buffers as the reference's device kernels do it (include/loops/special_kernels.h:710-742,
// 757-809): a running sum in the data type starting from zero, in table order; average divides the sum by n, writes
// it to z when z is there, and with `propagate` back to every input.  (The CPU loops of include/ops/impl/specials.cpp:
// 344-440 differ by rounding only: they add x[k] / n term by term, and accumulate adds into what z already holds.)
// (compiled without the reciprocal / reassociation licences the rest of this file inherits from the reference's CPU
// flags: the device kernel divides and adds in IEEE arithmetic)
template <typename T>
__attribute__((optimize("no-reciprocal-math", "no-associative-math", "no-unsafe-math-optimizations"))) void accumulateBuffers(
    T **x, T *z, int n, Long length, bool average, bool propagate) {
    for (Long i = 0; i < length; i++) {
        T acc = (T)0.0f;
        for (int k = 0; k < n; k++) acc += x[k][i];
        if (average) acc = acc / (T)n;
        if (z != nullptr) z[i] = acc;
        if (propagate)
            for (int k = 0; k < n; k++) x[k][i] = acc;
    }
}

// conversions: include/loops/type_conversions.h:592-611 - z[i] = (D)((float)x[i])
template <typename S, typename D> void convert(const void *x, Long n, void *z) {
    const S *in = (const S *)x;
    D *out = (D *)z;
    for (Long i = 0; i < n; i++) out[i] = (D)((float)in[i]);
}
}  // namespace oracle

using namespace oracle;

#define ND4J_CPU_FAMILY(SUF, T)                                                                                \
    void nd4j_cpu_reduce3_scalar_##SUF(int op, void *x, Long *xSI, void *extra, void *y, Long *ySI, void *out) { \
        *(T *)out = reduce3Scalar<T>(op, (T *)x, xSI, (T *)extra, (T *)y, ySI);                                \
    }                                                                                                          \
    void nd4j_cpu_reduce3_##SUF(int op, void *x, Long *xSI, void *extra, void *y, Long *ySI, void *z,          \
                                Long *zSI, int *dim, int dimLen) {                                             \
        reduce3Dims<T>(op, (T *)x, xSI, (T *)extra, (T *)y, ySI, (T *)z, zSI, dim, dimLen);                    \
    }                                                                                                          \
    void nd4j_cpu_reduce3_tad_##SUF(int op, void *x, Long *xSI, void *extra, void *y, Long *ySI, void *z,      \
                                    Long *zSI, int *dim, int dimLen) {                                         \
        reduce3Dims<T>(op, (T *)x, xSI, (T *)extra, (T *)y, ySI, (T *)z, zSI, dim, dimLen);                    \
    }                                                                                                          \
    void nd4j_cpu_reduce3_all_##SUF(int op, void *x, Long *xSI, void *extra, void *y, Long *ySI, void *z,      \
                                    Long *zSI, int *dim, int dimLen) {                                         \
        (void)zSI;                                                                                             \
        reduce3All<T>(op, (T *)x, xSI, (T *)extra, (T *)y, ySI, (T *)z, dim, dimLen);                          \
    }                                                                                                          \
    void nd4j_cpu_scalar_##SUF(int op, void *x, Long *xSI, void *z, Long *zSI, double scalar, void *extra) {   \
        scalarShaped<T>(op, (T *)x, xSI, (T *)z, zSI, sizeof(T) < 8 ? (T)(float)scalar : (T)scalar, (T *)extra); \
    }                                                                                                          \
    void nd4j_cpu_scalar_strided_##SUF(int op, void *x, Long xs, void *z, Long zs, double scalar, void *extra, \
                                       Long n) {                                                               \
        Bin b = scalarBin(op);                                                                                 \
        if (b == Invalid) { printf("[ERROR] Unknown opNum=%d (oracle scalar)\n", op); return; }                \
        scalarStrided<T>(b, (T *)x, xs, (T *)z, zs, sizeof(T) < 8 ? (T)(float)scalar : (T)scalar, (T *)extra, n); \
    }                                                                                                          \
    void nd4j_cpu_scalar_tad_##SUF(int op, void *x, Long *xSI, void *z, Long *zSI, void *scalars, void *extra, \
                                   int *dim, int dimLen) {                                                     \
        scalarTad<T>(op, (T *)x, xSI, (T *)z, zSI, (T *)scalars, (T *)extra, dim, dimLen);                     \
    }                                                                                                          \
    void nd4j_cpu_transform_##SUF(int op, void *x, Long *xSI, void *z, Long *zSI, void *extra) {               \
        transformShaped<T>(op, (T *)x, xSI, (T *)z, zSI, (T *)extra);                                          \
    }                                                                                                          \
    void nd4j_cpu_transform_strided_##SUF(int op, void *x, Long xs, void *z, Long zs, void *extra, Long n) {   \
        transformStrided<T>(op, (T *)x, xs, (T *)z, zs, (T *)extra, n);                                        \
    }                                                                                                          \
    void nd4j_cpu_pairwise_##SUF(int op, void *x, Long *xSI, void *y, Long *ySI, void *z, Long *zSI,           \
                                 void *extra) {                                                                \
        pairwiseShaped<T>(op, (T *)x, xSI, (T *)y, ySI, (T *)z, zSI, (T *)extra);                              \
    }                                                                                                          \
    void nd4j_cpu_pairwise_strided_##SUF(int op, void *x, Long xs, void *y, Long ys, void *z, Long zs,         \
                                         void *extra, Long n) {                                                \
        Bin b = pairwiseBin(op);                                                                               \
        if (b == Invalid) { printf("[ERROR] Unknown opNum=%d (oracle pairwise)\n", op); return; }              \
        pairwiseStrided<T>(b, (T *)x, xs, (T *)y, ys, (T *)z, zs, (T *)extra, n);                              \
    }                                                                                                          \
    void nd4j_cpu_broadcast_##SUF(int op, void *x, Long *xSI, void *y, Long *ySI, void *z, Long *zSI,          \
                                  int *dim, int dimLen) {                                                      \
        broadcast<T>(op, (T *)x, xSI, (T *)y, ySI, (T *)z, zSI, dim, dimLen);                                  \
    }                                                                                                          \
    void nd4j_cpu_reduce_##SUF(int op, void *x, Long *xSI, void *extra, void *z, Long *zSI, int *dim,          \
                               int dimLen) {                                                                   \
        if (op == 19) reduceDims<T>(3, (T *)x, xSI, (T *)extra, (T *)z, zSI, dim, dimLen);                     \
        reduceDims<T>(op, (T *)x, xSI, (T *)extra, (T *)z, zSI, dim, dimLen);                                  \
    }                                                                                                          \
    void nd4j_cpu_reduce_scalar_##SUF(int op, void *x, Long *xSI, void *extra, void *out) {                    \
        if (op == 19) {                                                                                        \
            T mx = reduceScalar<T>(3, (T *)x, xSI, (T *)extra);                                                \
            *(T *)out = reduceScalar<T>(19, (T *)x, xSI, &mx);                                                 \
        } else {                                                                                               \
            *(T *)out = reduceScalar<T>(op, (T *)x, xSI, (T *)extra);                                          \
        }                                                                                                      \
    }                                                                                                          \
    void nd4j_cpu_indexreduce_##SUF(int op, void *x, Long *xSI, void *extra, void *z, Long *zSI, int *dim,     \
                                    int dimLen) {                                                              \
        indexDims<T>(op, (T *)x, xSI, (T *)extra, (T *)z, zSI, dim, dimLen);                                   \
    }                                                                                                          \
    void nd4j_cpu_indexreduce_scalar_##SUF(int op, void *x, Long *xSI, void *extra, void *out) {               \
        *(T *)out = indexScalar<T>(op, (T *)x, xSI, (T *)extra);                                               \
    }                                                                                                          \
    void nd4j_cpu_summarystats_##SUF(int op, int bias, void *x, Long *xSI, void *, void *z, Long *zSI,         \
                                     int *dim, int dimLen) {                                                   \
        statsDims<T>(op, bias != 0, (T *)x, xSI, (T *)z, zSI, dim, dimLen);                                    \
    }                                                                                                          \
    void nd4j_cpu_summarystats_scalar_##SUF(int op, int bias, void *x, Long *xSI, void *, void *out) {         \
        *(T *)out = statsScalar<T>(op, bias != 0, (T *)x, xSI);                                                \
    }                                                                                                          \
    void nd4j_cpu_random_z_##SUF(int op, void *state, void *z, Long *zSI, void *args) {                        \
        randomExec<T>(op, (Rng *)state, 1, nullptr, nullptr, nullptr, nullptr, (T *)z, zSI, (T *)args);        \
    }                                                                                                          \
    void nd4j_cpu_random_xz_##SUF(int op, void *state, void *x, Long *xSI, void *z, Long *zSI, void *args) {   \
        randomExec<T>(op, (Rng *)state, 2, (T *)x, xSI, nullptr, nullptr, (T *)z, zSI, (T *)args);             \
    }                                                                                                          \
    void nd4j_cpu_random_xyz_##SUF(int op, void *state, void *x, Long *xSI, void *y, Long *ySI, void *z,       \
                                   Long *zSI, void *args) {                                                    \
        randomExec<T>(op, (Rng *)state, 3, (T *)x, xSI, (T *)y, ySI, (T *)z, zSI, (T *)args);                  \
    }

extern "C" {

const char *nd4j_cpu_kind() { return "port"; }

ND4J_CPU_FAMILY(f32, float)
ND4J_CPU_FAMILY(f16, half)
ND4J_CPU_FAMILY(f64, double)

#define ND4J_CPU_SPECIALS(SUF, T)                                                                                  \
    void nd4j_cpu_flatten_##SUF(int offset, int order, void *z, Long *zSI, void *x, Long *xSI) {                   \
        flatten<T>(offset, (char)order, (T *)z, zSI, (T *)x, xSI);                                                 \
    }                                                                                                              \
    void nd4j_cpu_concat_##SUF(int dim, int n, void **data, Long **infos, void *z, Long *zSI) {                    \
        concat<T>(dim, n, (T **)data, infos, (T *)z, zSI);                                                         \
    }                                                                                                              \
    void nd4j_cpu_pullrows_##SUF(void *x, Long *xSI, void *z, Long *zSI, long long n, Long *idx, Long *tadSI,      \
                                 Long *tadOff, Long *zTadSI, Long *zTadOff) {                                      \
        (void)xSI; (void)zSI;                                                                                      \
        pullRows<T>((T *)x, (T *)z, n, idx, tadSI, tadOff, zTadSI, zTadOff);                                       \
    }                                                                                                              \
    void nd4j_cpu_tear_##SUF(void *x, Long *xSI, void **targets, Long *zSI, Long *tadSI, Long *tadOff) {           \
        tear<T>((T *)x, xSI, (T **)targets, zSI, tadSI, tadOff);                                                   \
    }                                                                                                              \
    void nd4j_cpu_shuffle_##SUF(void **x, Long **xSI, int N, int *map, Long **tadSI, Long **tadOff) {              \
        shuffle<T>((T **)x, xSI, N, map, tadSI, tadOff);                                                           \
    }                                                                                                              \
    void nd4j_cpu_average_##SUF(void **x, void *z, int n, long long length, int propagate) {                       \
        accumulateBuffers<T>((T **)x, (T *)z, n, length, true, propagate != 0);                                    \
    }                                                                                                              \
    void nd4j_cpu_accumulate_##SUF(void **x, void *z, int n, long long length) {                                   \
        accumulateBuffers<T>((T **)x, (T *)z, n, length, false, false);                                            \
    }
ND4J_CPU_SPECIALS(f32, float)
ND4J_CPU_SPECIALS(f16, half)
ND4J_CPU_SPECIALS(f64, double)

// type codes of type_conversions.h:11-18 (3 half, 6 float, 7 double); returns 0 for any other pair
int nd4j_cpu_convert(int srcType, void *x, long long n, int dstType, void *z) {
    if (srcType == 3 && dstType == 6) convert<half, float>(x, n, z);
    else if (srcType == 3 && dstType == 7) convert<half, double>(x, n, z);
    else if (srcType == 6 && dstType == 3) convert<float, half>(x, n, z);
    else if (srcType == 6 && dstType == 7) convert<float, double>(x, n, z);
    else if (srcType == 7 && dstType == 3) convert<double, half>(x, n, z);
    else if (srcType == 7 && dstType == 6) convert<double, float>(x, n, z);
    else return 0;
    return 1;
}

// blas/cpu/NativeOps.cpp:2877-2906
void *nd4j_cpu_rng_init(long long seed, long long size, uint64_t *buffer) {
    Rng *g = new Rng();
    g->size = size; g->buffer = buffer; g->seed = seed; g->generation = 1; g->currentPosition = 0; g->amplifier = seed;
    g->fill();
    return g;
}
void nd4j_cpu_rng_refresh(void *state, long long seed) {
    Rng *g = (Rng *)state;
    g->seed = seed; g->amplifier = seed; g->generation = 1;
    g->currentPosition = 0;
    g->fill();
}
void nd4j_cpu_rng_reseed(void *state, long long seed) { ((Rng *)state)->amplifier = seed; }
void nd4j_cpu_rng_destroy(void *state) { delete (Rng *)state; }
void nd4j_cpu_rng_rewind(void *state, long long n) { ((Rng *)state)->rewind(n); }
void nd4j_cpu_rng_set_offset(void *state, long long off) { ((Rng *)state)->currentPosition = off; }
void nd4j_cpu_rng_state(void *state, long long *out) {
    Rng *g = (Rng *)state;
    out[0] = g->size; out[1] = g->currentPosition; out[2] = g->seed; out[3] = g->generation; out[4] = g->amplifier;
}
int nd4j_cpu_rng_sizeof() { return 88; }
void nd4j_cpu_rng_elements(void *state, long long start, long long n, uint64_t *out) {
    Rng *g = (Rng *)state;
    for (long long i = 0; i < n; i++) out[i] = g->element(start + i);
}
void nd4j_cpu_rng_uniform_f32(void *state, long long start, long long n, float *out) {
    Rng *g = (Rng *)state;
    for (long long i = 0; i < n; i++) out[i] = g->unit<float>(start + i);
}

long long nd4j_cpu_tad_only_shape_info(Long *xSI, int *dim, int dimLen, Long *target, Long *offsets) {
    TadPack tp;
    computeTad(xSI, dim, dimLen, tp, offsets != nullptr);
    std::memcpy(target, tp.shapeInfo.data(), tp.shapeInfo.size() * sizeof(Long));
    if (offsets != nullptr) std::memcpy(offsets, tp.offsets.data(), tp.offsets.size() * sizeof(Long));
    return tp.numTads;
}
long long nd4j_cpu_tad_count(Long *xSI, int *dim, int dimLen) {
    return dimLen == 0 ? 1 : siNumel(xSI) / tadLengthOf(xSI, dim, dimLen);
}
void nd4j_cpu_shape_buffer(int rank, Long *shp, int order, Long *out) { makeShapeInfo(rank, shp, (char)order, out); }
int nd4j_cpu_compute_ews(int rank, Long *shp, Long *stride, int isFOrder) { return computeEws(rank, shp, stride, isFOrder); }
int nd4j_cpu_get_order(int rank, Long *shp, Long *stride, int elementStride) { return orderOf(rank, shp, stride, elementStride); }
void nd4j_cpu_ind2sub(int order, int rank, Long *shp, long long index, Long *out) {
    if (order == 'c') ind2subC(rank, shp, (int)index, out);
    else ind2subF(rank, shp, (int)index, out);
}
void nd4j_cpu_set_thresholds(int elementThreshold, int tadThreshold) {
    gElementThreshold = elementThreshold;
    gTadThreshold = tadThreshold;
}
void nd4j_cpu_set_threads(int n) { omp_set_num_threads(n); }
int nd4j_cpu_get_threads() { return omp_get_max_threads(); }

}  // extern "C"
