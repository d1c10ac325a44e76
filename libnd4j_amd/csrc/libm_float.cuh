// Single-precision exp / log / pow / sin / cos / expm1 / tanh that follow, step for step, the algorithms of the
// C library the reference calls them from: the reference's nd4j_exp<float> etc. are expf, logf, sinf, cosf,
// tanhf of the host libm (include/templatemath.h:537-847), which is not part of the reference tree.  On the
// image this was built for that is glibc 2.35:
//   expf   sysdeps/ieee754/flt-32/e_expf.c    (2^(k/32) table + cubic in double, one rounding to float)
//   logf   sysdeps/ieee754/flt-32/e_logf.c    (16-entry 1/c, log c table + cubic in double)
//   sinf / cosf   sysdeps/ieee754/flt-32/s_sincosf.h (pi/2 reduction in double, degree 7/8 polynomials)
//   powf   sysdeps/ieee754/flt-32/e_powf.c    (log2 table + degree-5 polynomial, y log2 x, 2^t; all in double)
//   expm1f sysdeps/ieee754/flt-32/s_expm1f.c, tanhf sysdeps/ieee754/flt-32/s_tanhf.c (fdlibm, float ops)
// Restating them (instead of rounding a double-precision result) reproduces the library's own rounding
// decisions, so transforms built from these functions agree with the CPU path bit for bit in all but a
// ~1e-8 fraction of arguments, and they are several times cheaper than the double-precision routines.
// Each routine was checked against the host libm on 3e8 arguments before being moved to the device.
#pragma once

#include <hip/hip_runtime.h>

namespace nd4j_amd {
namespace lm {

__device__ __forceinline__ unsigned asU32(float f) { return __builtin_bit_cast(unsigned, f); }
__device__ __forceinline__ float asF32(unsigned u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ unsigned long long asU64(double d) { return __builtin_bit_cast(unsigned long long, d); }
__device__ __forceinline__ double asF64(unsigned long long u) { return __builtin_bit_cast(double, u); }

// bits of 2^(i/32) with i << 47 subtracted
__device__ static const unsigned long long kExp2Tab[32] = {
    0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL, 0x3fef9301d0125b51ULL,
    0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL, 0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL,
    0x3fef06fe0a31b715ULL, 0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,
    0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL, 0x3feea47eb03a5585ULL,
    0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL, 0x3feea11473eb0187ULL, 0x3feea589994cce13ULL,
    0x3feeace5422aa0dbULL, 0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,
    0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL, 0x3fef3720dcef9069ULL,
    0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL, 0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL,
};

// While a kernel runs, the three lookup tables below (exp2, log, and pow's log2; 256 bytes each) are read from LDS:
// a per-lane table read from global memory goes through the vector cache next to the kernel's own streaming
// loads and costs a fused softmax row a third of its time, an LDS read does not.  Every kernel that may evaluate
// expf_, logf_ or powf_ calls loadTables() first, with all threads of the block, before any thread leaves.
struct Tables {
    unsigned long long exp2[32];
    double log[16][2];
    double powLog2[16][2];
};
static __shared__ Tables sTab;

__device__ __forceinline__ float expf_(float x) {
    const double invLn2N = 0x1.71547652b82fep+0 * 32;
    const double c0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32, c1 = 0x1.ebfce50fac4f3p-3 / 32 / 32,
                 c2 = 0x1.62e42ff0c52d6p-1 / 32;
    const double shift = 0x1.8p+52;
    const unsigned abstop = (asU32(x) >> 20) & 0x7ff;
    if (abstop >= 0x42b) {  // |x| >= 88 or not finite
        if (asU32(x) == 0xff800000u) return 0.0f;
        if (abstop >= 0x7f8) return x + x;
        if (x > 0x1.62e42ep6f) return __builtin_inff();
        if (x < -0x1.9fe368p6f) return 0.0f;
    }
    double z = invLn2N * (double)x;
    double kd = z + shift;
    unsigned long long ki = asU64(kd);
    kd -= shift;
    double r = z - kd;
    unsigned long long t = sTab.exp2[ki % 32];
    t += ki << (52 - 5);
    double s = asF64(t);
    z = c0 * r + c1;
    double r2 = r * r;
    double y = c2 * r + 1;
    y = z * r2 + y;
    y = y * s;
    return (float)y;
}

__device__ static const double kLogTab[16][2] = {
    {0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2}, {0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2},
    {0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2},  {0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3},
    {0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3}, {0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3},
    {0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4}, {0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4},
    {0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5}, {0x1p+0, 0x0p+0},
    {0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5},  {0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4},
    {0x1.b2036576afce6p-1, 0x1.526e57720db08p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3},
    {0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2},  {0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2},
};

__device__ __forceinline__ float logf_(float x) {
    const double a0 = -0x1.00ea348b88334p-2, a1 = 0x1.5575b0be00b6ap-2, a2 = -0x1.ffffef20a4123p-2;
    const double ln2 = 0x1.62e42fefa39efp-1;
    unsigned ix = asU32(x);
    if (ix == 0x3f800000u) return 0.0f;
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {
        if (ix * 2 == 0) return -__builtin_inff();
        if (ix == 0x7f800000u) return x;
        if ((ix & 0x80000000u) || ix * 2 >= 0xff000000u) return __builtin_nanf("");
        ix = asU32(x * 0x1p23f);  // subnormal: normalise
        ix -= 23u << 23;
    }
    unsigned tmp = ix - 0x3f330000u;
    int i = (tmp >> (23 - 4)) % 16;
    int k = (int)tmp >> 23;
    unsigned iz = ix - (tmp & (0x1ffu << 23));
    double invc = sTab.log[i][0], logc = sTab.log[i][1];
    double z = (double)asF32(iz);
    double r = z * invc - 1;
    double y0 = logc + (double)k * ln2;
    double r2 = r * r;
    double y = a1 * r + a2;
    y = a0 * r2 + y;
    y = y * r2 + (y0 + r);
    return (float)y;
}

// polynomial of s_sincosf.h: sine for even n, cosine for odd n; `neg` selects the sign-flipped table
__device__ __forceinline__ float sincosPoly(double x, double x2, int n, bool neg) {
    const double c1 = -0x1.ffffffd0c621cp-2, c2 = 0x1.55553e1068f19p-5, c3 = -0x1.6c087e89a359dp-10,
                 c4 = 0x1.99343027bf8c3p-16;
    const double s1 = -0x1.555545995a603p-3, s2 = 0x1.1107605230bc4p-7, s3 = -0x1.994eb3774cf24p-13;
    if ((n & 1) == 0) {
        double x3 = x * x2;
        double t1 = s2 + x2 * s3;
        double x7 = x3 * x2;
        double s = x + x3 * s1;
        return (float)(s + x7 * t1);
    }
    const double sg = neg ? -1.0 : 1.0;
    double x4 = x2 * x2;
    double t2 = sg * c3 + x2 * (sg * c4);
    double t1 = sg + x2 * (sg * c1);
    double x6 = x4 * x2;
    double c = t1 + x4 * (sg * c2);
    return (float)(c + x6 * t2);
}

// valid for |y| < 120; larger arguments take the double-precision routine in the caller
__device__ __forceinline__ float sincosCore(float y, bool wantCos) {
    const double hpiInv = 0x1.45F306DC9C883p+23, hpi = 0x1.921FB54442D18p0;
    double x = (double)y;
    // (The C library returns early below pi/4 - the polynomial on the argument itself - and below 2^-12 - the argument,
    // or 1.  The general path gives the same bits there: the quadrant comes out as 0 exactly, and the polynomial of so
    // small an argument rounds to the argument, or to 1.  Without the early returns the lanes of a wave stay together.)
    double r = x * hpiInv;
    int n = ((int)r + 0x800000) >> 24;
    x = x - (double)n * hpi;
    const int q = n & 3;
    const double s = (q == 1 || q == 2) ? -1.0 : 1.0;  // sign[n & 3] of the first table
    const bool neg = (n & 2) != 0;  // quadrants 2 and 3 use the table with the negated cosine polynomial
    return sincosPoly(x * s, x * x, wantCos ? (n ^ 1) : n, neg);
}

// expm1f exactly as fdlibm branches it; the branch-free expm1f_ below covers 2^-25 <= |x| < 27 ln2 and
// leaves the rest (tiny, huge, infinite, NaN arguments) to this one.
static __device__ __noinline__ float expm1fSlow_(float x) {
    const float one = 1.0f, tiny = 1.0e-30f, hugev = 1.0e30f, o_threshold = 8.8721679688e+01f,
                ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f,
                Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f,
                Q5 = -2.0109921195e-07f;
    float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
    int k;
    unsigned hx = asU32(x);
    const unsigned xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;
    if (hx >= 0x4195b844u) {  // |x| >= 27 ln2
        if (hx >= 0x42b17218u) {
            if (hx > 0x7f800000u) return x + x;
            if (hx == 0x7f800000u) return xsb == 0 ? x : -1.0f;
            if (x > o_threshold) return hugev * hugev;
        }
        if (xsb != 0) return tiny - one;
    }
    if (hx > 0x3eb17218u) {  // |x| > 0.5 ln2
        if (hx < 0x3F851592u) {
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int)(invln2 * x + (xsb == 0 ? 0.5f : -0.5f));
            t = (float)k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {
        return x;
    } else {
        k = 0;
    }
    hfx = 0.5f * x;
    hxs = x * hfx;
    r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    t = 3.0f - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0f - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5f * (x - e) - 0.5f;
    if (k == 1) {
        if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
        return one + 2.0f * (x - e);
    }
    if (k <= -2 || k > 56) {
        y = one - (e - x);
        if (k == 128) y = y * 2.0f * 0x1p127f;
        else y = asF32(asU32(y) + ((unsigned)k << 23));
        return y - one;
    }
    if (k < 23) {
        t = asF32(0x3f800000u - (0x1000000u >> k));
        y = t - (e - x);
        y = asF32(asU32(y) + ((unsigned)k << 23));
    } else {
        t = asF32((unsigned)(0x7f - k) << 23);
        y = x - (e + t);
        y += one;
        y = asF32(asU32(y) + ((unsigned)k << 23));
    }
    return y;
}

// a / b for operands that need neither scaling nor special cases (normal, far from overflow and underflow): reciprocal
// estimate, quotient, two residual corrections - six instructions where the general correctly rounded division takes
// eleven.  expm1f_ and tanhf_ divide such operands only; with this division they return, for every one of the 2^32 float
// arguments, the bits they return with the general one (compared exhaustively on the device).
__device__ __forceinline__ float divShort_(float a, float b) {
    const float y = __builtin_amdgcn_rcpf(b);
    float q = a * y;
    float r = __builtin_fmaf(-b, q, a);
    q = __builtin_fmaf(r, y, q);
    r = __builtin_fmaf(-b, q, a);
    return __builtin_fmaf(r, y, q);
}

// The same arithmetic with the case distinctions turned into selects: every lane of a wave runs one
// instruction stream whatever case its argument falls in.  fdlibm's cases differ only in k (0, +-1 near
// +-ln2, round(x / ln2) otherwise - with t = k the reduction x - t ln2_hi, t ln2_lo is the same expression in
// all of them) and in how the result is put together from the shared polynomial.
__device__ __forceinline__ float expm1f_(float x0) {
    const float one = 1.0f, ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f,
                Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f,
                Q5 = -2.0109921195e-07f;
    unsigned hx = asU32(x0);
    const bool neg = (hx >> 31) != 0;
    hx &= 0x7fffffffu;
    if (__builtin_expect(hx >= 0x4195b844u || hx < 0x33000000u, 0)) return expm1fSlow_(x0);
    const bool red = hx > 0x3eb17218u, nearLn2 = hx < 0x3F851592u;
    const int kg = (int)(invln2 * x0 + (neg ? -0.5f : 0.5f));
    const int k = red ? (nearLn2 ? (neg ? -1 : 1) : kg) : 0;
    float t = (float)k;
    const float hi = x0 - t * ln2_hi, lo = t * ln2_lo;
    const float x = hi - lo;
    const float c = (hi - x) - lo;
    const float hfx = 0.5f * x, hxs = x * hfx;
    const float r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    t = 3.0f - r1 * hfx;
    const float e = hxs * divShort_(r1 - t, 6.0f - x * t);
    const float res0 = x - (x * e - hxs);  // k == 0
    float e2 = (x * (e - c) - c);
    e2 -= hxs;
    const float resM1 = 0.5f * (x - e2) - 0.5f;  // k == -1
    const float resP1 = x < -0.25f ? -2.0f * (e2 - (x + 0.5f)) : one + 2.0f * (x - e2);  // k == 1
    const unsigned sh = (unsigned)k << 23;
    float yn = one - (e2 - x);  // k <= -2
    yn = asF32(asU32(yn) + sh) - one;
    const int kk = k < 0 ? 0 : (k > 31 ? 31 : k);
    float ya = asF32(0x3f800000u - (0x1000000u >> kk)) - (e2 - x);  // 2 <= k < 23
    ya = asF32(asU32(ya) + sh);
    float yb = x - (e2 + asF32((unsigned)(0x7f - k) << 23));  // 23 <= k
    yb += one;
    yb = asF32(asU32(yb) + sh);
    float r = k < 23 ? ya : yb;
    r = k <= -2 ? yn : r;
    r = k == 1 ? resP1 : r;
    r = k == -1 ? resM1 : r;
    r = k == 0 ? res0 : r;
    return r;
}

// tanhf (s_tanhf.c): |x| >= 1: 1 - 2 / (expm1(2|x|) + 2); |x| < 1: -t / (t + 2) with t = expm1(-2|x|); |x| >= 22: 1;
// |x| < 2^-55: x (1 + x).  One expm1f and one division serve all lanes.
__device__ __forceinline__ float tanhf_(float x) {
    const float one = 1.0f, two = 2.0f, tiny = 1.0e-30f;
    const int jx = (int)asU32(x);
    const int ix = jx & 0x7fffffff;
    if (__builtin_expect(ix >= 0x7f800000, 0)) return jx >= 0 ? one / x + one : one / x - one;
    const bool big = ix >= 0x3f800000, sat = ix >= 0x41b00000;
    float arg = (big ? two : -two) * __builtin_fabsf(x);
    if (sat) arg = one;  // result unused; keeps expm1f_ on its main path
    const float t = expm1f_(arg);
    const float q = divShort_(big ? two : -t, t + two);
    float z = big ? one - q : q;
    z = sat ? one - tiny : z;
    float r = jx >= 0 ? z : -z;
    r = ix < 0x24000000 ? x * (one + x) : r;
    return r;
}

// powf: sysdeps/ieee754/flt-32/e_powf.c.  log2(x) from a 16-entry 1/c, log2 c table and a degree-5 polynomial
// in double, y * log2(x) in double, then 2^t through the 2^(k/32) table and a cubic: one rounding to float.
__device__ static const double kPowLog2Tab[16][2] = {
    {0x1.661ec79f8f3bep+0, -0x1.efec65b963019p-2}, {0x1.571ed4aaf883dp+0, -0x1.b0b6832d4fca4p-2},
    {0x1.49539f0f010bp+0, -0x1.7418b0a1fb77bp-2},  {0x1.3c995b0b80385p+0, -0x1.39de91a6dcf7bp-2},
    {0x1.30d190c8864a5p+0, -0x1.01d9bf3f2b631p-2}, {0x1.25e227b0b8eap+0, -0x1.97c1d1b3b7afp-3},
    {0x1.1bb4a4a1a343fp+0, -0x1.2f9e393af3c9fp-3}, {0x1.12358f08ae5bap+0, -0x1.960cbbf788d5cp-4},
    {0x1.0953f419900a7p+0, -0x1.a6f9db6475fcep-5}, {0x1p+0, 0x0p+0},
    {0x1.e608cfd9a47acp-1, 0x1.338ca9f24f53dp-4},  {0x1.ca4b31f026aap-1, 0x1.476a9543891bap-3},
    {0x1.b2036576afce6p-1, 0x1.e840b4ac4e4d2p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.40645f0c6651cp-2},
    {0x1.886e6037841edp-1, 0x1.88e9c2c1b9ff8p-2},  {0x1.767dcf5534862p-1, 0x1.ce0a44eb17bccp-2},
};

__device__ __forceinline__ void loadTables() {
    for (int t = threadIdx.x; t < 96; t += blockDim.x) {
        if (t < 32) sTab.exp2[t] = kExp2Tab[t];
        else if (t < 64) (&sTab.log[0][0])[t - 32] = (&kLogTab[0][0])[t - 32];
        else (&sTab.powLog2[0][0])[t - 64] = (&kPowLog2Tab[0][0])[t - 64];
    }
    __syncthreads();
}

__device__ __forceinline__ bool zeroInfNan(unsigned i) { return 2 * i - 1 >= 2u * 0x7f800000u - 1; }

// 0: y is not an integer, 1: odd integer, 2: even integer
__device__ __forceinline__ int checkInt(unsigned iy) {
    const int e = (iy >> 23) & 0xff;
    if (e < 0x7f) return 0;
    if (e > 0x7f + 23) return 2;
    if (iy & ((1u << (0x7f + 23 - e)) - 1)) return 0;
    if (iy & (1u << (0x7f + 23 - e))) return 1;
    return 2;
}

__device__ __forceinline__ float powf_(float x, float y) {
    unsigned signBias = 0;
    unsigned ix = asU32(x);
    const unsigned iy = asU32(y);
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u || zeroInfNan(iy)) {
        if (zeroInfNan(iy)) {
            const bool xSignalling = 2 * (ix ^ 0x00400000u) > 2u * 0x7fc00000u;
            if (2 * iy == 0) return xSignalling ? x + y : 1.0f;
            if (ix == 0x3f800000u) return (2 * (iy ^ 0x00400000u) > 2u * 0x7fc00000u) ? x + y : 1.0f;
            if (2 * ix > 2u * 0x7f800000u || 2 * iy > 2u * 0x7f800000u) return x + y;
            if (2 * ix == 2 * 0x3f800000u) return 1.0f;
            if ((2 * ix < 2 * 0x3f800000u) == !(iy & 0x80000000u)) return 0.0f;
            return y * y;
        }
        if (zeroInfNan(ix)) {
            float x2 = x * x;
            if ((ix & 0x80000000u) && checkInt(iy) == 1) {
                x2 = -x2;
                signBias = 1;
            }
            if (2 * ix == 0 && (iy & 0x80000000u)) return signBias ? -__builtin_inff() : __builtin_inff();
            return (iy & 0x80000000u) ? 1 / x2 : x2;
        }
        if (ix & 0x80000000u) {  // finite x < 0
            const int yint = checkInt(iy);
            if (yint == 0) return __builtin_nanf("");
            if (yint == 1) signBias = 1u << (5 + 11);
            ix &= 0x7fffffffu;
        }
        if (ix < 0x00800000u) {  // subnormal x
            ix = asU32(x * 0x1p23f);
            ix &= 0x7fffffffu;
            ix -= 23u << 23;
        }
    }
    // log2(x) = log1p(z / c - 1) / ln2 + log2(c) + k
    const unsigned tmp = ix - 0x3f330000u;
    const int i = (tmp >> (23 - 4)) % 16;
    const unsigned top = tmp & 0xff800000u;
    const int k = (int)top >> 23;
    const double z = (double)asF32(ix - top);
    const double r = z * sTab.powLog2[i][0] - 1;
    const double y0 = sTab.powLog2[i][1] + (double)k;
    const double r2 = r * r;
    double yy = 0x1.27616c9496e0bp-2 * r + -0x1.71969a075c67ap-2;
    const double p = 0x1.ec70a6ca7baddp-2 * r + -0x1.7154748bef6c8p-1;
    const double r4 = r2 * r2;
    double q = 0x1.71547652ab82bp0 * r + y0;
    q = p * r2 + q;
    yy = yy * r4 + q;
    const double ylogx = (double)y * yy;
    if (((asU64(ylogx) >> 47) & 0xffff) >= (asU64(126.0) >> 47)) {  // |y log2 x| >= 126
        if (ylogx > 0x1.fffffffd1d571p+6) return signBias ? -__builtin_inff() : __builtin_inff();
        if (ylogx <= -150.0) return signBias ? -0.0f : 0.0f;
    }
    const double shift = 0x1.8p+52 / 32;
    double kd = ylogx + shift;
    const unsigned long long ki = asU64(kd);
    kd -= shift;
    const double rr = ylogx - kd;
    unsigned long long t = sTab.exp2[ki % 32];
    t += (ki + signBias) << (52 - 5);
    const double s = asF64(t);
    const double zz = 0x1.c6af84b912394p-5 * rr + 0x1.ebfce50fac4f3p-3;
    const double rr2 = rr * rr;
    double out = 0x1.62e42ff0c52d6p-1 * rr + 1;
    out = zz * rr2 + out;
    out = out * s;
    return (float)out;
}

}  // namespace lm
}  // namespace nd4j_amd
