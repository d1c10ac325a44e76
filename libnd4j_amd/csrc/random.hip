// Random family: z[i] = op([x[i], [y[i],]] i, length, generator, args), a counter-based generator.
// Reference loops: include/loops/cpu/random.cpp:11-199; ops include/ops/random_ops.h:36-197 and
// include/ops/special_random_ops.h (Choice 14-238, Gaussian 246-397, Binomial 405-520, BinomialEx 531-650,
// TruncatedNormal 654-815, LogNormal 818-969); generator include/helpers/helper_generator.h:185-242.
// opNum table: include/loops/legacy_ops.h:225-239.
//
// Element i of a draw depends only on (state, i), so every lane computes its own elements; the host
// advances the state afterwards (rewindH).  The integer stream is reproduced bit for bit: all 64-bit
// wrap-around products, the `x / y + 11` branch of safeShift and the `% 2147483647` of next64.
#include "elementwise.cuh"
#include "launch.h"

namespace nd4j_amd {

typedef unsigned long long u64;

__device__ __forceinline__ u64 rotl64(u64 x, int k) { return (x << k) | (x >> (64 - k)); }

__device__ __forceinline__ u64 seedConvDev(u64 x) {
    u64 z = (x += 0x9E3779B97F4A7C15ULL);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

// x mod (2^31 - 1): 2^31 == 1 (mod M), so the three 31-bit digits of x are summed and folded.
__device__ __forceinline__ u64 modMersenne31(u64 x) {
    const u64 M = 2147483647ULL;
    u64 s = (x & M) + ((x >> 31) & M) + (x >> 62);
    s = (s & M) + (s >> 31);
    if (s >= M) s -= M;
    return s;
}

// RandomBuffer::next64 (helper_generator.h:222-232)
__device__ __forceinline__ u64 next64Dev(u64 s0) {
    u64 s1 = modMersenne31(s0) + 11;
    s1 ^= s0;
    u64 r0 = rotl64(s0, 55) ^ s1 ^ (s1 << 14);
    u64 r1 = rotl64(s1, 36);
    return r0 + r1;
}

// floor(n / y) for n < y * 2^32 (so the quotient fits 32 bits), through a double estimate that is then
// corrected with the exact remainder.  ry approximates 1/y to ~2^-52, so the estimate is off by at most one.
__device__ __forceinline__ unsigned quot32(u64 n, unsigned y, double ry) {
    double qd = (double)n * ry;
    if (qd > 4294967295.0) qd = 4294967295.0;
    unsigned q = (unsigned)qd;
    long long rem = (long long)(n - (u64)q * (u64)y);
    if (rem < 0) { q--; }
    else if ((u64)rem >= (u64)y) { q++; }
    return q;
}

// 1 / y in double for 1 <= y < 2^32: hardware estimate plus two Newton steps
__device__ __forceinline__ double recip32(unsigned y) {
    const double yd = (double)y;
    double ry = __builtin_amdgcn_rcp(yd);
    ry = ry * (2.0 - yd * ry);
    ry = ry * (2.0 - yd * ry);
    return ry;
}

// floor(x / y) for 1 <= y < 2^32, ry ~ 1 / y: schoolbook division with two 32-bit quotient digits
__device__ __forceinline__ u64 divU64By32(u64 x, unsigned y, double ry) {
    const unsigned hi = (unsigned)(x >> 32);
    const unsigned qhi = quot32((u64)hi, y, ry);
    const unsigned r = hi - qhi * y;
    const u64 n2 = ((u64)r << 32) | (x & 0xffffffffULL);
    const unsigned qlo = quot32(n2, y, ry);
    return ((u64)qhi << 32) | qlo;
}

// floor((2^64 - 1) / y) for 1 <= y < 2^32: the multiplier that turns x / y into a high multiplication
__device__ __forceinline__ u64 magicFor(u64 y) {
    if (y == 0 || (y >> 32) != 0) return 0;
    return divU64By32(0xffffffffffffffffULL, (unsigned)y, recip32((unsigned)y));
}

// RandomBuffer::safeShift (helper_generator.h:238-242): x > MAX / y ? x / y + 11 : x * y + 11.
// For y < 2^32 the caller passes m = floor((2^64 - 1) / y), which is the threshold of the comparison itself, and the
// quotient is mulhi(x, m) or one more (x / y - x m / 2^64 lies in [0, 1)); the remainder that decides is below 2 y, so
// for y < 2^31 its low 32 bits are enough.
__device__ __forceinline__ u64 safeShiftDev(u64 x, u64 y, u64 m) {
    if (y == 0) return 11;
    if ((y >> 32) == 0) {
        const unsigned ys = (unsigned)y;
        if (x > m) {
            u64 q = __umul64hi(x, m);
            if ((ys >> 31) == 0) {
                const unsigned rem = (unsigned)x - (unsigned)q * ys;
                if (rem >= ys) q++;
            } else if (x - q * (u64)ys >= (u64)ys) {
                q++;
            }
            return q + 11;
        }
        // x * y fits 64 bits
        return (((x >> 32) * ys) << 32) + (u64)(unsigned)x * ys + 11;
    }
    if (x > 0xffffffffffffffffULL / y) return x / y + 11;
    return x * y + 11;
}

// Per-thread memory between the elements a thread draws: the quotient / remainder of the last position by
// the buffer size (positions that advance by less than `size` need no division) and the multiplier of the
// last generation divisor.
struct RngWalk {
    Long lastP, q, rem;
    u64 y, m;
    bool valid;
    __device__ __forceinline__ RngWalk() : lastP(0), q(0), rem(0), y(0), m(0), valid(false) {}
    __device__ __forceinline__ u64 element(const RngState &st, Long position);
};

// RandomBuffer::getElement (helper_generator.h:185-220)
__device__ __forceinline__ u64 rngElement(const RngState &st, Long position, RngWalk &w) {
    const Long p = st.position + position;
    Long q, r;
    if (w.valid && p >= w.lastP && p - w.lastP < st.size) {
        q = w.q;
        r = w.rem + (p - w.lastP);
        if (r >= st.size) { r -= st.size; q++; }
    } else if (p < st.size) {
        q = 0;
        r = p;
    } else {
        if ((u64)st.size < (1ULL << 32) && ((u64)p >> 32) < (u64)st.size) q = (Long)quot32((u64)p, (unsigned)st.size, st.rSize);
        else q = (Long)((u64)p / (u64)st.size);
        r = p - q * st.size;
    }
    w.lastP = p; w.q = q; w.rem = r; w.valid = true;
    u64 x = st.buffer[r];
    const bool genDiffers = q != 0;
    if (genDiffers) {
        const u64 tempGen = (u64)(st.generation + q);
        if (tempGen != w.y) { w.y = tempGen; w.m = magicFor(tempGen); }
        x = safeShiftDev(x, tempGen, w.m);
    }
    if (st.generation > 1) x = safeShiftDev(x, (u64)st.generation, st.mGeneration);
    if (st.amplifier != st.seed) x = safeShiftDev(x, (u64)st.amplifier, st.mAmplifier);
    if (st.amplifier != st.seed || st.generation > 1 || genDiffers) x = next64Dev(seedConvDev(x));
    return x;
}
__device__ __forceinline__ u64 rngElement(const RngState &st, Long position) {
    RngWalk w;
    return rngElement(st, position, w);
}
__device__ __forceinline__ u64 RngWalk::element(const RngState &st, Long position) { return rngElement(st, position, *this); }

// getElement for a block whose elements lie within one trip round the buffer of each other: the block's first position
// is divided by the buffer size once (by its first thread, through LDS), after which an element's index is an addition
// with at most one wrap, its buffer round is the block's or the next, and the multipliers of both rounds' divisors are
// the block's too.  Needs size < 2^31 and generation + round + 1 < 2^31 (the host checks both).
struct RngBlockWalk {
    Long first;   // index of the block's first element in the draw
    Long q0, r0;  // buffer round and index of position + first
    u64 mA, mB;   // floor((2^64 - 1) / (generation + q0)) and the same for the next round
    // where element i's word lies in the buffer, and whether it belongs to the round after the block's first
    __device__ __forceinline__ unsigned locate(const RngState &st, Long i, bool &wrapped) const {
        // (32-bit arithmetic: the block's elements span no more than the buffer, which holds fewer than 2^31 words, and the
        // generations stay below 2^31)
        const unsigned size = (unsigned)st.size;
        unsigned r = (unsigned)r0 + (unsigned)(i - first);
        wrapped = r >= size;
        if (wrapped) r -= size;
        return r;
    }
    __device__ __forceinline__ u64 element(const RngState &st, Long i) const {
        bool wrapped;
        const unsigned r = locate(st, i, wrapped);
        return finish(st, st.buffer[r], wrapped);
    }
    // the draw from its buffer word
    __device__ __forceinline__ u64 finish(const RngState &st, u64 x, bool wrapped) const {
        const bool genDiffers = q0 != 0 || wrapped;
        if (genDiffers) {
            const unsigned gen = (unsigned)(st.generation + q0) + (wrapped ? 1u : 0u);
            __builtin_assume(gen != 0 && (gen >> 31) == 0);
            x = safeShiftDev(x, (u64)gen, wrapped ? mB : mA);
        }
        if (st.generation > 1) x = safeShiftDev(x, (u64)st.generation, st.mGeneration);
        if (st.amplifier != st.seed) x = safeShiftDev(x, (u64)st.amplifier, st.mAmplifier);
        if (st.amplifier != st.seed || st.generation > 1 || genDiffers) x = next64Dev(seedConvDev(x));
        return x;
    }
};
// A draw whose buffer word has been loaded ahead of time
struct RngFetched {
    const RngBlockWalk &walk;
    u64 word;
    bool wrapped;
    __device__ __forceinline__ u64 element(const RngState &st, Long) const { return walk.finish(st, word, wrapped); }
};
// all threads of the block call this together (it holds a barrier)
__device__ __forceinline__ RngBlockWalk rngBlockWalk(const RngState &st, Long first) {
    __shared__ unsigned long long shared[4];
    if (threadIdx.x == 0) {
        const Long p = st.position + first;
        Long q = 0;
        if (p >= st.size) q = ((u64)p >> 32) < (u64)st.size ? (Long)quot32((u64)p, (unsigned)st.size, st.rSize) : (Long)((u64)p / (u64)st.size);
        shared[0] = (u64)q;
        shared[1] = (u64)(p - q * st.size);
        shared[2] = magicFor((u64)(st.generation + q));
        shared[3] = magicFor((u64)(st.generation + q + 1));
    }
    __syncthreads();
    RngBlockWalk w;
    w.first = first;
    w.q0 = (Long)shared[0];
    w.r0 = (Long)shared[1];
    w.mA = shared[2];
    w.mB = shared[3];
    return w;
}

// relativeT<T>(index): u64 -> [0, 1] (helper_generator.h:481-486).  (T)MAX_UINT is exactly 2^64.
template <typename C> __device__ __forceinline__ C toUnit(u64 r);
template <> __device__ __forceinline__ float toUnit<float>(u64 r) { return (float)r * 5.42101086242752217e-20f; }
template <> __device__ __forceinline__ double toUnit<double>(u64 r) { return (double)r * 5.42101086242752217e-20; }

template <typename TT> struct RandomCtx {
    typedef typename Compute<TT>::type C;
    RngState st;
    Params<TT> args;
    Long length;
    template <class Walk> __device__ __forceinline__ C unit(Long i, Walk &w) const {
        C u = toUnit<C>(w.element(st, i));
        // storage types narrower than float round the draw to the storage type first (481-484)
        if (sizeof(TT) < 4) u = toCompute(fromCompute<TT>(u));
        return u;
    }
    __device__ __forceinline__ C unit(Long i) const {
        RngWalk w;
        return unit(i, w);
    }
    template <class Walk> __device__ __forceinline__ C unit(Long i, C from, C to, Walk &w) const { return from + (unit(i, w) * (to - from)); }
    __device__ __forceinline__ C unit(Long i, C from, C to) const { return from + (unit(i) * (to - from)); }
};

// Plain (non-special) ops.  nOperands: 1 = (z), 2 = (x, z), 3 = (x, y, z).  Overloads an op does not define
// return the reference's marker values -1 / -2 / -3 (random_ops.h:15-17).
template <int OP, typename TT, class Walk>
__device__ __forceinline__ typename Compute<TT>::type randomOp(const RandomCtx<TT> &c, int nOperands,
                                                               typename Compute<TT>::type x,
                                                               typename Compute<TT>::type y, Long i, Walk &w) {
    typedef typename Compute<TT>::type C;
    const C undefinedValue = nOperands == 1 ? (C)-1 : (nOperands == 2 ? (C)-2 : (C)-3);
    switch (OP) {
        case 0:  // UniformDistribution
            if (nOperands != 1) return undefinedValue;
            return c.unit(i, c.args[0], c.args[1], w);
        case 1:  // DropOut
            if (nOperands != 2) return undefinedValue;
            return c.unit(i, w) >= c.args[0] ? (C)0 : x;
        case 2: {  // DropOutInverted
            if (nOperands != 2) return undefinedValue;
            C prob = c.args[0];
            return c.unit(i, w) >= prob ? (C)0 : x / prob;
        }
        case 3:  // ProbablisticMerge
            if (nOperands != 3) return undefinedValue;
            return c.unit(i, w) <= c.args[0] ? y : x;
        case 4: {  // Linspace
            if (nOperands != 1) return undefinedValue;
            C from = c.args[0];
            C to = c.args[1];
            // the reference's release flags (-freciprocal-math) hoist 1 / (length - 1) out of its loop
            C step = (C)i * ((C)1 / ((C)c.length - (C)1));
            return from * ((C)1 - step) + step * to;
        }
        case 7:  // BernoulliDistribution
            if (nOperands == 1) return c.args[0] >= c.unit(i, w) ? (C)1 : (C)0;
            if (nOperands == 2) return x >= c.unit(i, w) ? (C)1 : (C)0;
            return undefinedValue;
        case 12: {  // AlphaDropOut: args = p, a, b, alphaPrime
            if (nOperands != 2) return undefinedValue;
            C u = c.unit(i, w);
            return u >= c.args[0] ? c.args[1] * c.args[3] + c.args[2] : c.args[1] * x + c.args[2];
        }
        case 13: {  // ExponentialDistribution
            C lambda = c.args[0];
            if (nOperands == 1) {
                // DataTypeUtils::min<T>(): smallest positive normal of the data type
                C lo = sizeof(TT) == 8 ? (C)2.2250738585072014e-308 : (sizeof(TT) == 4 ? (C)1.175494e-38f : (C)6.1035e-05f);
                C v = c.unit(i, lo, (C)1, w);
                return (C)1 - m::pow_((C)2.718281828459045, -(lambda * v));
            }
            if (nOperands == 2) return x <= (C)0 ? (C)0 : (C)1 - m::pow_((C)2.718281828459045, -(lambda * x));
            return undefinedValue;
        }
        default:
            // special ops reached through an overload without specialOp: marker values
            return undefinedValue;
    }
}

// Elements per thread of the two hot kernels: a block takes kRngIter * kBlock consecutive elements, so the
// positions one thread visits advance by kBlock and its RngWalk state stays valid across them.
static constexpr int kRngIter = 8;

template <typename TT, int OP>
__global__ void __launch_bounds__(kBlock) randomPlainKernel(RandomCtx<TT> c, const TT *x, const TT *y, TT *z, int nOperands,
                                                            int strided, Long xEws, Long yEws, Long zEws, DimMap xm,
                                                            DimMap ym, DimMap zm) {
    lm::loadTables();
    typedef typename Compute<TT>::type C;
    const Long chunk = (Long)kBlock * kRngIter;
    RngWalk w;
    // a block takes consecutive chunks: its positions then stay within one or two generations of the buffer, and the
    // multiplier of the generation divisor (RngWalk::m) is rarely recomputed
    const Long nChunks = (c.length + chunk - 1) / chunk, perBlock = (nChunks + gridDim.x - 1) / gridDim.x;
    Long lastChunk = ((Long)blockIdx.x + 1) * perBlock;
    if (lastChunk > nChunks) lastChunk = nChunks;
    for (Long ci = (Long)blockIdx.x * perBlock; ci < lastChunk; ci++) {
        const Long base = ci * chunk;
        for (int k = 0; k < kRngIter; k++) {
            const Long i = base + (Long)k * kBlock + threadIdx.x;
            if (i >= c.length) break;
            Long ox, oy, oz;
            if (strided) {
                ox = i * xEws; oy = i * yEws; oz = i * zEws;
            } else {
                ox = nOperands >= 2 ? mapOffsetAny(xm, i) : 0;
                oy = nOperands >= 3 ? mapOffsetAny(ym, i) : 0;
                oz = mapOffsetAny(zm, i);
            }
            C xv = nOperands >= 2 ? toCompute(x[ox]) : (C)0;
            C yv = nOperands >= 3 ? toCompute(y[oy]) : (C)0;
            z[oz] = fromCompute<TT>(randomOp<OP, TT>(c, nOperands, xv, yv, i, w));
        }
    }
}

// The same ops for the usual call: operands with element-wise strides, a buffer of fewer than 2^31 words, generations
// below 2^31.  A block takes `perBlock` consecutive elements (no more than the buffer holds), so its elements' buffer
// rounds and divisor multipliers are the block's (RngBlockWalk); the operand count and unit strides are compile-time.
template <typename TT, int OP, int NOPS, bool UNIT>
__global__ void __launch_bounds__(kBlock) randomLeanKernel(RandomCtx<TT> c, const TT *x, const TT *y, TT *z, Long xEws, Long yEws,
                                                           Long zEws, Long perBlock) {
    if (OP == 13) lm::loadTables();  // ExponentialDistribution's pow
    typedef typename Compute<TT>::type C;
    const Long first = (Long)blockIdx.x * perBlock;
    RngBlockWalk w = rngBlockWalk(c.st, first);
    const unsigned count = (unsigned)(c.length - first < perBlock ? c.length - first : perBlock);
    if constexpr (UNIT && sizeof(TT) == 4) {
        // dense 4-byte operands on 16-byte boundaries: a thread draws four neighbouring elements and moves them as one vector
        const bool aligned = ((reinterpret_cast<uintptr_t>(z) | (NOPS >= 2 ? reinterpret_cast<uintptr_t>(x) : 0) |
                               (NOPS >= 3 ? reinterpret_cast<uintptr_t>(y) : 0)) & 15) == 0 && perBlock % 4 == 0;
        if (aligned) {
            for (unsigned o = threadIdx.x * 4; o < count; o += kBlock * 4) {
                const Long i = first + o;
                if (o + 4 <= count) {
                    // The four buffer words are requested first and the operands behind them: loads return in the order
                    // they were issued, so the draws' arithmetic (which needs only the words, from the caches) starts while
                    // the operands are still on their way from memory and covers their latency.  The other way round every
                    // round waited for its operands before its first instruction: 23 us per 2^26 elements of dropout.
                    u64 word[4];
                    bool wrapped[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) word[e] = c.st.buffer[w.locate(c.st, i + e, wrapped[e])];
                    __builtin_amdgcn_sched_barrier(0);
                    Pack<TT> xv, yv, out;
                    if (NOPS >= 2) xv = loadPack(reinterpret_cast<const Pack<TT> *>(x + i));
                    if (NOPS >= 3) yv = loadPack(reinterpret_cast<const Pack<TT> *>(y + i));
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        RngFetched f{w, word[e], wrapped[e]};
                        out.v[e] = fromCompute<TT>(randomOp<OP, TT>(c, NOPS, NOPS >= 2 ? toCompute(xv.v[e]) : (C)0,
                                                                    NOPS >= 3 ? toCompute(yv.v[e]) : (C)0, i + e, f));
                    }
                    storePack(reinterpret_cast<Pack<TT> *>(z + i), out);
                } else {
                    for (unsigned e = o; e < count; e++)
                        z[first + e] = fromCompute<TT>(randomOp<OP, TT>(c, NOPS, NOPS >= 2 ? toCompute(x[first + e]) : (C)0,
                                                                        NOPS >= 3 ? toCompute(y[first + e]) : (C)0, first + e, w));
                }
            }
            return;
        }
    }
    for (unsigned o = threadIdx.x; o < count; o += kBlock) {
        const Long i = first + o;
        const C xv = NOPS >= 2 ? toCompute(x[UNIT ? i : i * xEws]) : (C)0;
        const C yv = NOPS >= 3 ? toCompute(y[UNIT ? i : i * yEws]) : (C)0;
        z[UNIT ? i : i * zEws] = fromCompute<TT>(randomOp<OP, TT>(c, NOPS, xv, yv, i, w));
    }
}

// Box-Muller pairs (2k, 2k+1) sharing u0 = draw(2k), u1 = draw(2k+1) (special_random_ops.h:333-396):
// z[2k] = sqrt(-2 ln u0) cos(2 pi u1) * stddev + mean, z[2k+1] = ... sin(...).  EXP applies exp() on top
// (LogNormal, 900-969).
template <typename TT, bool EXP, class Walk>
__device__ __forceinline__ void gaussianPair(const RandomCtx<TT> &c, const TT *y, TT *z, int yIsZ, Long yEws, Long zEws, bool pairStores,
                                             Long k, Walk &w) {
    typedef typename Compute<TT>::type C;
    const C twoPi = (C)(2.0 * 3.14159265358979323846);
    const C mean = c.args[0];
    const C stddev = c.args[1];
    const Long e = 2 * k;
    C u0 = c.unit(e, (C)1e-5f, (C)1, w);
    C u1 = c.unit(e + 1, (C)1e-5f, (C)1, w);
    C r = m::sqrt_((C)-2 * m::log_(u0));
    C ang = twoPi * u1;
    C z0 = r * m::cos_(ang);
    C z1 = r * m::sin_(ang);
    C m0 = yIsZ ? mean : toCompute(y[e * yEws]);
    C v0 = z0 * stddev + m0;
    const TT r0 = fromCompute<TT>(EXP ? m::exp_(v0) : v0);
    if (e + 1 < c.length) {
        C m1 = yIsZ ? mean : toCompute(y[(e + 1) * yEws]);
        C v1 = z1 * stddev + m1;
        const TT r1 = fromCompute<TT>(EXP ? m::exp_(v1) : v1);
        if (pairStores) {
            // one store per pair: a wave's store then covers one contiguous stretch instead of every other element
            struct alignas(2 * sizeof(TT)) Two { TT a, b; } two = {r0, r1};
            *reinterpret_cast<Two *>(z + e) = two;
        } else {
            z[e * zEws] = r0;
            z[(e + 1) * zEws] = r1;
        }
    } else {
        z[e * zEws] = r0;
    }
}
template <typename TT, bool EXP>
__global__ void __launch_bounds__(kBlock) gaussianKernel(RandomCtx<TT> c, const TT *y, TT *z, int yIsZ, Long yEws, Long zEws) {
    lm::loadTables();
    const Long pairs = (c.length + 1) / 2;
    const Long chunk = (Long)kBlock * kRngIter;
    const bool pairStores = zEws == 1 && (reinterpret_cast<uintptr_t>(z) & (2 * sizeof(TT) - 1)) == 0;
    RngWalk w;
    // consecutive chunks per block, as in randomPlainKernel
    const Long nChunks = (pairs + chunk - 1) / chunk, perBlock = (nChunks + gridDim.x - 1) / gridDim.x;
    Long lastChunk = ((Long)blockIdx.x + 1) * perBlock;
    if (lastChunk > nChunks) lastChunk = nChunks;
    for (Long base = (Long)blockIdx.x * perBlock * chunk; base < lastChunk * chunk; base += chunk)
    for (int it = 0; it < kRngIter; it++) {
        const Long k = base + (Long)it * kBlock + threadIdx.x;
        if (k >= pairs) break;
        gaussianPair<TT, EXP>(c, y, z, yIsZ, yEws, zEws, pairStores, k, w);
    }
}
// the usual call (see randomLeanKernel): a block takes `pairsPerBlock` consecutive pairs, twice as many positions
template <typename TT, bool EXP>
__global__ void __launch_bounds__(kBlock) gaussianLeanKernel(RandomCtx<TT> c, const TT *y, TT *z, int yIsZ, Long yEws, Long zEws,
                                                             Long pairsPerBlock) {
    lm::loadTables();
    const Long pairs = (c.length + 1) / 2;
    const bool pairStores = zEws == 1 && (reinterpret_cast<uintptr_t>(z) & (2 * sizeof(TT) - 1)) == 0;
    const Long first = (Long)blockIdx.x * pairsPerBlock;
    RngBlockWalk w = rngBlockWalk(c.st, 2 * first);
    Long last = first + pairsPerBlock;
    if (last > pairs) last = pairs;
    for (Long k = first + threadIdx.x; k < last; k += kBlock) gaussianPair<TT, EXP>(c, y, z, yIsZ, yEws, zEws, pairStores, k, w);
}

// TruncatedNormal (special_random_ops.h:731-790): pairs (e, e + middle), redrawn with the index advanced
// by zLength until both lie within two standard deviations.
template <typename TT>
__global__ void __launch_bounds__(kBlock) truncatedNormalKernel(RandomCtx<TT> c, const TT *y, TT *z, int yIsZ, Long yEws,
                                                                Long zEws) {
    lm::loadTables();
    typedef typename Compute<TT>::type C;
    const C twoPi = (C)(2.0 * 3.14159265358979323846);
    const C mean = c.args[0];
    const C stddev = c.args[1];
    const Long n = c.length;
    const Long middle = (n % 2 == 0) ? n / 2 : n / 2 + 1;
    const C ds = m::abs_(stddev) * (C)2;
    const Long stride = (Long)gridDim.x * kBlock;
    for (Long e = (Long)blockIdx.x * kBlock + threadIdx.x; e < middle; e += stride) {
        C m0 = yIsZ ? mean : toCompute(y[e * yEws]);
        C m1 = (yIsZ || e + middle >= n) ? (yIsZ ? mean : (C)0) : toCompute(y[(e + middle) * yEws]);
        C r0 = (C)0, r1 = (C)0;
        Long gen = 0;
        // the acceptance probability per round is about 0.91; the bound only guarantees termination
        for (int tries = 0; tries < 4096; tries++) {
            C u0 = c.unit(e + gen, (C)1e-6f, (C)1);
            C u1 = c.unit(e + middle + gen, (C)1e-6f, (C)1);
            C l = m::sqrt_((C)-2 * m::log_(u0));
            C ang = twoPi * u1;
            r0 = (l * m::cos_(ang)) * stddev + m0;
            r1 = (l * m::sin_(ang)) * stddev + m1;
            gen += n;
            if (!(m::abs_(m0) + m::abs_(r0) > ds || m::abs_(m1) + m::abs_(r1) > ds)) break;
        }
        z[e * zEws] = fromCompute<TT>(r0);
        if (e + middle < n) z[(e + middle) * zEws] = fromCompute<TT>(r1);
    }
}

// Binomial (405-520): trials draws at index (e+1)*t; probabilities args[1] or y[t-1] (EX: y[e], 531-650).
template <typename TT, bool EX>
__global__ void __launch_bounds__(kBlock) binomialKernel(RandomCtx<TT> c, const TT *y, TT *z, int yIsZ, Long yEws, Long zEws) {
    lm::loadTables();
    typedef typename Compute<TT>::type C;
    const int trials = m::toIntX86(c.args[0]);
    const Long stride = (Long)gridDim.x * kBlock;
    for (Long e = (Long)blockIdx.x * kBlock + threadIdx.x; e < c.length; e += stride) {
        C prob = c.args[1];
        int success = 0;
        for (int t = 1; t <= trials; t++) {
            C v = c.unit((e + 1) * t);
            if (!yIsZ) prob = toCompute(y[(EX ? e : (Long)(t - 1)) * yEws]);
            if (v < prob) success++;
        }
        z[e * zEws] = fromCompute<TT>((C)success);
    }
}

// Choice (145-238): inverse CDF over probabilities y, values x.
template <typename TT>
__global__ void __launch_bounds__(kBlock) choiceKernel(RandomCtx<TT> c, const TT *x, const TT *y, TT *z, int strided,
                                                       Long xEws, Long yEws, Long zEws, DimMap xm, DimMap ym, DimMap zm,
                                                       Long yLength) {
    lm::loadTables();
    typedef typename Compute<TT>::type C;
    const Long stride = (Long)gridDim.x * kBlock;
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < c.length; i += stride) {
        C prob = c.unit(i);
        C cum = (C)0;
        Long oz = strided ? i * zEws : mapOffsetAny(zm, i);
        for (Long f = 0; f < yLength; f++) {
            // in the coordinate branch the reference indexes the probabilities with the OUTPUT index i
            Long oy = strided ? f * yEws : mapOffsetAny(ym, i);
            cum = toCompute(fromCompute<TT>(cum + toCompute(y[oy])));
            if (prob <= cum || f == yLength - 1) {
                Long ox = strided ? f * xEws : mapOffsetAny(xm, f);
                z[oz] = x[ox];
                break;
            }
        }
    }
}

__global__ void __launch_bounds__(kBlock) rngDumpKernel(RngState st, Long start, Long n, u64 *out) {
    const Long stride = (Long)gridDim.x * kBlock;
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) out[i] = rngElement(st, start + i);
}

__global__ void __launch_bounds__(kBlock) copyKernel(uint4 *dst, const uint4 *src, Long nvec, unsigned char *dtail,
                                                     const unsigned char *stail, int tail) {
    const Long stride = (Long)gridDim.x * kBlock;
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += stride) dst[i] = src[i];
    if (blockIdx.x == 0 && (int)threadIdx.x < tail) dtail[threadIdx.x] = stail[threadIdx.x];
}

// Elements a block of the lean kernels takes (`positions` draws in all), or 0 when the call does not qualify: operands
// with element-wise strides, a buffer of at least one block's and fewer than 2^31 words, and every generation the
// draw can reach (the generator's own plus the buffer rounds up to its last position, plus one) below 2^31.
static Long leanElementsPerBlock(const RngState &st, const RandomPlan &pl, Long positions) {
    if (!pl.strided || st.size < kBlock || st.size >= (1LL << 31) || st.position < 0 || st.generation < 0) return 0;
    if (positions < 0 || st.position > (1LL << 62) - positions) return 0;
    const Long rounds = (st.position + positions) / st.size;
    if (st.generation > (1LL << 31) - 3 - rounds) return 0;
    const Long most = 8192;
    const Long fit = st.size / kBlock * kBlock;
    return fit < most ? fit : most;
}

template <typename T> struct RandomPlainBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const RandomCtx<T> &c, const T *x, const T *y, T *z, const RandomPlan &pl,
                        int operands) {
            const Long perBlock = leanElementsPerBlock(c.st, pl, pl.n);
            if (perBlock > 0 && (pl.n + perBlock - 1) / perBlock <= 0x7fffffffLL) {
                const dim3 lean((unsigned)((pl.n + perBlock - 1) / perBlock));
                const bool unit = pl.xEws == 1 && pl.yEws == 1 && pl.zEws == 1;
#define ND4J_LEAN(NOPS)                                                                                                          \
    do {                                                                                                                         \
        if (unit) ND4J_LAUNCH((randomLeanKernel<T, OP, NOPS, true>), lean, dim3(kBlock), 0, s, c, x, y, z, pl.xEws, pl.yEws, pl.zEws, perBlock); \
        else ND4J_LAUNCH((randomLeanKernel<T, OP, NOPS, false>), lean, dim3(kBlock), 0, s, c, x, y, z, pl.xEws, pl.yEws, pl.zEws, perBlock);     \
    } while (0)
                if (operands == 1) ND4J_LEAN(1);
                else if (operands == 2) ND4J_LEAN(2);
                else ND4J_LEAN(3);
#undef ND4J_LEAN
                return true;
            }
            int grid = gridFor(pl.n, kBlock * kRngIter, kMaxGrid);
            ND4J_LAUNCH((randomPlainKernel<T, OP>), dim3(grid), dim3(kBlock), 0, s, c, x, y, z, operands,
                               pl.strided ? 1 : 0, pl.xEws, pl.yEws, pl.zEws, pl.xm, pl.ym, pl.zm);
            return true;
        }
    };
};

template <typename T>
bool launchRandom(hipStream_t s, int opNum, const RngState &rng, const T *x, const T *y, T *z, const T *args,
                  const RandomPlan &pl, int operands, bool yIsZ) {
    if (opNum < 0 || opNum > 13) return false;
    if (pl.n <= 0) return true;
    RandomCtx<T> c;
    c.st = rng;
    c.args.p = args;
    c.length = pl.n;
    const bool special = opNum == 5 || opNum == 6 || (opNum >= 8 && opNum <= 11);
    if (special && operands == 3) {
        int yz = yIsZ ? 1 : 0;
        switch (opNum) {
            case 5: {
                int grid = gridFor(pl.n, kBlock, kGridCap);
                ND4J_LAUNCH((choiceKernel<T>), dim3(grid), dim3(kBlock), 0, s, c, x, y, z, pl.strided ? 1 : 0, pl.xEws,
                                   pl.yEws, pl.zEws, pl.xm, pl.ym, pl.zm, pl.yLength);
                break;
            }
            case 6:
            case 10: {
                const Long pairs = (pl.n + 1) / 2;
                // (an odd length draws one position beyond its last element's, like the reference)
                const Long perBlock = leanElementsPerBlock(c.st, pl, 2 * pairs) / 2 / kBlock * kBlock;
                if (perBlock > 0 && (pairs + perBlock - 1) / perBlock <= 0x7fffffffLL) {
                    const dim3 lean((unsigned)((pairs + perBlock - 1) / perBlock));
                    if (opNum == 6) ND4J_LAUNCH((gaussianLeanKernel<T, false>), lean, dim3(kBlock), 0, s, c, y, z, yz, pl.yEws, pl.zEws, perBlock);
                    else ND4J_LAUNCH((gaussianLeanKernel<T, true>), lean, dim3(kBlock), 0, s, c, y, z, yz, pl.yEws, pl.zEws, perBlock);
                    break;
                }
                int grid = gridFor(pairs, kBlock * kRngIter, kMaxGrid);
                if (opNum == 6) ND4J_LAUNCH((gaussianKernel<T, false>), dim3(grid), dim3(kBlock), 0, s, c, y, z, yz, pl.yEws, pl.zEws);
                else ND4J_LAUNCH((gaussianKernel<T, true>), dim3(grid), dim3(kBlock), 0, s, c, y, z, yz, pl.yEws, pl.zEws);
                break;
            }
            case 8: {
                int grid = gridFor(pl.n, kBlock, kGridCap);
                ND4J_LAUNCH((binomialKernel<T, false>), dim3(grid), dim3(kBlock), 0, s, c, y, z, yz, pl.yEws, pl.zEws);
                break;
            }
            case 9: {
                int grid = gridFor(pl.n, kBlock, kGridCap);
                ND4J_LAUNCH((binomialKernel<T, true>), dim3(grid), dim3(kBlock), 0, s, c, y, z, yz, pl.yEws, pl.zEws);
                break;
            }
            case 11: {
                int grid = gridFor((pl.n + 1) / 2, kBlock, kGridCap);
                ND4J_LAUNCH((truncatedNormalKernel<T>), dim3(grid), dim3(kBlock), 0, s, c, y, z, yz, pl.yEws, pl.zEws);
                break;
            }
        }
        return true;
    }
    return dispatchSeq<RandomPlainBody<T>::template Run>(opNum, std::make_integer_sequence<int, 14>{}, s, c, x, y, z, pl,
                                                         operands);
}

void launchRngDump(hipStream_t s, const RngState &rng, Long start, Long n, unsigned long long *out) {
    if (n <= 0) return;
    int grid = gridFor(n, kBlock * 4, kGridCap);
    ND4J_LAUNCH(rngDumpKernel, dim3(grid), dim3(kBlock), 0, s, rng, start, n, out);
}

void launchCopy(hipStream_t s, void *dst, const void *src, Long bytes) {
    if (bytes <= 0) return;
    Long nvec = bytes / 16;
    int tail = (int)(bytes - nvec * 16);
    int grid = gridFor(nvec > 0 ? nvec : 1, kBlock * 4, kGridCap);
    ND4J_LAUNCH(copyKernel, dim3(grid), dim3(kBlock), 0, s, reinterpret_cast<uint4 *>(dst),
                       reinterpret_cast<const uint4 *>(src), nvec, reinterpret_cast<unsigned char *>(dst) + nvec * 16,
                       reinterpret_cast<const unsigned char *>(src) + nvec * 16, tail);
}

__global__ void __launch_bounds__(kBlock) fillZeroKernel(uint4 *dst, Long nvec) {
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += (Long)gridDim.x * kBlock) dst[i] = make_uint4(0, 0, 0, 0);
}
void launchFill(hipStream_t s, void *dst, size_t bytes) {
    const Long nvec = (Long)(bytes / 16);
    if (nvec <= 0) return;
    ND4J_LAUNCH(fillZeroKernel, dim3(gridFor(nvec, kBlock, kGridCap)), dim3(kBlock), 0, s, reinterpret_cast<uint4 *>(dst), nvec);
}

#define INST(T)                                                                                                   \
    template bool launchRandom<T>(hipStream_t, int, const RngState &, const T *, const T *, T *, const T *,        \
                                  const RandomPlan &, int, bool);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
