// Transform family: z = op(x, extraParams).  Reference loop: include/loops/cpu/transform.cpp:28-135.
#include "elementwise.cuh"
#include "launch.h"

namespace nd4j_amd {

static constexpr int kWave = 64;

// ---- tanh (opNum 15) over contiguous float / half arrays -------------------------------
// The C library's tanhf, which the reference calls, is within 1 ULP of the correctly rounded value for |x| >= 1 but up to
// 2 ULP off below (its expm1-based quotient): a cheaper routine can stand in for it above 1 and stay within the 2 ULP
// allowed, below 1 only the library's own arithmetic can (lm::tanhf_, bit for bit, some 90 instructions).  So every
// element gets the cheap form, 1 - 2 / (exp(2|x|) + 1) on the hardware's exp2 and reciprocal, and the elements below 1
// (NaN too) are set aside: each wave packs theirs into a stretch of LDS, runs the exact routine over that stretch with
// all lanes busy, and hands the results back.  On inputs spread over [-4, 4] the exact routine then runs for a quarter
// of the elements instead of all.
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

static constexpr int kTanhPacks = 2;  // 16-byte vectors a lane holds per round
template <typename T>
__global__ void __launch_bounds__(kBlock) tanhVecKernel(const T *x, T *z, Long n, int head) {
    constexpr int VEC = Pack<T>::N, PACKS = kTanhPacks, kTanhPerLane = VEC * PACKS;
    __shared__ float aside[kBlock / kWave][kWave * VEC * PACKS];
    const int wave = threadIdx.x / kWave;
    float *mine = aside[wave];
    const Long nvec = (n - head) / VEC;
    const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x + head);
    Pack<T> *zv = reinterpret_cast<Pack<T> *>(z + head);
    const Long perRound = (Long)kBlock * PACKS;
    for (Long v0 = (Long)blockIdx.x * perRound; v0 < nvec; v0 += (Long)gridDim.x * perRound) {
        Pack<T> in[PACKS];
#pragma unroll
        for (int k = 0; k < PACKS; k++) {
            const Long v = v0 + k * kBlock + threadIdx.x;
            if (v < nvec) in[k] = loadPack(xv + v);
        }
        float res[kTanhPerLane];
        int slot[kTanhPerLane];  // where in the wave's stretch element e was put; -1: not set aside
        int count = 0;           // the wave's elements set aside so far (the same in every lane)
#pragma unroll
        for (int k = 0; k < PACKS; k++) {
            const bool have = v0 + k * kBlock + threadIdx.x < nvec;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                const float xe = toCompute(in[k].v[e]), ax = __builtin_fabsf(xe);
                res[k * VEC + e] = __builtin_copysignf(tanhAboveOne_(ax), xe);
                const bool small = have && !(ax >= 1.0f);
                const unsigned long long who = __builtin_amdgcn_ballot_w64(small);
                const int at = count + (int)__builtin_amdgcn_mbcnt_hi((unsigned)(who >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)who, 0u));
                slot[k * VEC + e] = small ? at : -1;
                if (small) mine[at] = xe;
                count += __builtin_popcountll(who);
            }
        }
        // (LDS accesses of one wave are served in order; the fences keep the compiler from moving them across)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        for (int t = threadIdx.x % kWave; t < count; t += kWave) mine[t] = lm::tanhf_(mine[t]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int i = 0; i < kTanhPerLane; i++)
            if (slot[i] >= 0) res[i] = mine[slot[i]];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < PACKS; k++) {
            const Long v = v0 + k * kBlock + threadIdx.x;
            if (v < nvec) {
                Pack<T> o;
#pragma unroll
                for (int e = 0; e < VEC; e++) o.v[e] = fromCompute<T>(res[k * VEC + e]);
                storePack(zv + v, o);
            }
        }
    }
    // the elements before the first and after the last whole vector
    const Long gtid = (Long)blockIdx.x * kBlock + threadIdx.x;
    const Long tailStart = head + nvec * VEC;
    if (gtid < head + (n - tailStart)) {
        const Long i = gtid < head ? gtid : tailStart + (gtid - head);
        z[i] = fromCompute<T>(lm::tanhf_(toCompute(x[i])));
    }
}

// true when the call was taken: contiguous float or half operands that share one misalignment
template <typename T> bool launchTanhVec(hipStream_t s, const T *x, Long xs, T *z, Long zs, Long n) {
    if constexpr (sizeof(T) == 8) {
        return false;
    } else {
        if (xs != 1 || zs != 1 || n <= 0) return false;
        int head = commonHead<T>(x, nullptr, z);
        if (head < 0) return false;
        if (head > n) head = (int)n;
        const Long nvec = (n - head) / Pack<T>::N;
        const int grid = gridFor(nvec > 0 ? nvec : 1, (Long)kBlock * kTanhPacks, kMaxGrid);
        ND4J_LAUNCH((tanhVecKernel<T>), dim3(grid), dim3(kBlock), 0, s, x, z, n, head);
        return true;
    }
}

template <typename T> struct TransformStridedBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const T *x, Long xs, T *z, Long zs, const T *extra, Long n) {
            if constexpr (TransformOp<OP>::valid) {
                // (the derivative 1 - tanh^2 keeps the exact routine throughout: near saturation one ULP of tanh is a
                // multiple of the result)
                if constexpr (OP == 15) {
                    if (launchTanhVec<T>(s, x, xs, z, zs, n)) return true;
                }
                launchStrided<T, TransformF<OP>>(s, x, xs, nullptr, 0, z, zs, extra, n);
                return true;
            } else {
                return false;
            }
        }
    };
};
template <typename T> struct TransformGeneralBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const T *x, const DimMap &xm, T *z, const DimMap &zm, const T *extra, Long n) {
            if constexpr (TransformOp<OP>::valid) {
                launchGeneral<T, TransformF<OP>>(s, x, xm, nullptr, xm, z, zm, extra, n);
                return true;
            } else {
                return false;
            }
        }
    };
};

template <typename T>
bool launchTransformStrided(hipStream_t s, int opNum, const T *x, Long xs, T *z, Long zs, const T *extra, Long n) {
    return dispatchSeq<TransformStridedBody<T>::template Run>(opNum, std::make_integer_sequence<int, kTransformOpCount>{},
                                                              s, x, xs, z, zs, extra, n);
}
template <typename T>
bool launchTransformGeneral(hipStream_t s, int opNum, const T *x, const DimMap &xm, T *z, const DimMap &zm,
                            const T *extra, Long n) {
    return dispatchSeq<TransformGeneralBody<T>::template Run>(opNum, std::make_integer_sequence<int, kTransformOpCount>{},
                                                              s, x, xm, z, zm, extra, n);
}

#define INST(T)                                                                                                  \
    template bool launchTransformStrided<T>(hipStream_t, int, const T *, Long, T *, Long, const T *, Long);      \
    template bool launchTransformGeneral<T>(hipStream_t, int, const T *, const DimMap &, T *, const DimMap &,    \
                                            const T *, Long);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
