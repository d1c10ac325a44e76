// Whole-array special transforms that travel through execTransform: SoftMax (38), SoftMaxDerivative (39),
// LogSoftMax (40) over the rows of a matrix or over a vector, and IsMax (41).
// Reference: include/ops/special_ops.h:1422-1573 (SoftMax), 1575-1730 (LogSoftMax), 1734-1943 (SoftMaxDerivative),
// 1945-2260 (IsMax); the CUDA back end runs the first three as five separate launches
// (blas/cuda/NativeOps.cu:3138-3252: max-reduce, subtract-broadcast, exp, sum-reduce, divide-broadcast).
//
// Here one launch does a row: maximum, sum of exp(x - max), then the result - exp is evaluated twice instead of
// being stored and read back, so a row costs one read of x from HBM (the second and third pass hit the caches
// for rows of ordinary length) and one write of z: 8 bytes per element instead of the chain's 32.
#include "elementwise.cuh"
#include "launch.h"
#include "reduce_engine.cuh"

namespace nd4j_amd {

template <typename C> struct MaxMerge {
    typedef C Acc;
    __device__ __forceinline__ C combine(C a, C b) const { return m::max_(a, b); }
};
template <typename C> struct SumMerge {
    typedef C Acc;
    __device__ __forceinline__ C combine(C a, C b) const { return a + b; }
};

template <typename C> __device__ __forceinline__ C laneBroadcast(C v, int srcLane, int width) {
    static_assert(sizeof(C) % 4 == 0, "compute type is a multiple of 4 bytes");
    constexpr int W = sizeof(C) / 4;
    struct Words { int w[W]; };
    Words in = __builtin_bit_cast(Words, v), out;
#pragma unroll
    for (int i = 0; i < W; i++) out.w[i] = __shfl(in.w[i], srcLane, width);
    return __builtin_bit_cast(C, out);
}

// MODE 0: softmax, 1: softmax * (1 - softmax), 2: log(softmax)
template <int MODE, typename C> __device__ __forceinline__ C softmaxFinish(C e, C sum) {
    C v = e / sum;
    if (MODE == 1) return v * ((C)1 - v);
    if (MODE == 2) return m::log_(v);
    return v;
}

// Rows whose elements are `xEl` / `zEl` apart, row r starting at r * xRow / r * zRow; GROUP lanes per row.
template <typename T, int MODE, int GROUP>
__global__ void __launch_bounds__(kBlock) softmaxRowKernel(const T *x, T *z, Long numRows, Long length, Long xRow, Long xEl,
                                                           Long zRow, Long zEl) {
    typedef typename Compute<T>::type C;
    constexpr int GROUPS = kBlock / GROUP;
    __shared__ C smem[kBlock / kWave];
    __shared__ C bcast;
    const int g = threadIdx.x / GROUP, lane = threadIdx.x % GROUP;
    for (Long r0 = (Long)blockIdx.x * GROUPS; r0 < numRows; r0 += (Long)gridDim.x * GROUPS) {
        const Long r = r0 + g;
        const bool live = r < numRows;
        const T *xr = x + (live ? r * xRow : 0);
        T *zr = z + (live ? r * zRow : 0);
        // FLOAT_MAX_VALUE of the reference's vector branch; rows of a matrix start from their first element there,
        // which gives the same maximum
        C mx = (C)-3.4028235e38;
        if (live)
            for (Long c = lane; c < length; c += GROUP) mx = m::max_(mx, toCompute(xr[c * xEl]));
        if (GROUP == kBlock) {
            MaxMerge<C> mg;
            mx = blockMerge<MaxMerge<C>>(mg, mx, smem);
            if (threadIdx.x == 0) bcast = mx;
            __syncthreads();
            mx = bcast;
        } else {
            MaxMerge<C> mg;
            mx = waveMerge<MaxMerge<C>, GROUP>(mg, mx);
            mx = laneBroadcast(mx, 0, GROUP);
        }
        C sum = (C)0;
        if (live)
            for (Long c = lane; c < length; c += GROUP) sum += m::exp_(toCompute(xr[c * xEl]) - mx);
        if (GROUP == kBlock) {
            SumMerge<C> mg;
            sum = blockMerge<SumMerge<C>>(mg, sum, smem);
            __syncthreads();
            if (threadIdx.x == 0) bcast = sum;
            __syncthreads();
            sum = bcast;
        } else {
            SumMerge<C> mg;
            sum = waveMerge<SumMerge<C>, GROUP>(mg, sum);
            sum = laneBroadcast(sum, 0, GROUP);
        }
        if (live)
            for (Long c = lane; c < length; c += GROUP)
                zr[c * zEl] = fromCompute<T>(softmaxFinish<MODE, C>(m::exp_(toCompute(xr[c * xEl]) - mx), sum));
        if (GROUP == kBlock) __syncthreads();
    }
}

// Rows that are adjacent in memory (an f-order matrix): lane <-> row, so a wave reads 64 neighbouring rows of one
// column at a time; the block's four waves split the columns and merge maximum and sum through LDS.
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock) softmaxColKernel(const T *x, T *z, Long numRows, Long length, Long xRow, Long xEl,
                                                           Long zRow, Long zEl) {
    typedef typename Compute<T>::type C;
    constexpr int WAVES = kBlock / kWave;
    __shared__ C smem[WAVES][kWave];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const Long r = (Long)blockIdx.x * kWave + lane;
    const bool live = r < numRows;
    const T *xr = x + (live ? r * xRow : 0);
    T *zr = z + (live ? r * zRow : 0);
    C mx = (C)-3.4028235e38;
    if (live) {
        Long c = wave;
        for (; c + 3 * WAVES < length; c += 4 * WAVES) {
            C v0 = toCompute(xr[c * xEl]), v1 = toCompute(xr[(c + WAVES) * xEl]), v2 = toCompute(xr[(c + 2 * WAVES) * xEl]),
              v3 = toCompute(xr[(c + 3 * WAVES) * xEl]);
            mx = m::max_(m::max_(mx, v0), m::max_(m::max_(v1, v2), v3));
        }
        for (; c < length; c += WAVES) mx = m::max_(mx, toCompute(xr[c * xEl]));
    }
    smem[wave][lane] = mx;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < WAVES; w++) mx = m::max_(mx, smem[w][lane]);
    __syncthreads();
    C sum = (C)0;
    if (live) {
        Long c = wave;
        for (; c + 3 * WAVES < length; c += 4 * WAVES) {
            C v0 = toCompute(xr[c * xEl]), v1 = toCompute(xr[(c + WAVES) * xEl]), v2 = toCompute(xr[(c + 2 * WAVES) * xEl]),
              v3 = toCompute(xr[(c + 3 * WAVES) * xEl]);
            sum += (m::exp_(v0 - mx) + m::exp_(v1 - mx)) + (m::exp_(v2 - mx) + m::exp_(v3 - mx));
        }
        for (; c < length; c += WAVES) sum += m::exp_(toCompute(xr[c * xEl]) - mx);
    }
    smem[wave][lane] = sum;
    __syncthreads();
    sum = (C)0;
#pragma unroll
    for (int w = 0; w < WAVES; w++) sum += smem[w][lane];
    if (live) {
        Long c = wave;
        for (; c + 3 * WAVES < length; c += 4 * WAVES) {
            C v0 = toCompute(xr[c * xEl]), v1 = toCompute(xr[(c + WAVES) * xEl]), v2 = toCompute(xr[(c + 2 * WAVES) * xEl]),
              v3 = toCompute(xr[(c + 3 * WAVES) * xEl]);
            zr[c * zEl] = fromCompute<T>(softmaxFinish<MODE, C>(m::exp_(v0 - mx), sum));
            zr[(c + WAVES) * zEl] = fromCompute<T>(softmaxFinish<MODE, C>(m::exp_(v1 - mx), sum));
            zr[(c + 2 * WAVES) * zEl] = fromCompute<T>(softmaxFinish<MODE, C>(m::exp_(v2 - mx), sum));
            zr[(c + 3 * WAVES) * zEl] = fromCompute<T>(softmaxFinish<MODE, C>(m::exp_(v3 - mx), sum));
        }
        for (; c < length; c += WAVES) zr[c * zEl] = fromCompute<T>(softmaxFinish<MODE, C>(m::exp_(toCompute(xr[c * xEl]) - mx), sum));
    }
}

template <typename T, int MODE> void runSoftmax(hipStream_t s, const T *x, T *z, const SoftmaxPlan &pl) {
    if (pl.numRows <= 0 || pl.length <= 0) return;
    if (pl.xRow == 1 && pl.zRow == 1 && pl.numRows >= kWave) {
        int grid = (int)((pl.numRows + kWave - 1) / kWave);
        hipLaunchKernelGGL((softmaxColKernel<T, MODE>), dim3(grid), dim3(kBlock), 0, s, x, z, pl.numRows, pl.length, pl.xRow, pl.xEl,
                           pl.zRow, pl.zEl);
        return;
    }
    if (pl.length >= 2048 || pl.numRows < 4) {
        int grid = gridFor(pl.numRows, 1, kGridCap);
        hipLaunchKernelGGL((softmaxRowKernel<T, MODE, kBlock>), dim3(grid), dim3(kBlock), 0, s, x, z, pl.numRows, pl.length, pl.xRow,
                           pl.xEl, pl.zRow, pl.zEl);
    } else if (pl.length >= 128) {
        int grid = gridFor(pl.numRows, kBlock / 64, kGridCap);
        hipLaunchKernelGGL((softmaxRowKernel<T, MODE, 64>), dim3(grid), dim3(kBlock), 0, s, x, z, pl.numRows, pl.length, pl.xRow,
                           pl.xEl, pl.zRow, pl.zEl);
    } else {
        int grid = gridFor(pl.numRows, kBlock / 16, kGridCap);
        hipLaunchKernelGGL((softmaxRowKernel<T, MODE, 16>), dim3(grid), dim3(kBlock), 0, s, x, z, pl.numRows, pl.length, pl.xRow,
                           pl.xEl, pl.zRow, pl.zEl);
    }
}

template <typename T> bool launchSoftmax(hipStream_t s, int opNum, const T *x, T *z, const SoftmaxPlan &pl) {
    switch (opNum) {
        case 38: runSoftmax<T, 0>(s, x, z, pl); return true;
        case 39: runSoftmax<T, 1>(s, x, z, pl); return true;
        case 40: runSoftmax<T, 2>(s, x, z, pl); return true;
        default: return false;
    }
}

// IsMax: z = 1 where the (first) maximum sits, 0 elsewhere.  `index` holds the winning position as the index
// reductions store it (in the data type): one value for the whole array, or one per TAD.
template <typename T>
__global__ void __launch_bounds__(kBlock) isMaxFillKernel(T *z, const T *index, Long n, int strided, Long ews, DimMap zm) {
    typedef typename Compute<T>::type C;
    const Long hit = (Long)toCompute(index[0]);
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += (Long)gridDim.x * kBlock) {
        const Long o = strided ? i * ews : mapOffset64(zm, (unsigned long long)i);
        z[o] = fromCompute<T>(i == hit ? (C)1 : (C)0);
    }
}
template <typename T>
__global__ void __launch_bounds__(kBlock) isMaxTadFillKernel(T *z, const T *index, const Long *offsets, Long tadLength, Long numTads,
                                                             int strided, Long tadEws, DimMap tm) {
    typedef typename Compute<T>::type C;
    const Long total = tadLength * numTads;
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < total; i += (Long)gridDim.x * kBlock) {
        const Long r = i / tadLength, f = i - r * tadLength;
        const Long o = offsets[r] + (strided ? f * tadEws : mapOffset64(tm, (unsigned long long)f));
        z[o] = fromCompute<T>(f == (Long)toCompute(index[r]) ? (C)1 : (C)0);
    }
}

template <typename T> void launchIsMaxFill(hipStream_t s, T *z, const T *index, const FlatPlan &zp) {
    if (zp.n <= 0) return;
    int grid = gridFor(zp.n, kBlock * 4, kGridCap);
    hipLaunchKernelGGL((isMaxFillKernel<T>), dim3(grid), dim3(kBlock), 0, s, z, index, zp.n, zp.strided ? 1 : 0, zp.ews, zp.xm);
}
template <typename T> void launchIsMaxTadFill(hipStream_t s, T *z, const T *index, const TadPlan &zt) {
    if (zt.numTads <= 0 || zt.tadLength <= 0) return;
    int grid = gridFor(zt.numTads * zt.tadLength, kBlock * 4, kGridCap);
    hipLaunchKernelGGL((isMaxTadFillKernel<T>), dim3(grid), dim3(kBlock), 0, s, z, index, zt.offsets, zt.tadLength, zt.numTads,
                       zt.kind == TadPlan::GENERAL ? 0 : 1, zt.tadEws, zt.tm);
}

#define INST(T)                                                                                           \
    template bool launchSoftmax<T>(hipStream_t, int, const T *, T *, const SoftmaxPlan &);                \
    template void launchIsMaxFill<T>(hipStream_t, T *, const T *, const FlatPlan &);                      \
    template void launchIsMaxTadFill<T>(hipStream_t, T *, const T *, const TadPlan &);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
