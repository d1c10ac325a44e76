// Scalar family: z = op(x, scalar, extraParams), the scalar either one value for the whole array (passed by
// value) or one value per TAD along `dimension`.  Reference loops: include/loops/cpu/scalar.cpp:14-62 (per
// TAD), 121-215 (shaped), 218-285 (strided); opNum table include/loops/legacy_ops.h SCALAR_OPS.
#include "elementwise.cuh"
#include "launch.h"

namespace nd4j_amd {

template <typename T> struct ScalarStridedBody {
    template <int KIND> struct Run {
        static bool run(hipStream_t s, const T *x, Long xs, T *z, Long zs, typename Compute<T>::type scalar, const T *extra,
                        Long n) {
            launchStrided<T, Scalar3F<KIND>>(s, x, xs, nullptr, 0, z, zs, extra, n, scalar);
            return true;
        }
    };
};
template <typename T> struct ScalarGeneralBody {
    template <int KIND> struct Run {
        static bool run(hipStream_t s, const T *x, const DimMap &xm, T *z, const DimMap &zm,
                        typename Compute<T>::type scalar, const T *extra, Long n) {
            launchGeneral<T, Scalar3F<KIND>>(s, x, xm, nullptr, xm, z, zm, extra, n, scalar);
            return true;
        }
    };
};
template <typename T> struct ScalarTadBody {
    template <int KIND> struct Run {
        static bool run(hipStream_t s, const T *x, const T *scalars, T *z, const T *extra, const BroadcastPlan &pl) {
            typedef ScalarTad3F<KIND> F;
            if (pl.numTads <= 0 || pl.tadLength <= 0) return true;
            Params<T> p{extra};
            if (pl.flatInner > 0 && pl.flatInner < 0xffffffffLL && pl.flatExtent < 0xffffffffLL &&
                (((uintptr_t)x | (uintptr_t)z) & 15) == 0) {
                const Long n = pl.numTads * pl.tadLength;
                ND4J_LAUNCH((bcFlatInnerKernel<T, F>), dim3(gridFor(n / Pack<T>::N + 1, kBlock, F::tables ? kGridCap : kMaxGrid)),
                                   dim3(kBlock), 0, s, x, scalars, z, n, pl.flatInner, pl.flatExtent, p);
                return true;
            }
            if (pl.kind == BroadcastPlan::ROW) {
                constexpr int VEC = Pack<T>::N;
                Long vecsPerTad = (pl.tadLength + VEC - 1) / VEC;
                int colShift = 0;
                while ((1 << colShift) < kBlock && (1LL << colShift) < vecsPerTad) colShift++;
                const int colThreads = 1 << colShift, rowsPerBlock = kBlock >> colShift;
                Long gy = (vecsPerTad + colThreads - 1) / colThreads;
                if (gy > 65535) gy = 65535;
                int gx = gridFor(pl.numTads, (Long)rowsPerBlock * kBcRows, kMaxGrid);
                int aligned = (((uintptr_t)x | (uintptr_t)z) & 15) == 0 ? 1 : 0;
                ND4J_LAUNCH((bcRowKernel<T, F, true>), dim3(gx, (unsigned)gy), dim3(kBlock), 0, s, x, scalars, z,
                                   pl.xOffsets, pl.zOffsets, pl.tadLength, pl.numTads, aligned, colShift, p);
            } else {
                int gx = (int)((pl.numTads + kBlock - 1) / kBlock);
                Long gy = (Long)kGridCap / gx;
                if (gy < 1) gy = 1;
                if (gy > pl.tadLength) gy = pl.tadLength;
                if (gy > 65535) gy = 65535;
                ND4J_LAUNCH((bcColKernel<T, F, true>), dim3(gx, (unsigned)gy), dim3(kBlock), 0, s, x, scalars, z,
                                   pl.xOffsets, pl.zOffsets, pl.tadLength, pl.numTads, pl.tadEws, (Long)0, pl.zEws, p);
            }
            return true;
        }
    };
};

template <typename T>
bool launchScalarStrided(hipStream_t s, int opNum, const T *x, Long xs, T *z, Long zs, typename Compute<T>::type scalar,
                         const T *extra, Long n) {
    int kind = scalarKind(opNum);
    if (kind == B_Invalid) return false;
    return dispatchSeq<ScalarStridedBody<T>::template Run>(kind, std::make_integer_sequence<int, B_FMod + 1>{}, s, x, xs, z,
                                                           zs, scalar, extra, n);
}
template <typename T>
bool launchScalarGeneral(hipStream_t s, int opNum, const T *x, const DimMap &xm, T *z, const DimMap &zm,
                         typename Compute<T>::type scalar, const T *extra, Long n) {
    int kind = scalarKind(opNum);
    if (kind == B_Invalid) return false;
    return dispatchSeq<ScalarGeneralBody<T>::template Run>(kind, std::make_integer_sequence<int, B_FMod + 1>{}, s, x, xm, z,
                                                           zm, scalar, extra, n);
}
template <typename T>
bool launchScalarTad(hipStream_t s, int opNum, const T *x, const T *scalars, T *z, const T *extra,
                     const BroadcastPlan &plan) {
    int kind = scalarKind(opNum);
    if (kind == B_Invalid) return false;
    return dispatchSeq<ScalarTadBody<T>::template Run>(kind, std::make_integer_sequence<int, B_FMod + 1>{}, s, x, scalars, z,
                                                       extra, plan);
}

#define INST(T)                                                                                                     \
    template bool launchScalarStrided<T>(hipStream_t, int, const T *, Long, T *, Long, Compute<T>::type, const T *, \
                                         Long);                                                                     \
    template bool launchScalarGeneral<T>(hipStream_t, int, const T *, const DimMap &, T *, const DimMap &,          \
                                         Compute<T>::type, const T *, Long);                                        \
    template bool launchScalarTad<T>(hipStream_t, int, const T *, const T *, T *, const T *, const BroadcastPlan &);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
