// Pairwise family: z = op(x, y, extraParams).  Reference loop: include/loops/pairwise_transform.h:154-424.
#include "elementwise.cuh"
#include "launch.h"

namespace nd4j_amd {

template <typename T> struct PairwiseStridedBody {
    template <int KIND> struct Run {
        static bool run(hipStream_t s, const T *x, Long xs, const T *y, Long ys, T *z, Long zs, const T *extra, Long n) {
            launchStrided<T, Pairwise3F<KIND>>(s, x, xs, y, ys, z, zs, extra, n);
            return true;
        }
    };
};
template <typename T> struct PairwiseGeneralBody {
    template <int KIND> struct Run {
        static bool run(hipStream_t s, const T *x, const DimMap &xm, const T *y, const DimMap &ym, T *z,
                        const DimMap &zm, const T *extra, Long n) {
            launchGeneral<T, Pairwise3F<KIND>>(s, x, xm, y, ym, z, zm, extra, n);
            return true;
        }
    };
};

template <typename T>
bool launchPairwiseStrided(hipStream_t s, int opNum, const T *x, Long xs, const T *y, Long ys, T *z, Long zs,
                           const T *extra, Long n) {
    int kind = pairwiseKind(opNum);
    if (kind == B_Invalid) return false;
    return dispatchSeq<PairwiseStridedBody<T>::template Run>(kind, std::make_integer_sequence<int, B_Invalid>{}, s, x, xs,
                                                             y, ys, z, zs, extra, n);
}
template <typename T>
bool launchPairwiseGeneral(hipStream_t s, int opNum, const T *x, const DimMap &xm, const T *y, const DimMap &ym, T *z,
                           const DimMap &zm, const T *extra, Long n) {
    int kind = pairwiseKind(opNum);
    if (kind == B_Invalid) return false;
    return dispatchSeq<PairwiseGeneralBody<T>::template Run>(kind, std::make_integer_sequence<int, B_Invalid>{}, s, x, xm,
                                                             y, ym, z, zm, extra, n);
}

#define INST(T)                                                                                                   \
    template bool launchPairwiseStrided<T>(hipStream_t, int, const T *, Long, const T *, Long, T *, Long,         \
                                           const T *, Long);                                                      \
    template bool launchPairwiseGeneral<T>(hipStream_t, int, const T *, const DimMap &, const T *, const DimMap &, \
                                           T *, const DimMap &, const T *, Long);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
