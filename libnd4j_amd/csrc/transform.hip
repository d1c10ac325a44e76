// Transform family: z = op(x, extraParams).  Reference loop: include/loops/cpu/transform.cpp:28-135.
#include "elementwise.cuh"
#include "launch.h"

namespace nd4j_amd {

template <typename T> struct TransformStridedBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const T *x, Long xs, T *z, Long zs, const T *extra, Long n) {
            if constexpr (TransformOp<OP>::valid) {
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
