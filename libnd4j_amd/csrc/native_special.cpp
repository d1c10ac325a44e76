// NativeOps boundary, part 4: the data-movement specials - flatten, concat, pullRows, tear, shuffle and the
// conversions between half, float and double.  Pointer conventions are those of the reference's CUDA back end:
//   flatten   blas/cuda/NativeOps.cu:3764-3860   (extraPointers[7] = host shapeInfo of the input)
//   concat    blas/cuda/NativeOps.cu:4417-4515   (data[0] / inputShapeInfo[0] = device tables of device pointers,
//                                                 extraPointers[0] = host shapeInfo of the result,
//                                                 extraPointers[9] = host table of host shapeInfo pointers)
//   pullRows  blas/cuda/NativeOps.cu:4833-4861, tear 5560-5584, shuffle 4991-5035 (every argument a device pointer,
//             the tables of pointers included)
//   convert   include/loops/type_conversions.h:38-49, 696-850
#include <cstdio>

#include "../../include/NativeOps.h"
#include "runtime.h"

using namespace nd4j_amd;

namespace {

constexpr int kIdentity = 27;  // TRANSFORM_OPS Identity: z = x

template <typename T>
void flattenImpl(Nd4jPointer *extra, int offset, char order, T *result, Long *resultInfo, T *input, Long *inputInfo) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_Y_SHAPE, inputInfo, sx, s);
    if (hx == nullptr) return;
    const Long n = siNumel(hx);
    if (n <= 0) return;
    const Long xe = siEws(hx);
    T *z = result + offset;
    bool ok;
    if (siOrder(hx) == order && xe >= 1) {
        // same order on both sides: the input's memory order is the requested order.  Only this branch honours the
        // result's element-wise stride; no slot carries a host copy of the result's shapeInfo, so unless the argument
        // itself is host memory the kernel reads the field
        if (resultInfo == nullptr || !isDeviceMemory(resultInfo)) {
            const Long ze = (resultInfo != nullptr && siEws(resultInfo) >= 1) ? siEws(resultInfo) : 1;
            ok = launchTransformStrided<T>(s, kIdentity, input, xe, z, ze, nullptr, n);
        } else {
            launchCopyToEws<T>(s, input, xe, z, resultInfo, n);
            ok = true;
        }
    } else {
        // walk the input in the requested order (F order = C order over the reversed dimensions), write densely
        const int rank = siRank(hx);
        Long shp[kMaxRank], str[kMaxRank];
        for (int i = 0; i < rank; i++) {
            const int d = order == 'f' ? rank - 1 - i : i;
            shp[i] = siShape(hx)[d];
            str[i] = siStride(hx)[d];
        }
        DimMap xm, zm;
        ownCanon(rank, shp, str, xm);
        if (xm.rank == 2 && xm.stride[0] == 1 && xm.stride[1] >= (Long)xm.shape[0]) {
            // the input runs along the slower dimension of the requested order: a matrix transpose
            launchTransposeCopy<T>(s, input, z, xm.shape[0], xm.shape[1], xm.stride[1], xm.shape[1]);
            checkLaunch("flatten", s);
            return;
        }
        zm.rank = 1;
        zm.shape[0] = (unsigned)(n > 0xffffffffLL ? 0xffffffffu : n);
        zm.stride[0] = 1;
        ok = launchTransformGeneral<T>(s, kIdentity, input, xm, z, zm, nullptr, n);
    }
    if (!ok) { reportUnknownOp("flatten", kIdentity); return; }
    checkLaunch("flatten", s);
}

template <typename T>
void concatImpl(Nd4jPointer *extra, int dimension, int numArrays, Nd4jPointer *data, Nd4jPointer *inputShapeInfo, T *result,
                Long *resultInfo) {
    hipStream_t s = streamOf(extra);
    if (numArrays <= 0 || data == nullptr || inputShapeInfo == nullptr) return;
    std::vector<Long> sz;
    const Long *hz = hostShapeInfo(extra, X_HOST_X_SHAPE, resultInfo, sz, s);
    if (hz == nullptr) return;
    const int rank = siRank(hz);
    if (dimension < 0) dimension += rank;
    if (dimension < 0 || dimension >= rank) throw std::runtime_error("concat: dimension out of range");
    ConcatView v;
    v.rank = rank;
    v.dim = dimension;
    v.zContig = (siOrder(hz) == 'c' && siEws(hz) == 1) ? 1 : 0;
    v.inner = 1;
    for (int d = 0; d < rank; d++) {
        v.zStride[d] = siStride(hz)[d];
        if (d > dimension) v.inner *= siShape(hz)[d];
    }
    v.dimTotal = siShape(hz)[dimension];
    // the largest input bounds the grid; without the host table of input shapes the result's length does
    Long maxLength = siNumel(hz);
    if (Long **hostShapes = reinterpret_cast<Long **>(slotOf(extra, X_HOST_TAD_SHAPE))) {
        maxLength = 0;
        for (int i = 0; i < numArrays; i++)
            if (hostShapes[i] != nullptr && siNumel(hostShapes[i]) > maxLength) maxLength = siNumel(hostShapes[i]);
    }
    Workspace ws = workspaceFor(s, concatScratchBytes(numArrays));
    launchConcat<T>(s, reinterpret_cast<const T *const *>(data[0]), reinterpret_cast<const Long *const *>(inputShapeInfo[0]), result,
                    v, numArrays, maxLength, ws.ptr);
    checkLaunch("concat", s);
}

template <typename T>
void pullRowsImpl(Nd4jPointer *extra, T *x, T *z, Long n, Long *indexes, Long *tadInfo, Long *tadOffsets, Long *zTadInfo,
                  Long *zTadOffsets) {
    hipStream_t s = streamOf(extra);
    launchPullRows<T>(s, x, z, n, indexes, tadInfo, tadOffsets, zTadInfo, zTadOffsets);
    checkLaunch("pullRows", s);
}

template <typename T>
void tearImpl(Nd4jPointer *extra, T *x, Long *xInfo, Nd4jPointer *targets, Long *zInfo, Long *tadInfo, Long *tadOffsets) {
    hipStream_t s = streamOf(extra);
    launchTear<T>(s, x, xInfo, reinterpret_cast<T *const *>(targets), zInfo, tadInfo, tadOffsets, 0);
    checkLaunch("tear", s);
}

template <typename T>
void shuffleImpl(Nd4jPointer *extra, Nd4jPointer *dx, Nd4jPointer *xInfo, Nd4jPointer *dz, int N, int *shuffleMap,
                 Nd4jPointer *tadInfo, Nd4jPointer *tadOffsets) {
    hipStream_t s = streamOf(extra);
    launchShuffle<T>(s, reinterpret_cast<T *const *>(dx), reinterpret_cast<const Long *const *>(xInfo),
                     reinterpret_cast<T *const *>(dz), N, shuffleMap, reinterpret_cast<const Long *const *>(tadInfo),
                     reinterpret_cast<const Long *const *>(tadOffsets), 0);
    checkLaunch("shuffle", s);
}

}  // namespace

#define ND4J_SPECIAL_MEMBERS(SUFFIX, T)                                                                                  \
    void NativeOps::flatten##SUFFIX(Nd4jPointer *extraPointers, int offset, char order, T *result,                       \
                                    Nd4jLong *resultShapeInfo, T *input, Nd4jLong *inputShapeInfo) {                     \
        flattenImpl<T>(extraPointers, offset, order, result, resultShapeInfo, input, inputShapeInfo);                    \
    }                                                                                                                    \
    void NativeOps::concat##SUFFIX(Nd4jPointer *extraPointers, int dimension, int numArrays, Nd4jPointer *data,          \
                                   Nd4jPointer *inputShapeInfo, T *result, Nd4jLong *resultShapeInfo,                    \
                                   Nd4jPointer *tadPointers, Nd4jPointer *offsetPointers) {                              \
        (void)tadPointers; (void)offsetPointers; /* the kernel derives what it needs from the shapeInfos */              \
        concatImpl<T>(extraPointers, dimension, numArrays, data, inputShapeInfo, result, resultShapeInfo);               \
    }                                                                                                                    \
    void NativeOps::pullRows##SUFFIX(Nd4jPointer *extraPointers, T *x, Nd4jLong *xShapeInfo, T *z,                       \
                                     Nd4jLong *zShapeInfo, Nd4jLong n, Nd4jLong *indexes, Nd4jLong *tadShapeInfo,        \
                                     Nd4jLong *tadOffsets, Nd4jLong *zTadShapeInfo, Nd4jLong *zTadOffsets) {             \
        (void)xShapeInfo; (void)zShapeInfo;                                                                              \
        pullRowsImpl<T>(extraPointers, x, z, n, indexes, tadShapeInfo, tadOffsets, zTadShapeInfo, zTadOffsets);          \
    }                                                                                                                    \
    void NativeOps::tear##SUFFIX(Nd4jPointer *extraPointers, T *x, Nd4jLong *xShapeInfo, Nd4jPointer *targets,           \
                                 Nd4jLong *zShapeInfo, Nd4jLong *tadShapeInfo, Nd4jLong *tadOffsets) {                   \
        tearImpl<T>(extraPointers, x, xShapeInfo, targets, zShapeInfo, tadShapeInfo, tadOffsets);                        \
    }                                                                                                                    \
    void NativeOps::shuffle##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, Nd4jPointer *xShapeInfo, Nd4jPointer *dz,      \
                                    Nd4jPointer *zShapeInfo, int N, int *shuffleMap, Nd4jPointer *tadShapeInfo,          \
                                    Nd4jPointer *tadOffsets) {                                                           \
        (void)zShapeInfo;                                                                                                \
        shuffleImpl<T>(extras, dx, xShapeInfo, dz, N, shuffleMap, tadShapeInfo, tadOffsets);                             \
    }

#define ND4J_AVERAGE_MEMBERS(SUFFIX, T)                                                                                  \
    void NativeOps::average##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, T *dz, int n, Nd4jLong length, bool propagate) { \
        hipStream_t s = streamOf(extras);                                                                                \
        launchAverage<T>(s, reinterpret_cast<T *const *>(dx), dz, n, length, true, propagate);                           \
        checkLaunch("average", s);                                                                                       \
    }                                                                                                                    \
    void NativeOps::accumulate##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, T *dz, int n, Nd4jLong length) {            \
        hipStream_t s = streamOf(extras);                                                                                \
        launchAverage<T>(s, reinterpret_cast<T *const *>(dx), dz, n, length, false, false);                              \
        checkLaunch("accumulate", s);                                                                                    \
    }
ND4J_AVERAGE_MEMBERS(Float, float)
ND4J_AVERAGE_MEMBERS(Half, float16)
ND4J_AVERAGE_MEMBERS(Double, double)

ND4J_SPECIAL_MEMBERS(Float, float)
ND4J_SPECIAL_MEMBERS(Half, float16)
ND4J_SPECIAL_MEMBERS(Double, double)

// Device buffers only: the reference's member is a host loop over host memory, which stays with the host library.
void NativeOps::convertTypes(Nd4jPointer *extras, int srcType, Nd4jPointer x, Nd4jLong N, int dstType, Nd4jPointer z) {
    hipStream_t s = streamOf(extras);
    if (N <= 0) return;
    if (!isDeviceMemory(x) || !isDeviceMemory(z)) {
        std::printf("convertTypes: host buffers are not on this path\n");
        return;
    }
    if (!launchConvert(s, srcType, x, N, dstType, z)) {
        std::printf("Unsupported types conversion: [%i] -> [%i]\n", srcType, dstType);
        return;
    }
    checkLaunch("convertTypes", s);
}
