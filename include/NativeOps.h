// class NativeOps - the drop-in surface of the legacy op-execution path.
//
// Same class name, member names, argument order and POD argument types as the reference's
// blas/NativeOps.h.  The members on the hot path (transform, pairwise, broadcast, scalar, reduce, reduce3,
// index-reduce, summary-stats, random, the data-movement specials) and the lifecycle members a host needs
// around them do their work; every other member of the reference's class is declared at the end and
// defined as a stub.  A JavaCPP binding generated against the reference header resolves all of them to the
// same Itanium-mangled symbols in libnd4j_amd.so.
//
// Calling convention = the reference's CUDA backend (blas/cuda/NativeOps.cu):
//   * data pointers, shapeInfo arguments, `dimension` and `extraParams` are DEVICE pointers;
//   * extraPointers[0] host xShapeInfo, [1] the HIP stream handle by value, [2] device id,
//     [3] allocation scratch (unused here), [4] reduction scratch (unused here), [5] host-visible scalar
//     result (unused: scalars are returned by value; the library hands them over through pinned host memory
//     of its own, see below), [7] host yShapeInfo,
//     [8] host zShapeInfo, [9] host TAD shapeInfo, [10] device TAD shapeInfo, [11] device TAD offsets,
//     [12]/[13] device TAD shapeInfo/offsets of the result (broadcast);
//   * array results are enqueued on the stream and the call returns; scalar-returning members return once the
//     value has arrived: the last kernel writes it, tagged with the call's ticket, into pinned host memory that
//     the library keeps per (device, stream), and the host waits for those words (asking the stream as well after
//     50 us, and handing over to a stream synchronisation after 300 us, or at once in debug mode).  Everything
//     enqueued earlier on the stream has completed by then, as after a synchronisation.
//   * one host thread per stream at a time: the scalar slot, its tickets and the stream's scratch memory are per
//     (device, stream) and not shared safely between threads that use one stream (the null stream included).
//   * enableDebugMode synchronises after every launch and reports asynchronous errors; with enableVerboseMode on
//     as well every kernel launch prints its name and launch dimensions.  setOmpNumThreads / setOmpMinThreads,
//     setGridLimit, setElementThreshold and setTADThreshold store their values for the getters and tune nothing:
//     launch geometry here follows the operand shapes.
//   Missing host copies ([0],[7],[8],[9] null) are fetched from the device pointers, and missing TAD
//   tables are computed and cached by the library, at the price of a stream synchronise.
#pragma once

#include "nd4j_types.h"

#include <string>

// Return types of three graph members that are only declared here (see "Members outside the path" below)
namespace nd4j {
class ShapeList;
namespace graph {
template <typename T> class VariablesSet;
}
}  // namespace nd4j

#ifndef ND4J_EXPORT
#define ND4J_EXPORT __attribute__((visibility("default")))
#endif

// One block of members per data type: SUFFIX in {Float, Half, Double}, T in {float, float16, double},
// R the scalar return type (float for Float and Half, double for Double).
#define ND4J_EXEC_MEMBERS(SUFFIX, T, R)                                                                         \
    /* reference: blas/NativeOps.h:544-602 (Float/Half), 80-113 (Double) */                                      \
    R execIndexReduceScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,          \
                                    T *extraParams);                                                             \
    void execIndexReduce##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,             \
                                 T *extraParams, T *result, Nd4jLong *resultShapeInfoBuffer, int *dimension,     \
                                 int dimensionLength);                                                           \
    /* reference: blas/NativeOps.h:615-649, 115-139 */                                                           \
    void execBroadcast##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *y,         \
                               Nd4jLong *yShapeInfo, T *result, Nd4jLong *resultShapeInfo, int *dimension,       \
                               int dimensionLength);                                                             \
    /* reference: blas/NativeOps.h:665-798, 141-210: strided, indexed (a no-op in both reference back ends:    \
       blas/cuda/NativeOps.cu:1928-1960) and shaped overloads */                                                 \
    void execPairwiseTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong xStride, T *y,    \
                                       Nd4jLong yStride, T *result, Nd4jLong resultStride, T *extraParams,       \
                                       Nd4jLong n);                                                              \
    void execPairwiseTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong *xShapeInfo,      \
                                       T *y, Nd4jLong *yShapeInfo, T *result, Nd4jLong *resultShapeInfo,         \
                                       T *extraParams, Nd4jLong *xIndexes, Nd4jLong *yIndexes,                   \
                                       Nd4jLong *resultIndexes);                                                 \
    void execPairwiseTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong *xShapeInfo,      \
                                       T *y, Nd4jLong *yShapeInfo, T *result, Nd4jLong *resultShapeInfo,         \
                                       T *extraParams);                                                          \
    /* reference: blas/NativeOps.h:809-906, 212-250 */                                                           \
    void execReduce##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *extraParams,  \
                            T *result, Nd4jLong *resultShapeInfo);                                               \
    void execReduce##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *extraParams,  \
                            T *result, Nd4jLong *resultShapeInfo, int *dimension, int dimensionLength);          \
    R execReduceScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,               \
                               T *extraParams);                                                                  \
    /* reference: blas/NativeOps.h:1223-1325, 438-490 */                                                         \
    R execSummaryStatsScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,         \
                                     T *extraParams, bool biasCorrected);                                        \
    void execSummaryStats##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,            \
                                  T *extraParams, T *result, Nd4jLong *resultShapeInfo, bool biasCorrected);     \
    void execSummaryStats##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,            \
                                  T *extraParams, T *result, Nd4jLong *resultShapeInfoBuffer, int *dimension,    \
                                  int dimensionLength, bool biasCorrected);                                      \
    /* reference: blas/NativeOps.h:1337-1443, 492-542: strided, shaped and indexed (no-op:                      \
       blas/cuda/NativeOps.cu:3598-3612) overloads */                                                            \
    void execTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong xStride, T *result,       \
                               Nd4jLong resultStride, T *extraParams, Nd4jLong n);                               \
    void execTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong *xShapeInfo, T *result,   \
                               Nd4jLong *resultShapeInfo, T *extraParams);                                       \
    void execTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong *xShapeInfo, T *result,   \
                               Nd4jLong *resultShapeInfo, T *extraParams, Nd4jLong *xIndexes,                    \
                               Nd4jLong *resultIndexes);                                                         \
    /* reference: blas/NativeOps.h:2327-2498: (z), (x,y,z) and (x,z) overloads; `state` is the pointer        \
       returned by initRandom */                                                                                 \
    void execRandom##SUFFIX(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *z,                     \
                            Nd4jLong *zShapeBuffer, T *extraArguments);                                          \
    void execRandom##SUFFIX(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *x,                     \
                            Nd4jLong *xShapeBuffer, T *y, Nd4jLong *yShapeBuffer, T *z, Nd4jLong *zShapeBuffer,  \
                            T *extraArguments);                                                                  \
    void execRandom##SUFFIX(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *x,                     \
                            Nd4jLong *xShapeBuffer, T *z, Nd4jLong *zShapeBuffer, T *extraArguments);

// Scalar family, reference: blas/NativeOps.h:1046-1146 and 1160-1226 (Float / Half), 377-440 and 1183-1203
// (Double): strided, shaped, indexed (launches nothing in the reference's CUDA back end:
// blas/cuda/NativeOps.cu:2788-2816) and one-scalar-per-TAD overloads.  S is the by-value scalar type.
#define ND4J_SCALAR_MEMBERS(SUFFIX, T, S)                                                                       \
    void execScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong xStride, T *result,           \
                            Nd4jLong resultStride, S scalar, T *extraParams, Nd4jLong n);                        \
    void execScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *result,       \
                            Nd4jLong *resultShapeInfo, S scalar, T *extraParams);                                \
    void execScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *result,       \
                            Nd4jLong *resultShapeInfo, S scalar, T *extraParams, Nd4jLong *xIndexes,             \
                            Nd4jLong *resultIndexes);                                                            \
    void execScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *z,            \
                            Nd4jLong *zShapeInfo, T *scalars, T *extraParams, int *dimension,                    \
                            int dimensionLength);

// Reduce3 family (two inputs, one number per pair of runs), reference: blas/NativeOps.h:919-1044 (Float / Half),
// 252-362 (Double and the all-pairs variant): whole arrays into result[0], whole arrays returned by value,
// along `dimension`, and every TAD of x against every TAD of y.
// Data-movement specials, reference: blas/NativeOps.h:1457-1499 (flatten), 1510-1555 (concat), 1904-1967
// (pullRows), 2076-2130 (shuffle), 2876-2899 (tear).  Pointer conventions of the CUDA back end: concat takes
// data[0] / inputShapeInfo[0] = device tables of device pointers, the result's host shapeInfo in extraPointers[0]
// and (optionally) a host table of the inputs' host shapeInfos in extraPointers[9]; tadPointers / offsetPointers
// are accepted and not needed.  flatten takes the input's host shapeInfo in extraPointers[7].  For pullRows, tear
// and shuffle every argument, the tables of pointers included, is a device pointer.  shuffle swaps TAD r with TAD
// shuffleMap[r] (entries < 0 are skipped; the pairs of one map must be disjoint) in each of the N arrays.
#define ND4J_SPECIAL_MEMBERS(SUFFIX, T)                                                                          \
    void flatten##SUFFIX(Nd4jPointer *extraPointers, int offset, char order, T *result, Nd4jLong *resultShapeInfo, \
                         T *input, Nd4jLong *inputShapeInfo);                                                    \
    void concat##SUFFIX(Nd4jPointer *extraPointers, int dimension, int numArrays, Nd4jPointer *data,             \
                        Nd4jPointer *inputShapeInfo, T *result, Nd4jLong *resultShapeInfo,                       \
                        Nd4jPointer *tadPointers, Nd4jPointer *offsetPointers);                                  \
    void pullRows##SUFFIX(Nd4jPointer *extraPointers, T *x, Nd4jLong *xShapeInfo, T *z, Nd4jLong *zShapeInfo,    \
                          Nd4jLong n, Nd4jLong *indexes, Nd4jLong *tadShapeInfo, Nd4jLong *tadOffsets,           \
                          Nd4jLong *zTadShapeInfo, Nd4jLong *zTadOffsets);                                       \
    void tear##SUFFIX(Nd4jPointer *extraPointers, T *x, Nd4jLong *xShapeInfo, Nd4jPointer *targets,              \
                      Nd4jLong *zShapeInfo, Nd4jLong *tadShapeInfo, Nd4jLong *tadOffsets);                       \
    void shuffle##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, Nd4jPointer *xShapeInfo, Nd4jPointer *dz,         \
                         Nd4jPointer *zShapeInfo, int N, int *shuffleMap, Nd4jPointer *tadShapeInfo,             \
                         Nd4jPointer *tadOffsets);

#define ND4J_REDUCE3_MEMBERS(SUFFIX, T, R)                                                                      \
    void execReduce3##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,                 \
                             T *extraParamsVals, T *y, Nd4jLong *yShapeInfo, T *result,                          \
                             Nd4jLong *resultShapeInfo);                                                         \
    R execReduce3Scalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,              \
                                T *extraParamsVals, T *y, Nd4jLong *yShapeInfo);                                 \
    void execReduce3##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,                 \
                             T *extraParamsVals, T *y, Nd4jLong *yShapeInfo, T *result,                          \
                             Nd4jLong *resultShapeInfoBuffer, int *dimension, int dimensionLength);              \
    void execReduce3All##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xInfo,                   \
                                T *extraParamsVals, T *y, Nd4jLong *yInfo, T *result,                            \
                                Nd4jLong *resultShapeInfoBuffer, int *dimension, int dimensionLength,            \
                                Nd4jLong *xTadShapeInfo, Nd4jLong *xOffsets, Nd4jLong *yTadShapeInfo,            \
                                Nd4jLong *yOffsets);

class ND4J_EXPORT NativeOps {
public:
    ND4J_REDUCE3_MEMBERS(Float, float, float)
    ND4J_REDUCE3_MEMBERS(Half, float16, float)
    ND4J_REDUCE3_MEMBERS(Double, double, double)

    ND4J_SCALAR_MEMBERS(Float, float, float)
    ND4J_SCALAR_MEMBERS(Half, float16, float)
    ND4J_SCALAR_MEMBERS(Double, double, double)
    // the reference's indexed Double variant carries an extra element count (blas/NativeOps.h:419-430)
    void execScalarDouble(Nd4jPointer *extraPointers, int opNum, double *x, Nd4jLong *xShapeInfo, double *result,
                          Nd4jLong *resultShapeInfo, double scalar, double *extraParams, Nd4jLong n, Nd4jLong *xIndexes,
                          Nd4jLong *resultIndexes);

    // n buffers of `length` elements summed (accumulate) or averaged (average) into dz; with `propagate` the average
    // is written back to every input as well.  dx is a device table of device pointers, dz may be null for average.
    // Reference: blas/NativeOps.h:1980-2040, kernels include/loops/special_kernels.h:700-822.  On one GPU all n
    // buffers are local; the reference's use of the same call across peer devices is not part of this build.
#define ND4J_AVERAGE_MEMBERS(SUFFIX, T)                                                              \
    void average##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, T *dz, int n, Nd4jLong length, bool propagate); \
    void accumulate##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, T *dz, int n, Nd4jLong length);
    ND4J_AVERAGE_MEMBERS(Float, float)
    ND4J_AVERAGE_MEMBERS(Half, float16)
    ND4J_AVERAGE_MEMBERS(Double, double)
#undef ND4J_AVERAGE_MEMBERS

    ND4J_SPECIAL_MEMBERS(Float, float)
    ND4J_SPECIAL_MEMBERS(Half, float16)
    ND4J_SPECIAL_MEMBERS(Double, double)
    // z[i] = (dst)(float)x[i] between device buffers; srcType / dstType 3 half, 6 float, 7 double
    // (reference: blas/NativeOps.h:2144, include/loops/type_conversions.h:11-18)
    void convertTypes(Nd4jPointer *extras, int srcType, Nd4jPointer x, Nd4jLong N, int dstType, Nd4jPointer z);

    ND4J_EXEC_MEMBERS(Float, float, float)
    ND4J_EXEC_MEMBERS(Half, float16, float)
    ND4J_EXEC_MEMBERS(Double, double, double)

    // ---- RNG lifecycle, reference: blas/NativeOps.h:2510-2539 ------------------------------------
    // extraPointers[0] = host u64 buffer (bufferSize entries), ptrToBuffer = device u64 buffer
    // (blas/cuda/NativeOps.cu:5384-5407).
    Nd4jPointer initRandom(Nd4jPointer *extraPointers, long seed, long bufferSize, Nd4jPointer ptrToBuffer);
    void refreshBuffer(Nd4jPointer *extraPointers, long seed, Nd4jPointer ptrRandom);
    void reSeedBuffer(Nd4jPointer *extraPointers, long seed, Nd4jPointer ptrRandom);
    void destroyRandom(Nd4jPointer ptrRandom);

    // ---- shape service, reference: blas/NativeOps.h:1880-1884 (host side in both back ends) -------
    void tadOnlyShapeInfo(Nd4jLong *xShapeInfo, int *dimension, int dimensionLength, Nd4jLong *targetBuffer,
                          Nd4jLong *offsetsBuffer);

    // ---- device / stream / memory lifecycle, reference: blas/NativeOps.h:1607-1864 ----------------
    void initializeDevicesAndFunctions();
    Nd4jPointer mallocHost(Nd4jLong memorySize, int flags);
    Nd4jPointer mallocDevice(Nd4jLong memorySize, Nd4jPointer ptrToDeviceId, int flags);
    int freeHost(Nd4jPointer pointer);
    int freeDevice(Nd4jPointer pointer, Nd4jPointer ptrToDeviceId);
    int ompGetMaxThreads();
    int ompGetNumThreads();
    void setOmpNumThreads(int threads);
    void setOmpMinThreads(int threads);
    Nd4jPointer createContext();
    Nd4jPointer createStream();
    Nd4jPointer createEvent();
    int registerEvent(Nd4jPointer event, Nd4jPointer stream);
    int destroyEvent(Nd4jPointer event);
    int setDevice(Nd4jPointer ptrToDeviceId);
    int getDevice();
    int streamSynchronize(Nd4jPointer stream);
    int eventSynchronize(Nd4jPointer event);
    Nd4jLong getDeviceFreeMemory(Nd4jPointer ptrToDeviceId);
    Nd4jLong getDeviceTotalMemory(Nd4jPointer ptrToDeviceId);
    int getDeviceMajor(Nd4jPointer ptrToDeviceId);
    int getDeviceMinor(Nd4jPointer ptrToDeviceId);
    const char *getDeviceName(Nd4jPointer ptrToDeviceId);
    // flags: 0 host-to-host, 1 host-to-device, 2 device-to-host, 3 device-to-device; `reserved` is the stream
    int memcpy(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved);
    int memcpyAsync(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved);
    int memset(Nd4jPointer dst, int value, Nd4jLong size, int flags, Nd4jPointer reserved);
    int memsetAsync(Nd4jPointer dst, int value, Nd4jLong size, int flags, Nd4jPointer reserved);
    int memcpyConstantAsync(Nd4jLong dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved);
    Nd4jPointer getConstantSpace();
    int getAvailableDevices();
    void enableDebugMode(bool reallyEnable);
    void enableVerboseMode(bool reallyEnable);
    void setGridLimit(int gridSize);
    void setElementThreshold(int num);
    void setTADThreshold(int num);

    // ---- Members outside the path ------------------------------------------------------------------
    // Everything else the reference's class declares (blas/NativeOps.h: 1557-1605 specialConcat, 1609 initializeFunctions,
    // 2047-2060 P2P switches, 2172-2330 aggregates, 2564-2760 meta-ops, 2815-2870 numpy helpers, 2902-2935 gradient
    // compression, 2940-2960 sort, 2963-3026 mmap, graphs, custom ops and their helpers), with the same signatures,
    // so that a binding generated from the reference header links against this library.  They do
    // no work here: each prints one line naming itself and returns 0 / null / false (isP2PAvailable,
    // isExperimentalEnabled: false; pointerForAddress, lengthForShapeBufferPointer and the delete*Array helpers do
    // what their names say).  Implemented in libnd4j_amd/csrc/native_stubs.cpp.
#define ND4J_OFFPATH_MEMBERS(SUFFIX, T)                                                                            \
    void specialConcat##SUFFIX(Nd4jPointer *extraPointers, int dimension, int numArrays, Nd4jPointer *data,       \
                               Nd4jPointer *inputShapeInfo, T *result, Nd4jLong *resultShapeInfo,                 \
                               Nd4jPointer *tadPointers, Nd4jPointer *offsetPointers);                            \
    void execAggregate##SUFFIX(Nd4jPointer *extraPointers, int opNum, T **arguments, int numArguments,            \
                               Nd4jLong **shapeArguments, int numShapeArguments, int *indexArguments,             \
                               int numIndexArguments, int **intArrays, int numIntArrays, T *realArguments,        \
                               int numRealArguments);                                                             \
    void execAggregateBatch##SUFFIX(Nd4jPointer *extraPointers, int numAggregates, int opNum, int maxArgs,        \
                                    int maxShapes, int maxIntArrays, int maxIntArraySize, int maxIdx, int maxReals, \
                                    void *ptrToArguments);                                                        \
    void execMetaPredicateStrided##SUFFIX(Nd4jPointer *extras, const int opTypeA, const int opNumA,               \
                                          const int opTypeB, const int opNumB, Nd4jLong N, T *dx, Nd4jLong xStride, \
                                          T *dy, Nd4jLong yStride, T *dz, Nd4jLong zStride, T *extraA, T *extraB, \
                                          S scalarA, S scalarB);                                                  \
    void execMetaPredicateShape##SUFFIX(Nd4jPointer *extras, const int opTypeA, const int opNumA, const int opTypeB, \
                                        const int opNumB, Nd4jLong N, T *dx, Nd4jLong *xShapeInfo, T *dy,         \
                                        Nd4jLong *yShapeInfo, T *dz, Nd4jLong *zShapeInfo, T *extraA, T *extraB,  \
                                        S scalarA, S scalarB);                                                    \
    Nd4jLong encodeBitmap##SUFFIX(Nd4jPointer *extraPointers, T *dx, Nd4jLong N, int *dz, float threshold);       \
    void decodeBitmap##SUFFIX(Nd4jPointer *extraPointers, void *dx, Nd4jLong N, T *dz);                           \
    void encodeThresholdP1##SUFFIX(Nd4jPointer *extraPointers, T *dx, Nd4jLong N, int *dz, float threshold);      \
    void encodeThresholdP3##SUFFIX(Nd4jPointer *extraPointers, T *dx, int *offsets, Nd4jLong N, int *dz);         \
    void decodeThreshold##SUFFIX(Nd4jPointer *extraPointers, void *dx, Nd4jLong N, T *dz);                        \
    void sort##SUFFIX(Nd4jPointer *extraPointers, T *x, Nd4jLong *xShapeInfo, bool descending);                   \
    void sortTad##SUFFIX(Nd4jPointer *extraPointers, T *x, Nd4jLong *xShapeInfo, int *dimension,                  \
                         int dimensionLength, Nd4jLong *tadShapeInfo, Nd4jLong *tadOffsets, bool descending);     \
    void sortCooIndices##SUFFIX(Nd4jPointer *extraPointers, Nd4jLong *indices, T *values, Nd4jLong length, int rank); \
    Nd4jPointer executeFlatGraph##SUFFIX(Nd4jPointer *extraPointers, Nd4jPointer flatBufferPointer);              \
    int execCustomOp##SUFFIX(Nd4jPointer *extraPointers, Nd4jLong hash, Nd4jPointer *inputBuffers,                \
                             Nd4jPointer *inputShapes, int numInputs, Nd4jPointer *outputBuffers,                 \
                             Nd4jPointer *outputShapes, int numOutputs, T *tArgs, int numTArgs, Nd4jLong *iArgs,  \
                             int numIArgs, bool isInplace);                                                       \
    nd4j::ShapeList *calculateOutputShapes##SUFFIX(Nd4jPointer *extraPointers, Nd4jLong hash,                     \
                                                   Nd4jPointer *inputShapes, int numInputShapes, T *tArgs,        \
                                                   int numTArgs, Nd4jLong *iArgs, int numIArgs);                  \
    nd4j::ShapeList *calculateOutputShapes##SUFFIX(Nd4jPointer *extraPointers, Nd4jLong hash,                     \
                                                   Nd4jPointer *inputBuffers, Nd4jPointer *inputShapes,           \
                                                   int numInputShapes, T *tArgs, int numTArgs, Nd4jLong *iArgs,   \
                                                   int numIArgs);                                                 \
    int registerGraph##SUFFIX(Nd4jPointer *extraPointers, Nd4jLong graphId, Nd4jPointer flatBufferPointer);       \
    nd4j::graph::VariablesSet<T> *executeStoredGraph##SUFFIX(Nd4jPointer *extraPointers, Nd4jLong graphId,        \
                                                             Nd4jPointer *inputBuffers, Nd4jPointer *inputShapes, \
                                                             int *inputIndices, int numInputs);                   \
    void deleteVariablesSet##SUFFIX(Nd4jPointer pointer);                                                         \
    Nd4jPointer getGraphState##SUFFIX(Nd4jLong id);                                                               \
    void deleteGraphState##SUFFIX(Nd4jPointer state);                                                             \
    Nd4jStatus execCustomOpWithScope##SUFFIX(Nd4jPointer *extraPointers, Nd4jPointer state, Nd4jLong opHash,      \
                                             Nd4jLong *scopes, int numScopes, Nd4jPointer *inputBuffers,          \
                                             Nd4jPointer *inputShapes, int numInputs, Nd4jPointer *outputBuffers, \
                                             Nd4jPointer *outputShapes, int numOutputs);
#define S float
    ND4J_OFFPATH_MEMBERS(Float, float)
    ND4J_OFFPATH_MEMBERS(Half, float16)
#undef S
#define S double
    ND4J_OFFPATH_MEMBERS(Double, double)
#undef S
#undef ND4J_OFFPATH_MEMBERS
    void execMetaPredicateReduceFloat(Nd4jPointer *extras, const int opTypeA, const int opNumA, const int opTypeB,
                                      const int opNumB, float *dx, Nd4jLong *xShapeInfo, float *dy, Nd4jLong *yShapeInfo,
                                      float *dz, Nd4jLong *zShapeInfo, int *dimension, int dimensionLength,
                                      Nd4jLong *tadShapeInfo, Nd4jLong *tadOffsets, float *extraA, float *extraB,
                                      float scalarA, float scalarB, bool scalarReturned);
    void encodeThresholdP2Int(Nd4jPointer *extraPointers, int *dx, Nd4jLong N, int *dz);
    Nd4jPointer executeProtoGraphFloat(Nd4jPointer *extraPointers, Nd4jPointer protoBufferPointer);
    Nd4jPointer executeProtoGraphFloat(Nd4jPointer *extraPointers, const char *fileName);
    void initializeFunctions(Nd4jPointer *functions);
    void enableP2P(bool enable);
    void checkP2P();
    bool isP2PAvailable();
    bool isExperimentalEnabled();
    Nd4jPointer shapeBufferForNumpy(Nd4jPointer npyArray);
    Nd4jPointer dataPointForNumpy(Nd4jPointer npArray);
    Nd4jPointer numpyFromFile(std::string path);
    void releaseNumpy(Nd4jPointer npyArray);
    int lengthForShapeBufferPointer(Nd4jPointer buffer);
    int elementSizeForNpyArray(Nd4jPointer npyArray);
    Nd4jPointer pointerForAddress(Nd4jLong address);
    Nd4jLong *mmapFile(Nd4jPointer *extraPointers, const char *fileName, Nd4jLong length);
    void munmapFile(Nd4jPointer *extraPointers, Nd4jLong *ptrMap, Nd4jLong length);
    const char *getAllCustomOps();
    const char *getAllOperations();
    void deleteShapeList(Nd4jPointer shapeList);
    int unregisterGraph(Nd4jPointer *extraPointers, Nd4jLong graphId);
    void deleteIntArray(Nd4jPointer pointer);
    void deleteLongArray(Nd4jPointer pointer);
    void deletePointerArray(Nd4jPointer pointer);
};

#undef ND4J_EXEC_MEMBERS
#undef ND4J_SCALAR_MEMBERS
#undef ND4J_REDUCE3_MEMBERS
#undef ND4J_SPECIAL_MEMBERS
