/* C ABI of libnd4j_amd.so: one extern "C" entry point per NativeOps member on the legacy op-execution
 * path, for bindings that cannot call C++ members (ctypes, cgo, N-API ...).  Each function forwards to
 * the member of the same name in include/NativeOps.h; where the C++ class overloads a name, the C name
 * carries a suffix (Strided / Indexed / Full / XZ / XYZ).  Arguments are plain pointers and integers;
 * their meaning, the extraPointers convention and the synchronisation behaviour are those documented in
 * include/NativeOps.h.
 *
 * Reference declarations replaced (blas/NativeOps.h, Float / Half / Double):
 *   execIndexReduceScalar*  544-573, 80-94        execIndexReduce*      576-602, 96-113
 *   execBroadcast*          615-649, 115-139      execPairwiseTransform* 665-798, 141-210
 *   execReduce*             809-876, 212-244      execReduceScalar*     886-906, 246-250
 *   execSummaryStatsScalar* 1223-1242, 438-451    execSummaryStats*     1253-1325, 453-490
 *   execTransform*          1337-1443, 492-542    execRandom*           2327-2498
 *   initRandom/refreshBuffer/reSeedBuffer/destroyRandom 2510-2539        tadOnlyShapeInfo 1880-1884
 *   device, stream, event and memory members 1607-1864
 *
 * Error convention: the reference throws std::runtime_error on device failures; a C ABI cannot, so a
 * failed call records a message retrievable with nd4j_lastError() (empty string when the last call on
 * this thread succeeded) and returns 0 / NULL / leaves the output untouched.
 */
#ifndef ND4J_NATIVE_C_H
#define ND4J_NATIVE_C_H

#include "nd4j_types.h"

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

const char *nd4j_lastError(void);

#define ND4J_C_EXEC(SUFFIX, T, R)                                                                                 \
    R nd4j_execIndexReduceScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,       \
                                         T *extraParams);                                                         \
    void nd4j_execIndexReduce##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,          \
                                      T *extraParams, T *result, Nd4jLong *resultShapeInfoBuffer, int *dimension, \
                                      int dimensionLength);                                                       \
    void nd4j_execBroadcast##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *y,      \
                                    Nd4jLong *yShapeInfo, T *result, Nd4jLong *resultShapeInfo, int *dimension,   \
                                    int dimensionLength);                                                         \
    void nd4j_execPairwiseTransform##SUFFIX##Strided(Nd4jPointer *extraPointers, int opNum, T *dx,                \
                                                     Nd4jLong xStride, T *y, Nd4jLong yStride, T *result,         \
                                                     Nd4jLong resultStride, T *extraParams, Nd4jLong n);          \
    void nd4j_execPairwiseTransform##SUFFIX##Indexed(Nd4jPointer *extraPointers, int opNum, T *dx,                \
                                                     Nd4jLong *xShapeInfo, T *y, Nd4jLong *yShapeInfo, T *result, \
                                                     Nd4jLong *resultShapeInfo, T *extraParams,                   \
                                                     Nd4jLong *xIndexes, Nd4jLong *yIndexes,                      \
                                                     Nd4jLong *resultIndexes);                                    \
    void nd4j_execPairwiseTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong *xShapeInfo,   \
                                            T *y, Nd4jLong *yShapeInfo, T *result, Nd4jLong *resultShapeInfo,     \
                                            T *extraParams);                                                      \
    void nd4j_execReduce##SUFFIX##Full(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,         \
                                       T *extraParams, T *result, Nd4jLong *resultShapeInfo);                     \
    void nd4j_execReduce##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,               \
                                 T *extraParams, T *result, Nd4jLong *resultShapeInfo, int *dimension,            \
                                 int dimensionLength);                                                            \
    R nd4j_execReduceScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,            \
                                    T *extraParams);                                                              \
    R nd4j_execSummaryStatsScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,      \
                                          T *extraParams, int biasCorrected);                                     \
    void nd4j_execSummaryStats##SUFFIX##Full(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,   \
                                             T *extraParams, T *result, Nd4jLong *resultShapeInfo,                \
                                             int biasCorrected);                                                  \
    void nd4j_execSummaryStats##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,         \
                                       T *extraParams, T *result, Nd4jLong *resultShapeInfoBuffer,                \
                                       int *dimension, int dimensionLength, int biasCorrected);                   \
    void nd4j_execTransform##SUFFIX##Strided(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong xStride,      \
                                             T *result, Nd4jLong resultStride, T *extraParams, Nd4jLong n);       \
    void nd4j_execTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong *xShapeInfo,           \
                                    T *result, Nd4jLong *resultShapeInfo, T *extraParams);                        \
    void nd4j_execTransform##SUFFIX##Indexed(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong *xShapeInfo,  \
                                             T *result, Nd4jLong *resultShapeInfo, T *extraParams,                \
                                             Nd4jLong *xIndexes, Nd4jLong *resultIndexes);                        \
    void nd4j_execRandom##SUFFIX(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *z,                  \
                                 Nd4jLong *zShapeBuffer, T *extraArguments);                                      \
    void nd4j_execRandom##SUFFIX##XYZ(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *x,             \
                                      Nd4jLong *xShapeBuffer, T *y, Nd4jLong *yShapeBuffer, T *z,                 \
                                      Nd4jLong *zShapeBuffer, T *extraArguments);                                 \
    void nd4j_execRandom##SUFFIX##XZ(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *x,              \
                                     Nd4jLong *xShapeBuffer, T *z, Nd4jLong *zShapeBuffer, T *extraArguments);

ND4J_C_EXEC(Float, float, float)
ND4J_C_EXEC(Half, float16, float)
ND4J_C_EXEC(Double, double, double)
#undef ND4J_C_EXEC

/* Scalar family (blas/NativeOps.h:1046-1226, 377-440): z = op(x, scalar, extraParams).  Strided, shaped,
 * indexed (a no-op, as in the reference's CUDA back end) and one-scalar-per-TAD variants; S is float for
 * Float and Half, double for Double. */
#define ND4J_C_SCALAR(SUFFIX, T, S)                                                                              \
    void nd4j_execScalar##SUFFIX##Strided(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong xStride,         \
                                          T *result, Nd4jLong resultStride, S scalar, T *extraParams,             \
                                          Nd4jLong n);                                                            \
    void nd4j_execScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *result,   \
                                 Nd4jLong *resultShapeInfo, S scalar, T *extraParams);                            \
    void nd4j_execScalar##SUFFIX##Indexed(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,     \
                                          T *result, Nd4jLong *resultShapeInfo, S scalar, T *extraParams,         \
                                          Nd4jLong *xIndexes, Nd4jLong *resultIndexes);                           \
    void nd4j_execScalar##SUFFIX##AlongDimension(Nd4jPointer *extraPointers, int opNum, T *x,                    \
                                                 Nd4jLong *xShapeInfo, T *z, Nd4jLong *zShapeInfo, T *scalars,    \
                                                 T *extraParams, int *dimension, int dimensionLength);
ND4J_C_SCALAR(Float, float, float)
ND4J_C_SCALAR(Half, float16, float)
ND4J_C_SCALAR(Double, double, double)
#undef ND4J_C_SCALAR

/* Reduce3 family (blas/NativeOps.h:919-1044, 252-362): whole arrays into result[0] (Full), returned by value
 * (Scalar), along `dimension`, and all pairs of TADs (All). */
#define ND4J_C_REDUCE3(SUFFIX, T, R)                                                                             \
    void nd4j_execReduce3##SUFFIX##Full(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,       \
                                        T *extraParamsVals, T *y, Nd4jLong *yShapeInfo, T *result,                \
                                        Nd4jLong *resultShapeInfo);                                               \
    R nd4j_execReduce3Scalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,          \
                                     T *extraParamsVals, T *y, Nd4jLong *yShapeInfo);                             \
    void nd4j_execReduce3##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,             \
                                  T *extraParamsVals, T *y, Nd4jLong *yShapeInfo, T *result,                      \
                                  Nd4jLong *resultShapeInfoBuffer, int *dimension, int dimensionLength);          \
    void nd4j_execReduce3All##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xInfo,               \
                                     T *extraParamsVals, T *y, Nd4jLong *yInfo, T *result,                        \
                                     Nd4jLong *resultShapeInfoBuffer, int *dimension, int dimensionLength,        \
                                     Nd4jLong *xTadShapeInfo, Nd4jLong *xOffsets, Nd4jLong *yTadShapeInfo,        \
                                     Nd4jLong *yOffsets);
ND4J_C_REDUCE3(Float, float, float)
ND4J_C_REDUCE3(Half, float16, float)
ND4J_C_REDUCE3(Double, double, double)
#undef ND4J_C_REDUCE3

/* Data-movement specials (blas/NativeOps.h:1457-1499 flatten, 1510-1555 concat, 1904-1967 pullRows, 2076-2130
 * shuffle, 2876-2899 tear, 2144 convertTypes, 1980-2040 average / accumulate of n local buffers); pointer conventions as documented in include/NativeOps.h. */
#define ND4J_C_SPECIAL(SUFFIX, T)                                                                                \
    void nd4j_flatten##SUFFIX(Nd4jPointer *extraPointers, int offset, char order, T *result,                     \
                              Nd4jLong *resultShapeInfo, T *input, Nd4jLong *inputShapeInfo);                    \
    void nd4j_concat##SUFFIX(Nd4jPointer *extraPointers, int dimension, int numArrays, Nd4jPointer *data,        \
                             Nd4jPointer *inputShapeInfo, T *result, Nd4jLong *resultShapeInfo,                  \
                             Nd4jPointer *tadPointers, Nd4jPointer *offsetPointers);                             \
    void nd4j_pullRows##SUFFIX(Nd4jPointer *extraPointers, T *x, Nd4jLong *xShapeInfo, T *z,                     \
                               Nd4jLong *zShapeInfo, Nd4jLong n, Nd4jLong *indexes, Nd4jLong *tadShapeInfo,      \
                               Nd4jLong *tadOffsets, Nd4jLong *zTadShapeInfo, Nd4jLong *zTadOffsets);            \
    void nd4j_tear##SUFFIX(Nd4jPointer *extraPointers, T *x, Nd4jLong *xShapeInfo, Nd4jPointer *targets,         \
                           Nd4jLong *zShapeInfo, Nd4jLong *tadShapeInfo, Nd4jLong *tadOffsets);                  \
    void nd4j_shuffle##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, Nd4jPointer *xShapeInfo, Nd4jPointer *dz,    \
                              Nd4jPointer *zShapeInfo, int N, int *shuffleMap, Nd4jPointer *tadShapeInfo,        \
                              Nd4jPointer *tadOffsets);                                                          \
    void nd4j_average##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, T *dz, int n, Nd4jLong length, int propagate); \
    void nd4j_accumulate##SUFFIX(Nd4jPointer *extras, Nd4jPointer *dx, T *dz, int n, Nd4jLong length);
ND4J_C_SPECIAL(Float, float)
ND4J_C_SPECIAL(Half, float16)
ND4J_C_SPECIAL(Double, double)
#undef ND4J_C_SPECIAL
void nd4j_convertTypes(Nd4jPointer *extras, int srcType, Nd4jPointer x, Nd4jLong N, int dstType, Nd4jPointer z);

Nd4jPointer nd4j_initRandom(Nd4jPointer *extraPointers, long seed, long bufferSize, Nd4jPointer ptrToBuffer);
void nd4j_refreshBuffer(Nd4jPointer *extraPointers, long seed, Nd4jPointer ptrRandom);
void nd4j_reSeedBuffer(Nd4jPointer *extraPointers, long seed, Nd4jPointer ptrRandom);
void nd4j_destroyRandom(Nd4jPointer ptrRandom);

void nd4j_tadOnlyShapeInfo(Nd4jLong *xShapeInfo, int *dimension, int dimensionLength, Nd4jLong *targetBuffer,
                           Nd4jLong *offsetsBuffer);

void nd4j_initializeDevicesAndFunctions(void);
Nd4jPointer nd4j_mallocHost(Nd4jLong memorySize, int flags);
Nd4jPointer nd4j_mallocDevice(Nd4jLong memorySize, Nd4jPointer ptrToDeviceId, int flags);
int nd4j_freeHost(Nd4jPointer pointer);
int nd4j_freeDevice(Nd4jPointer pointer, Nd4jPointer ptrToDeviceId);
int nd4j_ompGetMaxThreads(void);
int nd4j_ompGetNumThreads(void);
void nd4j_setOmpNumThreads(int threads);
void nd4j_setOmpMinThreads(int threads);
Nd4jPointer nd4j_createContext(void);
Nd4jPointer nd4j_createStream(void);
Nd4jPointer nd4j_createEvent(void);
int nd4j_registerEvent(Nd4jPointer event, Nd4jPointer stream);
int nd4j_destroyEvent(Nd4jPointer event);
int nd4j_setDevice(Nd4jPointer ptrToDeviceId);
int nd4j_getDevice(void);
int nd4j_streamSynchronize(Nd4jPointer stream);
int nd4j_eventSynchronize(Nd4jPointer event);
Nd4jLong nd4j_getDeviceFreeMemory(Nd4jPointer ptrToDeviceId);
Nd4jLong nd4j_getDeviceTotalMemory(Nd4jPointer ptrToDeviceId);
int nd4j_getDeviceMajor(Nd4jPointer ptrToDeviceId);
int nd4j_getDeviceMinor(Nd4jPointer ptrToDeviceId);
const char *nd4j_getDeviceName(Nd4jPointer ptrToDeviceId);
int nd4j_memcpy(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved);
int nd4j_memcpyAsync(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved);
int nd4j_memset(Nd4jPointer dst, int value, Nd4jLong size, int flags, Nd4jPointer reserved);
int nd4j_memsetAsync(Nd4jPointer dst, int value, Nd4jLong size, int flags, Nd4jPointer reserved);
int nd4j_memcpyConstantAsync(Nd4jLong dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved);
Nd4jPointer nd4j_getConstantSpace(void);
int nd4j_getAvailableDevices(void);
void nd4j_enableDebugMode(int reallyEnable);
void nd4j_enableVerboseMode(int reallyEnable);
void nd4j_setGridLimit(int gridSize);
void nd4j_setElementThreshold(int num);
void nd4j_setTADThreshold(int num);

/* ---- measurement and parity aids: no counterpart in the reference ---------------------------------- */
/* out[i] = RandomBuffer::getElement(start + i) for the generator `ptrRandom`, computed on the device with
 * the state as it stands (reference for the values: include/helpers/helper_generator.h:185-220). `out` is
 * a device pointer. */
void nd4j_amd_rngDump(Nd4jPointer *extraPointers, Nd4jPointer ptrRandom, Nd4jLong start, Nd4jLong n,
                      unsigned long long *out);
/* state[0..4] = size, offset, seed, generation, amplifier of the generator */
void nd4j_amd_rngState(Nd4jPointer ptrRandom, Nd4jLong *state);
/* HIP events with timing enabled, to time work on the stream the ops are launched on; Record and Destroy
 * return 1 on success and 0 on failure, ElapsedMs waits for `stop` and returns -1 on failure */
Nd4jPointer nd4j_amd_timerCreate(void);
int nd4j_amd_timerRecord(Nd4jPointer timer, Nd4jPointer stream);
float nd4j_amd_timerElapsedMs(Nd4jPointer start, Nd4jPointer stop);
int nd4j_amd_timerDestroy(Nd4jPointer timer);
/* number of times, since the library was loaded, that a call had to read a shapeInfo or a dimension array back from
 * the device because the host copy / TAD tables of the CUDA convention were not passed: each one synchronises the
 * stream, so a caller that wants asynchronous array-result calls keeps this from growing */
Nd4jLong nd4j_amd_hostFetchCount(void);
/* No counterpart in the reference.  SoftMax / SoftMaxDerivative / LogSoftMax over long contiguous rows, and over f-order
 * matrices of more than 1024 columns, run as one pass in which the blocks that hold the slices of a row (of a group of
 * rows) wait for each other; every such wait is bounded, and a row whose blocks could not all see each other in time is
 * left untouched by them and computed by a repair kernel behind the launch.  `tries` is the number of polls a block spends on a slice that is not there yet (default 5000, each a
 * microsecond or two); 0 makes everything that is not there at the first look count as missing, which is how the tests
 * drive rows through the repair kernel. */
void nd4j_amd_setCooperativeWaitLimit(int tries);
/* plain device-to-device copy kernel of `bytes` bytes (16-byte vectors): the yardstick against which
 * hardware traffic counters are scaled */
void nd4j_amd_copyKernel(Nd4jPointer *extraPointers, void *dst, const void *src, Nd4jLong bytes);

/* yardstick for the fused softmax over f-order matrices: copies the f-order float matrix src [rows, cols] (rows adjacent in
 * memory, a multiple of 4 of them, 16-byte aligned) to dst in exactly the tiles and block order of that kernel - 64 rows
 * x 512 columns to a 512-thread block, 256 contiguous bytes of each column at a time - with no arithmetic and no exchange
 * between blocks */
void nd4j_amd_forderTileCopy(Nd4jPointer *extraPointers, float *dst, const float *src, Nd4jLong rows, Nd4jLong cols);
/* No counterpart in the reference (its scratch belongs to the caller).  The library keeps a workspace, reduction slots
 * and a pinned scalar block per (device, stream), allocated at the stream's first call that needs them.  A host that
 * destroys a stream calls this first, with the stream's device current: it waits for the stream to drain and frees them
 * (13 MiB of device memory and 256 bytes of pinned host memory a stream); a later call on the same handle allocates
 * afresh.  Without it they stay until the process ends. */
void nd4j_amd_releaseStream(Nd4jPointer stream);
/* test aid: sets the counter from which the launches on extraPointers[1]'s stream draw the tickets that tag their
 * exchange slots, so that a test can walk it across the points where the library clears the slots */
void nd4j_amd_setSlotTicket(Nd4jPointer *extraPointers, unsigned int value);

/* ---- for callers that cannot allocate: no counterpart in the reference ------------------------------- */
/* execReduceFloat over the whole array (no dimensions): result[0], a device pointer, receives what
 * nd4j_execReduceFloatFull leaves there, bit for bit.  For callers that may not call hipMalloc while they run
 * (code under HIP graph capture, tight serving loops, harnesses that forbid allocation): this entry point
 * allocates and frees nothing, reads nothing back and does not synchronise.  Its partial accumulators live in
 * a 64 KiB device array inside the library, one copy per GPU, kept until the process ends and shared by every
 * call on that GPU: calls that overlap on one GPU (two streams, two threads) race on it, so issue them one
 * after the other.  The host copy of xShapeInfo must be in extraPointers[0] (or xShapeInfo itself a host
 * pointer); extraPointers[1] is the stream.  Arrays of more than 2^36 elements, empty arrays, a missing host
 * shapeInfo and unknown opNums are rejected: nd4j_lastError() says why and result is left untouched. */
void nd4j_amd_execReduceFloatNoAlloc(Nd4jPointer *extraPointers, int opNum, float *x, Nd4jLong *xShapeInfo,
                                     float *extraParams, float *result);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif
