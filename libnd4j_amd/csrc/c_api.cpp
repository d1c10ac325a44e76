// extern "C" entry points: thin forwarders to the NativeOps members (include/nd4j_native_c.h).
#include <hip/hip_runtime.h>

#include <exception>
#include <string>

#include "../../include/NativeOps.h"
#include "../../include/nd4j_native_c.h"
#include "rng.h"
#include "runtime.h"

namespace {
thread_local std::string gLastError;
NativeOps gOps;

template <typename F> void guardVoid(F &&f) {
    gLastError.clear();
    try { f(); }
    catch (const std::exception &e) { gLastError = e.what(); }
    catch (...) { gLastError = "unknown exception"; }
}
template <typename R, typename F> R guardRet(R onError, F &&f) {
    gLastError.clear();
    try { return f(); }
    catch (const std::exception &e) { gLastError = e.what(); }
    catch (...) { gLastError = "unknown exception"; }
    return onError;
}
}  // namespace

extern "C" {

const char *nd4j_lastError(void) { return gLastError.c_str(); }

#define ND4J_C_EXEC(SUFFIX, T, R)                                                                                  \
    R nd4j_execIndexReduceScalar##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p) {                        \
        return guardRet<R>((R)0, [&] { return gOps.execIndexReduceScalar##SUFFIX(e, op, x, xs, p); });              \
    }                                                                                                              \
    void nd4j_execIndexReduce##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *r, Nd4jLong *rs,         \
                                      int *dim, int dl) {                                                           \
        guardVoid([&] { gOps.execIndexReduce##SUFFIX(e, op, x, xs, p, r, rs, dim, dl); });                          \
    }                                                                                                              \
    void nd4j_execBroadcast##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *y, Nd4jLong *ys, T *r,           \
                                    Nd4jLong *rs, int *dim, int dl) {                                               \
        guardVoid([&] { gOps.execBroadcast##SUFFIX(e, op, x, xs, y, ys, r, rs, dim, dl); });                        \
    }                                                                                                              \
    void nd4j_execPairwiseTransform##SUFFIX##Strided(Nd4jPointer *e, int op, T *x, Nd4jLong xs, T *y, Nd4jLong ys,  \
                                                     T *r, Nd4jLong rs, T *p, Nd4jLong n) {                         \
        guardVoid([&] { gOps.execPairwiseTransform##SUFFIX(e, op, x, xs, y, ys, r, rs, p, n); });                   \
    }                                                                                                              \
    void nd4j_execPairwiseTransform##SUFFIX##Indexed(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *y,              \
                                                     Nd4jLong *ys, T *r, Nd4jLong *rs, T *p, Nd4jLong *xi,          \
                                                     Nd4jLong *yi, Nd4jLong *ri) {                                  \
        guardVoid([&] { gOps.execPairwiseTransform##SUFFIX(e, op, x, xs, y, ys, r, rs, p, xi, yi, ri); });          \
    }                                                                                                              \
    void nd4j_execPairwiseTransform##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *y, Nd4jLong *ys, T *r,   \
                                            Nd4jLong *rs, T *p) {                                                   \
        guardVoid([&] { gOps.execPairwiseTransform##SUFFIX(e, op, x, xs, y, ys, r, rs, p); });                      \
    }                                                                                                              \
    void nd4j_execReduce##SUFFIX##Full(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *r, Nd4jLong *rs) {      \
        guardVoid([&] { gOps.execReduce##SUFFIX(e, op, x, xs, p, r, rs); });                                        \
    }                                                                                                              \
    void nd4j_execReduce##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *r, Nd4jLong *rs, int *dim,    \
                                 int dl) {                                                                          \
        guardVoid([&] { gOps.execReduce##SUFFIX(e, op, x, xs, p, r, rs, dim, dl); });                               \
    }                                                                                                              \
    R nd4j_execReduceScalar##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p) {                             \
        return guardRet<R>((R)0, [&] { return gOps.execReduceScalar##SUFFIX(e, op, x, xs, p); });                   \
    }                                                                                                              \
    R nd4j_execSummaryStatsScalar##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, int bc) {               \
        return guardRet<R>((R)0, [&] { return gOps.execSummaryStatsScalar##SUFFIX(e, op, x, xs, p, bc != 0); });    \
    }                                                                                                              \
    void nd4j_execSummaryStats##SUFFIX##Full(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *r, Nd4jLong *rs,  \
                                             int bc) {                                                              \
        guardVoid([&] { gOps.execSummaryStats##SUFFIX(e, op, x, xs, p, r, rs, bc != 0); });                         \
    }                                                                                                              \
    void nd4j_execSummaryStats##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *r, Nd4jLong *rs,        \
                                       int *dim, int dl, int bc) {                                                  \
        guardVoid([&] { gOps.execSummaryStats##SUFFIX(e, op, x, xs, p, r, rs, dim, dl, bc != 0); });                \
    }                                                                                                              \
    void nd4j_execTransform##SUFFIX##Strided(Nd4jPointer *e, int op, T *x, Nd4jLong xs, T *r, Nd4jLong rs, T *p,    \
                                             Nd4jLong n) {                                                          \
        guardVoid([&] { gOps.execTransform##SUFFIX(e, op, x, xs, r, rs, p, n); });                                  \
    }                                                                                                              \
    void nd4j_execTransform##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *r, Nd4jLong *rs, T *p) {         \
        guardVoid([&] { gOps.execTransform##SUFFIX(e, op, x, xs, r, rs, p); });                                     \
    }                                                                                                              \
    void nd4j_execTransform##SUFFIX##Indexed(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *r, Nd4jLong *rs, T *p,  \
                                             Nd4jLong *xi, Nd4jLong *ri) {                                          \
        guardVoid([&] { gOps.execTransform##SUFFIX(e, op, x, xs, r, rs, p, xi, ri); });                             \
    }                                                                                                              \
    void nd4j_execRandom##SUFFIX(Nd4jPointer *e, int op, Nd4jPointer st, T *z, Nd4jLong *zs, T *a) {                \
        guardVoid([&] { gOps.execRandom##SUFFIX(e, op, st, z, zs, a); });                                           \
    }                                                                                                              \
    void nd4j_execRandom##SUFFIX##XYZ(Nd4jPointer *e, int op, Nd4jPointer st, T *x, Nd4jLong *xs, T *y,             \
                                      Nd4jLong *ys, T *z, Nd4jLong *zs, T *a) {                                     \
        guardVoid([&] { gOps.execRandom##SUFFIX(e, op, st, x, xs, y, ys, z, zs, a); });                             \
    }                                                                                                              \
    void nd4j_execRandom##SUFFIX##XZ(Nd4jPointer *e, int op, Nd4jPointer st, T *x, Nd4jLong *xs, T *z,              \
                                     Nd4jLong *zs, T *a) {                                                          \
        guardVoid([&] { gOps.execRandom##SUFFIX(e, op, st, x, xs, z, zs, a); });                                    \
    }

ND4J_C_EXEC(Float, float, float)
ND4J_C_EXEC(Half, float16, float)
ND4J_C_EXEC(Double, double, double)
#undef ND4J_C_EXEC

#define ND4J_C_SCALAR(SUFFIX, T, S)                                                                                \
    void nd4j_execScalar##SUFFIX##Strided(Nd4jPointer *e, int op, T *x, Nd4jLong xs, T *r, Nd4jLong rs, S sc, T *p, \
                                          Nd4jLong n) {                                                             \
        guardVoid([&] { gOps.execScalar##SUFFIX(e, op, x, xs, r, rs, sc, p, n); });                                 \
    }                                                                                                              \
    void nd4j_execScalar##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *r, Nd4jLong *rs, S sc, T *p) {      \
        guardVoid([&] { gOps.execScalar##SUFFIX(e, op, x, xs, r, rs, sc, p); });                                    \
    }                                                                                                              \
    void nd4j_execScalar##SUFFIX##Indexed(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *r, Nd4jLong *rs, S sc,     \
                                          T *p, Nd4jLong *xi, Nd4jLong *ri) {                                       \
        guardVoid([&] { gOps.execScalar##SUFFIX(e, op, x, xs, r, rs, sc, p, xi, ri); });                            \
    }                                                                                                              \
    void nd4j_execScalar##SUFFIX##AlongDimension(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *z, Nd4jLong *zs,    \
                                                 T *scalars, T *p, int *dim, int dl) {                              \
        guardVoid([&] { gOps.execScalar##SUFFIX(e, op, x, xs, z, zs, scalars, p, dim, dl); });                      \
    }
ND4J_C_SCALAR(Float, float, float)
ND4J_C_SCALAR(Half, float16, float)
ND4J_C_SCALAR(Double, double, double)
#undef ND4J_C_SCALAR

#define ND4J_C_REDUCE3(SUFFIX, T, R)                                                                               \
    void nd4j_execReduce3##SUFFIX##Full(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *y, Nd4jLong *ys, T *r, \
                                        Nd4jLong *rs) {                                                             \
        guardVoid([&] { gOps.execReduce3##SUFFIX(e, op, x, xs, p, y, ys, r, rs); });                                \
    }                                                                                                              \
    R nd4j_execReduce3Scalar##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *y, Nd4jLong *ys) {        \
        return guardRet<R>((R)0, [&] { return gOps.execReduce3Scalar##SUFFIX(e, op, x, xs, p, y, ys); });           \
    }                                                                                                              \
    void nd4j_execReduce3##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *y, Nd4jLong *ys, T *r,       \
                                  Nd4jLong *rs, int *dim, int dl) {                                                 \
        guardVoid([&] { gOps.execReduce3##SUFFIX(e, op, x, xs, p, y, ys, r, rs, dim, dl); });                       \
    }                                                                                                              \
    void nd4j_execReduce3All##SUFFIX(Nd4jPointer *e, int op, T *x, Nd4jLong *xs, T *p, T *y, Nd4jLong *ys, T *r,    \
                                     Nd4jLong *rs, int *dim, int dl, Nd4jLong *xt, Nd4jLong *xo, Nd4jLong *yt,      \
                                     Nd4jLong *yo) {                                                                \
        guardVoid([&] { gOps.execReduce3All##SUFFIX(e, op, x, xs, p, y, ys, r, rs, dim, dl, xt, xo, yt, yo); });    \
    }
ND4J_C_REDUCE3(Float, float, float)
ND4J_C_REDUCE3(Half, float16, float)
ND4J_C_REDUCE3(Double, double, double)
#undef ND4J_C_REDUCE3

#define ND4J_C_SPECIAL(SUFFIX, T)                                                                                  \
    void nd4j_flatten##SUFFIX(Nd4jPointer *e, int offset, char order, T *r, Nd4jLong *rs, T *in, Nd4jLong *is) {   \
        guardVoid([&] { gOps.flatten##SUFFIX(e, offset, order, r, rs, in, is); });                                 \
    }                                                                                                              \
    void nd4j_concat##SUFFIX(Nd4jPointer *e, int dim, int n, Nd4jPointer *data, Nd4jPointer *infos, T *r,          \
                             Nd4jLong *rs, Nd4jPointer *tads, Nd4jPointer *offs) {                                 \
        guardVoid([&] { gOps.concat##SUFFIX(e, dim, n, data, infos, r, rs, tads, offs); });                        \
    }                                                                                                              \
    void nd4j_pullRows##SUFFIX(Nd4jPointer *e, T *x, Nd4jLong *xs, T *z, Nd4jLong *zs, Nd4jLong n, Nd4jLong *idx,  \
                               Nd4jLong *ti, Nd4jLong *to, Nd4jLong *zti, Nd4jLong *zto) {                         \
        guardVoid([&] { gOps.pullRows##SUFFIX(e, x, xs, z, zs, n, idx, ti, to, zti, zto); });                      \
    }                                                                                                              \
    void nd4j_tear##SUFFIX(Nd4jPointer *e, T *x, Nd4jLong *xs, Nd4jPointer *targets, Nd4jLong *zs, Nd4jLong *ti,   \
                           Nd4jLong *to) {                                                                         \
        guardVoid([&] { gOps.tear##SUFFIX(e, x, xs, targets, zs, ti, to); });                                      \
    }                                                                                                              \
    void nd4j_shuffle##SUFFIX(Nd4jPointer *e, Nd4jPointer *dx, Nd4jPointer *xs, Nd4jPointer *dz, Nd4jPointer *zs,  \
                              int N, int *map, Nd4jPointer *ti, Nd4jPointer *to) {                                 \
        guardVoid([&] { gOps.shuffle##SUFFIX(e, dx, xs, dz, zs, N, map, ti, to); });                               \
    }                                                                                                              \
    void nd4j_average##SUFFIX(Nd4jPointer *e, Nd4jPointer *dx, T *dz, int n, Nd4jLong length, int propagate) {     \
        guardVoid([&] { gOps.average##SUFFIX(e, dx, dz, n, length, propagate != 0); });                            \
    }                                                                                                              \
    void nd4j_accumulate##SUFFIX(Nd4jPointer *e, Nd4jPointer *dx, T *dz, int n, Nd4jLong length) {                 \
        guardVoid([&] { gOps.accumulate##SUFFIX(e, dx, dz, n, length); });                                         \
    }
ND4J_C_SPECIAL(Float, float)
ND4J_C_SPECIAL(Half, float16)
ND4J_C_SPECIAL(Double, double)
#undef ND4J_C_SPECIAL
void nd4j_convertTypes(Nd4jPointer *e, int st, Nd4jPointer x, Nd4jLong n, int dt, Nd4jPointer z) {
    guardVoid([&] { gOps.convertTypes(e, st, x, n, dt, z); });
}

Nd4jPointer nd4j_initRandom(Nd4jPointer *e, long seed, long size, Nd4jPointer buf) {
    return guardRet<Nd4jPointer>(nullptr, [&] { return gOps.initRandom(e, seed, size, buf); });
}
void nd4j_refreshBuffer(Nd4jPointer *e, long seed, Nd4jPointer r) { guardVoid([&] { gOps.refreshBuffer(e, seed, r); }); }
void nd4j_reSeedBuffer(Nd4jPointer *e, long seed, Nd4jPointer r) { guardVoid([&] { gOps.reSeedBuffer(e, seed, r); }); }
void nd4j_destroyRandom(Nd4jPointer r) { guardVoid([&] { gOps.destroyRandom(r); }); }

void nd4j_tadOnlyShapeInfo(Nd4jLong *xs, int *dim, int dl, Nd4jLong *target, Nd4jLong *offsets) {
    guardVoid([&] { gOps.tadOnlyShapeInfo(xs, dim, dl, target, offsets); });
}

void nd4j_initializeDevicesAndFunctions(void) { guardVoid([&] { gOps.initializeDevicesAndFunctions(); }); }
Nd4jPointer nd4j_mallocHost(Nd4jLong n, int f) { return guardRet<Nd4jPointer>(nullptr, [&] { return gOps.mallocHost(n, f); }); }
Nd4jPointer nd4j_mallocDevice(Nd4jLong n, Nd4jPointer d, int f) {
    return guardRet<Nd4jPointer>(nullptr, [&] { return gOps.mallocDevice(n, d, f); });
}
int nd4j_freeHost(Nd4jPointer p) { return guardRet<int>(0, [&] { return gOps.freeHost(p); }); }
int nd4j_freeDevice(Nd4jPointer p, Nd4jPointer d) { return guardRet<int>(0, [&] { return gOps.freeDevice(p, d); }); }
int nd4j_ompGetMaxThreads(void) { return gOps.ompGetMaxThreads(); }
int nd4j_ompGetNumThreads(void) { return gOps.ompGetNumThreads(); }
void nd4j_setOmpNumThreads(int t) { gOps.setOmpNumThreads(t); }
void nd4j_setOmpMinThreads(int t) { gOps.setOmpMinThreads(t); }
Nd4jPointer nd4j_createContext(void) { return gOps.createContext(); }
Nd4jPointer nd4j_createStream(void) { return guardRet<Nd4jPointer>(nullptr, [&] { return gOps.createStream(); }); }
Nd4jPointer nd4j_createEvent(void) { return guardRet<Nd4jPointer>(nullptr, [&] { return gOps.createEvent(); }); }
int nd4j_registerEvent(Nd4jPointer e, Nd4jPointer s) { return guardRet<int>(0, [&] { return gOps.registerEvent(e, s); }); }
int nd4j_destroyEvent(Nd4jPointer e) { return guardRet<int>(0, [&] { return gOps.destroyEvent(e); }); }
int nd4j_setDevice(Nd4jPointer d) { return guardRet<int>(0, [&] { return gOps.setDevice(d); }); }
int nd4j_getDevice(void) { return gOps.getDevice(); }
int nd4j_streamSynchronize(Nd4jPointer s) { return guardRet<int>(0, [&] { return gOps.streamSynchronize(s); }); }
int nd4j_eventSynchronize(Nd4jPointer e) { return guardRet<int>(0, [&] { return gOps.eventSynchronize(e); }); }
Nd4jLong nd4j_getDeviceFreeMemory(Nd4jPointer d) { return gOps.getDeviceFreeMemory(d); }
Nd4jLong nd4j_getDeviceTotalMemory(Nd4jPointer d) { return gOps.getDeviceTotalMemory(d); }
int nd4j_getDeviceMajor(Nd4jPointer d) { return gOps.getDeviceMajor(d); }
int nd4j_getDeviceMinor(Nd4jPointer d) { return gOps.getDeviceMinor(d); }
const char *nd4j_getDeviceName(Nd4jPointer d) { return gOps.getDeviceName(d); }
int nd4j_memcpy(Nd4jPointer a, Nd4jPointer b, Nd4jLong n, int f, Nd4jPointer r) { return gOps.memcpy(a, b, n, f, r); }
int nd4j_memcpyAsync(Nd4jPointer a, Nd4jPointer b, Nd4jLong n, int f, Nd4jPointer r) { return gOps.memcpyAsync(a, b, n, f, r); }
int nd4j_memset(Nd4jPointer a, int v, Nd4jLong n, int f, Nd4jPointer r) { return gOps.memset(a, v, n, f, r); }
int nd4j_memsetAsync(Nd4jPointer a, int v, Nd4jLong n, int f, Nd4jPointer r) { return gOps.memsetAsync(a, v, n, f, r); }
int nd4j_memcpyConstantAsync(Nd4jLong d, Nd4jPointer s, Nd4jLong n, int f, Nd4jPointer r) {
    return gOps.memcpyConstantAsync(d, s, n, f, r);
}
Nd4jPointer nd4j_getConstantSpace(void) { return gOps.getConstantSpace(); }
int nd4j_getAvailableDevices(void) { return gOps.getAvailableDevices(); }
void nd4j_enableDebugMode(int b) { gOps.enableDebugMode(b != 0); }
void nd4j_enableVerboseMode(int b) { gOps.enableVerboseMode(b != 0); }
void nd4j_setGridLimit(int g) { gOps.setGridLimit(g); }
void nd4j_setElementThreshold(int n) { gOps.setElementThreshold(n); }
void nd4j_setTADThreshold(int n) { gOps.setTADThreshold(n); }

// ---- measurement and parity aids ----------------------------------------------------------------------
void nd4j_amd_rngDump(Nd4jPointer *extraPointers, Nd4jPointer ptrRandom, Nd4jLong start, Nd4jLong n,
                      unsigned long long *out) {
    guardVoid([&] {
        auto *rb = reinterpret_cast<nd4j_amd::RandomBuffer *>(ptrRandom);
        hipStream_t s = nd4j_amd::streamOf(extraPointers);
        nd4j_amd::launchRngDump(s, rb->deviceState(), start, n, out);
        nd4j_amd::checkLaunch("rngDump", s);
    });
}
void nd4j_amd_rngState(Nd4jPointer ptrRandom, Nd4jLong *state) {
    auto *rb = reinterpret_cast<nd4j_amd::RandomBuffer *>(ptrRandom);
    state[0] = rb->size;
    state[1] = rb->currentPosition;
    state[2] = rb->seed;
    state[3] = rb->generation;
    state[4] = rb->amplifier;
}
Nd4jPointer nd4j_amd_timerCreate(void) {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    return reinterpret_cast<Nd4jPointer>(e);
}
int nd4j_amd_timerRecord(Nd4jPointer timer, Nd4jPointer stream) {
    return hipEventRecord(reinterpret_cast<hipEvent_t>(timer), reinterpret_cast<hipStream_t>(stream)) == hipSuccess ? 1 : 0;
}
float nd4j_amd_timerElapsedMs(Nd4jPointer start, Nd4jPointer stop) {
    float ms = -1.0f;
    if (hipEventSynchronize(reinterpret_cast<hipEvent_t>(stop)) != hipSuccess) { (void)hipGetLastError(); return -1.0f; }
    if (hipEventElapsedTime(&ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)) != hipSuccess) {
        (void)hipGetLastError();
        return -1.0f;
    }
    return ms;
}
int nd4j_amd_timerDestroy(Nd4jPointer timer) { return hipEventDestroy(reinterpret_cast<hipEvent_t>(timer)) == hipSuccess ? 1 : 0; }
void nd4j_amd_execReduceFloatNoAlloc(Nd4jPointer *extraPointers, int opNum, float *x, Nd4jLong *xShapeInfo, float *extraParams,
                                     float *result) {
    guardVoid([&] { nd4j_amd::reduceFloatNoAlloc(extraPointers, opNum, x, xShapeInfo, extraParams, result); });
}
void nd4j_amd_forderTileCopy(Nd4jPointer *extraPointers, float *dst, const float *src, Nd4jLong rows, Nd4jLong cols) {
    guardVoid([&] {
        nd4j_amd::launchForderTileCopy(nd4j_amd::streamOf(extraPointers), src, dst, rows, cols);
        nd4j_amd::checkLaunch("forderTileCopy", nd4j_amd::streamOf(extraPointers));
    });
}
void nd4j_amd_releaseStream(Nd4jPointer stream) {
    guardVoid([&] { nd4j_amd::releaseStreamResources(reinterpret_cast<hipStream_t>(stream)); });
}
void nd4j_amd_setSlotTicket(Nd4jPointer *extraPointers, unsigned int value) {
    guardVoid([&] { nd4j_amd::setSlotTicketForTesting(nd4j_amd::streamOf(extraPointers), value); });
}
Nd4jLong nd4j_amd_hostFetchCount(void) { return (Nd4jLong)nd4j_amd::hostFetchCount(); }
void nd4j_amd_setCooperativeWaitLimit(int tries) { nd4j_amd::setCooperativeWaitLimit(tries); }
void nd4j_amd_copyKernel(Nd4jPointer *extraPointers, void *dst, const void *src, Nd4jLong bytes) {
    guardVoid([&] {
        hipStream_t s = nd4j_amd::streamOf(extraPointers);
        nd4j_amd::launchCopy(s, dst, src, bytes);
        nd4j_amd::checkLaunch("copyKernel", s);
    });
}

}  // extern "C"
