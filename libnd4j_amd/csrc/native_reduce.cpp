// NativeOps boundary, part 2: reduce, index-reduce and summary-stats members.
// Branch selection follows the reference's CPU loops (the parity oracle):
//   reduce         include/loops/cpu/reduce.cpp:91-193, scalar 14-64 / 206-323; LogSumExp pre-pass
//                  blas/cpu/NativeOpExcutioner.cpp:122-147
//   index-reduce   include/loops/cpu/indexreduce.cpp:36-129, 131-228
//   summary stats  include/loops/cpu/summarystatsreduce.cpp:24-196
// extraPointers decoding follows blas/cuda/NativeOps.cu:2098-2139 and 1600-1643.
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>

#include "../../include/NativeOps.h"
#include "runtime.h"

using namespace nd4j_amd;

namespace {

static const size_t kScalarArea = 4096;          // first bytes of the workspace: scalar results
static const size_t kWorkspaceBytes = 8u << 20;  // default size; grows on demand

struct Scratch {
    void *scalars;   // kScalarArea bytes
    Workspace rest;  // partial accumulators
};
Scratch scratchFor(hipStream_t s, size_t wantRest = 0) {
    size_t want = kScalarArea + (wantRest > 0 ? wantRest : kWorkspaceBytes - kScalarArea);
    Workspace w = workspaceFor(s, want);
    Scratch sc;
    sc.scalars = w.ptr;
    sc.rest.ptr = reinterpret_cast<char *>(w.ptr) + kScalarArea;
    sc.rest.bytes = w.bytes - kScalarArea;
    addFlatSlots(sc.rest, s);
    return sc;
}

Workspace withSignal(Workspace w, const ScalarSignal &sig) {
    w.signal = sig.words;
    w.ticket = sig.ticket;
    return w;
}

void cLinearMap(const Long *info, DimMap &out) { ownCanon(siRank(info), siShape(info), siStride(info), out); }

// Order-independent full-array walk: 1-D strided when the EWS field says so, otherwise the view with its
// dimensions sorted by stride and merged (a dense f-order array becomes one contiguous run).
FlatPlan flatAnyOrder(const Long *hx) {
    FlatPlan pl;
    pl.n = siNumel(hx);
    Long ews = siEws(hx);
    if (ews >= 1) { pl.strided = true; pl.ews = ews; pl.xm.rank = 0; return pl; }
    const Long *strides[3] = {siStride(hx), nullptr, nullptr};
    DimMap maps[3];
    jointCanon(siRank(hx), siShape(hx), strides, maps);
    if (maps[0].rank == 1) { pl.strided = true; pl.ews = maps[0].stride[0]; pl.xm.rank = 0; return pl; }
    pl.strided = false;
    pl.ews = 0;
    pl.xm = maps[0];
    return pl;
}
// Full-array walk that keeps the element numbering of the reference: memory-linear i*ews when EWS >= 1,
// C-order logical index otherwise (cpu/indexreduce.cpp:43-75).
FlatPlan flatIndexed(const Long *hx) {
    FlatPlan pl;
    pl.n = siNumel(hx);
    Long ews = siEws(hx);
    if (ews >= 1) { pl.strided = true; pl.ews = ews; pl.xm.rank = 0; return pl; }
    pl.strided = false;
    pl.ews = 0;
    cLinearMap(hx, pl.xm);
    return pl;
}

TadPlan tadPlanFrom(const ResolvedTad &t) {
    TadPlan pl;
    pl.tadLength = t.tadLength;
    pl.numTads = t.numTads;
    pl.offsets = t.devOffsets;
    pl.tadEws = siEws(t.hostInfo);
    pl.tm.rank = 0;
    if (pl.tadEws == 1) pl.kind = TadPlan::ROW;
    else if (pl.tadEws > 1) pl.kind = TadPlan::COL;
    else {
        // No element-wise stride in the shapeInfo: the reference walks such a TAD by the C-order coordinates of its
        // elements (cpu/reduce.cpp:173-188, cpu/indexreduce.cpp:197-205).  TADs over several dimensions never carry
        // one (shape::TAD leaves it at -1), whatever their layout, so the layout decides here: a TAD whose dimensions merge
        // into one strided run is walked as the strided kinds walk theirs (same elements, same numbering).
        pl.kind = TadPlan::GENERAL;
        cLinearMap(t.hostInfo, pl.tm);
        if (pl.tm.rank == 1 && pl.tm.stride[0] >= 1) {
            pl.tadEws = pl.tm.stride[0];
            pl.kind = pl.tadEws == 1 ? TadPlan::ROW : TadPlan::COL;
        } else {
            if (pl.tadLength > 0x7fffffffLL)
                throw std::invalid_argument("a TAD without an element-wise stride holds 2^31 elements or more");
            if (pl.tm.stride[pl.tm.rank - 1] == 1 && pl.tm.shape[pl.tm.rank - 1] >= 2) pl.runLength = pl.tm.shape[pl.tm.rank - 1];
        }
    }
    return pl;
}

// The dimensions of the TAD are found among x's by extent and stride, in order (extents of 1 take no part); what is left
// are the dimensions that number the TADs, the last of them varying fastest.
TadPlan tadPlanFrom(const ResolvedTad &t, const Long *hx) {
    TadPlan pl = tadPlanFrom(t);
    const int rank = siRank(hx), tadRank = siRank(t.hostInfo);
    if (rank > kMaxDims) return pl;
    const Long *xs = siShape(hx), *xst = siStride(hx), *ts = siShape(t.hostInfo), *tst = siStride(t.hostInfo);
    bool inTad[kMaxDims];
    int k = 0, last = -1;
    while (k < tadRank && ts[k] == 1) k++;
    for (int d = 0; d < rank; d++) {
        inTad[d] = xs[d] != 1 && k < tadRank && xs[d] == ts[k] && xst[d] == tst[k];
        if (inTad[d]) {
            k++;
            while (k < tadRank && ts[k] == 1) k++;
        } else if (xs[d] != 1) last = d;
    }
    if (k != tadRank || last < 0 || xst[last] != 1 || xs[last] > 0x7fffffffLL) return pl;
    Long g = 0;
    for (int d = 0; d < rank; d++) {
        if (d == last || xs[d] == 1) continue;
        Long a = xst[d] < 0 ? -xst[d] : xst[d];
        while (a != 0) { const Long r = g % a; g = a; a = r; }
    }
    pl.keptInner = (unsigned)xs[last];
    pl.otherStrides = g;
    return pl;
}

float halfBitsToFloatHost(unsigned short h) {
    unsigned sign = (h >> 15) & 1u, exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    unsigned bits;
    if (exp == 0x1f) bits = man ? 0x7fffffffu : ((sign << 31) | 0x7f800000u);
    else if (exp == 0) {
        if (man == 0) bits = sign << 31;
        else {
            int e = -1;
            do { e++; man <<= 1; } while ((man & 0x400u) == 0);
            bits = (sign << 31) | ((unsigned)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else bits = (sign << 31) | ((exp + 112u) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}
template <typename T> struct ScalarOut;
template <> struct ScalarOut<float> { typedef float R; static R get(float v) { return v; } };
template <> struct ScalarOut<double> { typedef double R; static R get(double v) { return v; } };
template <> struct ScalarOut<float16> { typedef float R; static R get(float16 v) { return halfBitsToFloatHost(v.x); } };

template <typename T>
typename ScalarOut<T>::R readScalar(const void *, hipStream_t s, const char *what, const ScalarSignal &sig) {
    T v;
    takeScalar(sig, s, what, &v, sizeof(T));
    return ScalarOut<T>::get(v);
}

// ---- reduce -----------------------------------------------------------------------------------------
template <typename T>
bool reduceScalarTo(hipStream_t s, int opNum, const T *x, const Long *hx, const T *extra, T *zDev, const ScalarSignal &sig = ScalarSignal()) {
    Scratch sc = scratchFor(s);
    FlatPlan pl = flatAnyOrder(hx);
    if (opNum == 19) {
        // LogSumExp: maximum first, then exp(x - max) summed (NativeOpExcutioner.cpp:138-141)
        T *maxSlot = reinterpret_cast<T *>(reinterpret_cast<char *>(sc.scalars) + 64);
        if (!launchReduceScalar<T>(s, 3, x, extra, maxSlot, pl, sc.rest)) return false;
        return launchReduceScalar<T>(s, 19, x, maxSlot, zDev, pl, withSignal(sc.rest, sig));
    }
    return launchReduceScalar<T>(s, opNum, x, extra, zDev, pl, withSignal(sc.rest, sig));
}

template <typename T> typename ScalarOut<T>::R reduceScalar(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return 0;
    Scratch sc = scratchFor(s);
    T *slot = reinterpret_cast<T *>(pinnedScalarFor(s));
    const ScalarSignal sig = nextScalarSignal(s);
    if (!reduceScalarTo<T>(s, opNum, x, hx, params, slot, sig)) { reportUnknownOp("reduce", opNum); return 0; }
    return readScalar<T>(slot, s, "execReduceScalar", sig);
}

template <typename T> void reduceFull(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params, T *z) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return;
    if (!reduceScalarTo<T>(s, opNum, x, hx, params, z)) { reportUnknownOp("reduce", opNum); return; }
    // the reference blocks here (blas/cuda/NativeOps.cu:2049)
    syncAndCheck("execReduce", s);
}

template <typename T>
void reduceDims(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params, T *z, int *dimension, int dimLen) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return;
    if (dimension == nullptr || dimLen == siRank(hx)) {
        if (!reduceScalarTo<T>(s, opNum, x, hx, params, z)) { reportUnknownOp("reduce", opNum); return; }
        checkLaunch("execReduce", s);
        return;
    }
    ResolvedTad t;
    if (!resolveTad(extra, X_HOST_TAD_SHAPE, X_DEV_TAD_OFFSETS, hx, dimension, dimLen, t, s)) return;
    if (t.numTads == 1) {
        if (!reduceScalarTo<T>(s, opNum, x, hx, params, z)) { reportUnknownOp("reduce", opNum); return; }
        checkLaunch("execReduce", s);
        return;
    }
    Scratch sc = scratchFor(s);
    TadPlan pl = tadPlanFrom(t, hx);
    bool ok = true;
    if (opNum == 19) ok = launchReduceTad<T>(s, 3, x, params, z, pl, sc.rest);  // maxima into z first
    ok = ok && launchReduceTad<T>(s, opNum, x, params, z, pl, sc.rest);
    if (!ok) { reportUnknownOp("reduce", opNum); return; }
    checkLaunch("execReduce", s);
}

// ---- index reduce -----------------------------------------------------------------------------------
template <typename T>
bool indexScalarTo(hipStream_t s, int opNum, const T *x, const Long *hx, const T *extra, T *zDev, const ScalarSignal &sig = ScalarSignal()) {
    Scratch sc = scratchFor(s);
    FlatPlan pl = flatIndexed(hx);
    return launchIndexReduceScalar<T>(s, opNum, x, extra, zDev, pl, withSignal(sc.rest, sig));
}

template <typename T> typename ScalarOut<T>::R indexReduceScalar(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return 0;
    Scratch sc = scratchFor(s);
    T *slot = reinterpret_cast<T *>(pinnedScalarFor(s));
    const ScalarSignal sig = nextScalarSignal(s);
    if (!indexScalarTo<T>(s, opNum, x, hx, params, slot, sig)) { reportUnknownOp("indexreduce", opNum); return 0; }
    return readScalar<T>(slot, s, "execIndexReduceScalar", sig);
}

template <typename T>
void indexReduceDims(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params, T *z, Long *zInfo, int *dimension,
                     int dimLen) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return;
    const Long *hz = reinterpret_cast<const Long *>(slotOf(extra, X_HOST_Z_SHAPE));
    bool scalarResult = hz != nullptr ? siIsScalar(hz) : false;
    ResolvedTad t;
    if (!scalarResult) {
        if (dimension == nullptr || dimLen < 1) scalarResult = true;
        else if (!resolveTad(extra, X_HOST_TAD_SHAPE, X_DEV_TAD_OFFSETS, hx, dimension, dimLen, t, s)) return;
        else if (hz == nullptr && t.numTads == 1) scalarResult = true;
    }
    if (scalarResult) {
        if (!indexScalarTo<T>(s, opNum, x, hx, params, z)) { reportUnknownOp("indexreduce", opNum); return; }
        checkLaunch("execIndexReduce", s);
        return;
    }
    Scratch sc = scratchFor(s);
    TadPlan pl = tadPlanFrom(t, hx);
    if (!launchIndexReduceTad<T>(s, opNum, x, params, z, pl, sc.rest)) { reportUnknownOp("indexreduce", opNum); return; }
    checkLaunch("execIndexReduce", s);
}

// ---- summary stats ----------------------------------------------------------------------------------
template <typename T>
bool statsScalarTo(hipStream_t s, int opNum, bool bias, const T *x, const Long *hx, T *zDev, const ScalarSignal &sig = ScalarSignal()) {
    Scratch sc = scratchFor(s);
    FlatPlan pl = flatAnyOrder(hx);
    // the reference walks EWS == 1 arrays linearly and everything else by C-order coordinates
    // (cpu/summarystatsreduce.cpp:31-62); the moments do not depend on the visiting order
    return launchSummaryStatsScalar<T>(s, opNum, bias, x, zDev, pl, withSignal(sc.rest, sig));
}

template <typename T>
typename ScalarOut<T>::R statsScalar(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, bool bias) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return 0;
    Scratch sc = scratchFor(s);
    T *slot = reinterpret_cast<T *>(pinnedScalarFor(s));
    const ScalarSignal sig = nextScalarSignal(s);
    if (!statsScalarTo<T>(s, opNum, bias, x, hx, slot, sig)) { reportUnknownOp("summarystats", opNum); return 0; }
    return readScalar<T>(slot, s, "execSummaryStatsScalar", sig);
}

template <typename T> void statsFull(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *z, bool bias) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return;
    if (!statsScalarTo<T>(s, opNum, bias, x, hx, z)) { reportUnknownOp("summarystats", opNum); return; }
    checkLaunch("execSummaryStats", s);
}

template <typename T>
void statsDims(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *z, Long *zInfo, int *dimension, int dimLen, bool bias) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return;
    const Long *hz = reinterpret_cast<const Long *>(slotOf(extra, X_HOST_Z_SHAPE));
    bool scalarResult = hz != nullptr && siIsScalar(hz);
    ResolvedTad t;
    if (!scalarResult) {
        if (dimension == nullptr || dimLen < 1) scalarResult = true;
        else if (!resolveTad(extra, X_HOST_TAD_SHAPE, X_DEV_TAD_OFFSETS, hx, dimension, dimLen, t, s)) return;
        else {
            // resultLength == 1, all dimensions, or a TAD that is "the whole thing" (TAD.h:337-352) fall back
            // to the scalar routine writing result[0] (cpu/summarystatsreduce.cpp:82-90)
            Long n = siNumel(hx);
            bool whole = false;
            if (!siIsVector(hx))
                whole = t.numTads == 1 || ((dimLen == siRank(hx) || (t.numTads == n && siOrder(hx) == 'c')) && siEws(hx) == 1);
            else if (siIsScalar(hx))
                whole = true;
            Long resultLength = hz != nullptr ? siNumel(hz) : t.numTads;
            if (resultLength == 1 || dimLen == siRank(hx) || whole) scalarResult = true;
        }
    }
    if (scalarResult) {
        if (!statsScalarTo<T>(s, opNum, bias, x, hx, z)) { reportUnknownOp("summarystats", opNum); return; }
        checkLaunch("execSummaryStats", s);
        return;
    }
    Scratch sc = scratchFor(s);
    TadPlan pl = tadPlanFrom(t, hx);
    // single-dimension TADs without an element-wise stride start from a zero sample in the reference
    // (cpu/summarystatsreduce.cpp:92-146, `comp.initWithValue(0.0)`)
    bool phantomZero = dimLen == 1 && siEws(t.hostInfo) < 1;
    if (!launchSummaryStatsTad<T>(s, opNum, bias, phantomZero, x, z, pl, sc.rest)) { reportUnknownOp("summarystats", opNum); return; }
    checkLaunch("execSummaryStats", s);
}

}  // namespace

// ---- reduce3 (include/loops/reduce3.h) -------------------------------------------------------------------
// Index -> offset map of one operand walked by its own linear index in C order ('c') or Fortran order.
void orderedLinearMap(const Long *shape, const Long *stride, int rank, char order, DimMap &out) {
    if (order != 'f') {
        ownCanon(rank, shape, stride, out);
    } else {
        Long rs[kMaxRank], rt[kMaxRank];
        for (int i = 0; i < rank; i++) { rs[i] = shape[rank - 1 - i]; rt[i] = stride[rank - 1 - i]; }
        ownCanon(rank, rs, rt, out);
    }
    if (out.rank < 1) { out.rank = 1; out.shape[0] = 1; out.stride[0] = 1; }
}

// Whole arrays (reduce3.h:838-916): pairs are formed by linear index - memory-linear i * ews when both arrays
// have an element-wise stride and the same order, C-order logical index otherwise.
void reduce3WholePlan(const Long *hx, const Long *hy, Reduce3Launch &in) {
    in.runLength = siNumel(hx);
    in.numOut = 1;
    in.xDiv = in.yMod = 1;
    in.xOffsets = in.yOffsets = nullptr;
    const Long xe = siEws(hx), ye = siEws(hy);
    if (siOrder(hx) == siOrder(hy) && xe >= 1 && ye >= 1) {
        in.xm.rank = in.ym.rank = 1;
        in.xm.shape[0] = in.ym.shape[0] = (unsigned)(in.runLength > 0xffffffffLL ? 0xffffffffu : in.runLength);
        in.xm.stride[0] = xe;
        in.ym.stride[0] = ye;
    } else {
        orderedLinearMap(siShape(hx), siStride(hx), siRank(hx), 'c', in.xm);
        orderedLinearMap(siShape(hy), siStride(hy), siRank(hy), 'c', in.ym);
    }
}

template <typename T>
bool reduce3WholeTo(Nd4jPointer *extra, hipStream_t s, int opNum, T *x, Long *xInfo, T *params, T *y, Long *yInfo, T *zDev,
                    const ScalarSignal &sig = ScalarSignal()) {
    std::vector<Long> sx, sy;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    const Long *hy = hostShapeInfo(extra, X_HOST_Y_SHAPE, yInfo, sy, s);
    if (hx == nullptr || hy == nullptr) return true;
    Reduce3Launch in;
    reduce3WholePlan(hx, hy, in);
    Scratch sc = scratchFor(s);
    if (!launchReduce3<T>(s, opNum, x, y, zDev, params, in, withSignal(sc.rest, sig))) { reportUnknownOp("reduce3", opNum); return false; }
    return true;
}

template <typename T>
typename ScalarOut<T>::R reduce3Scalar(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params, T *y, Long *yInfo) {
    hipStream_t s = streamOf(extra);
    T *slot = reinterpret_cast<T *>(pinnedScalarFor(s));
    const ScalarSignal sig = nextScalarSignal(s);
    if (!reduce3WholeTo<T>(extra, s, opNum, x, xInfo, params, y, yInfo, slot, sig)) return 0;
    return readScalar<T>(slot, s, "execReduce3Scalar", sig);
}

template <typename T>
void reduce3Full(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params, T *y, Long *yInfo, T *z) {
    hipStream_t s = streamOf(extra);
    if (!reduce3WholeTo<T>(extra, s, opNum, x, xInfo, params, y, yInfo, z)) return;
    checkLaunch("execReduce3", s);
}

// Along `dimension` (reduce3.h:998-1081 with a caller's TAD tables, 1083-1346 without): result r is the pair
// (TAD r of x, TAD r of y) when the arrays are equally long, (TAD r of x, all of y) when y holds one TAD's
// worth of elements.  Elements pair up by their linear index inside the TAD in the TAD's own order.
template <typename T>
void reduce3Dims(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params, T *y, Long *yInfo, T *z, Long *zInfo,
                 int *dimension, int dimLen) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx, sy, sz;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    const Long *hy = hostShapeInfo(extra, X_HOST_Y_SHAPE, yInfo, sy, s);
    const Long *hz = hostShapeInfo(extra, X_HOST_Z_SHAPE, zInfo, sz, s);
    if (hx == nullptr || hy == nullptr || hz == nullptr) return;
    if (siIsScalar(hz) || dimension == nullptr || dimLen >= siRank(hx)) {
        reduce3Full<T>(extra, opNum, x, xInfo, params, y, yInfo, z);
        return;
    }
    if (siNumel(hx) < siNumel(hy)) {
        // x is the single run, y has the TADs (reduce3.h:1186-1215 picks the longer operand to iterate over)
        ResolvedTad ty;
        if (!resolveTad(nullptr, 0, 0, hy, dimension, dimLen, ty, s)) return;
        if (siNumel(hx) != ty.tadLength) {
            std::printf("reduce3: x holds %lld elements, neither the %lld of y nor the %lld of one TAD\n", (long long)siNumel(hx),
                        (long long)siNumel(hy), (long long)ty.tadLength);
            return;
        }
        Reduce3Launch in;
        in.runLength = ty.tadLength;
        in.numOut = ty.numTads;
        in.xDiv = 1;
        in.yMod = ty.numTads > 0 ? ty.numTads : 1;
        in.xOffsets = nullptr;
        in.yOffsets = ty.devOffsets;
        const char order = siOrder(ty.hostInfo) == 'f' ? 'f' : 'c';
        orderedLinearMap(siShape(hx), siStride(hx), siRank(hx), order, in.xm);
        orderedLinearMap(siShape(ty.hostInfo), siStride(ty.hostInfo), siRank(ty.hostInfo), order, in.ym);
        Scratch sc = scratchFor(s);
        if (!launchReduce3<T>(s, opNum, x, y, z, params, in, sc.rest)) { reportUnknownOp("reduce3", opNum); return; }
        checkLaunch("execReduce3", s);
        return;
    }
    ResolvedTad tx;
    if (!resolveTad(extra, X_HOST_TAD_SHAPE, X_DEV_TAD_OFFSETS, hx, dimension, dimLen, tx, s)) return;
    Reduce3Launch in;
    in.runLength = tx.tadLength;
    in.numOut = tx.numTads;
    in.xDiv = 1;
    in.yMod = tx.numTads > 0 ? tx.numTads : 1;
    in.xOffsets = tx.devOffsets;
    const char order = siOrder(tx.hostInfo) == 'f' ? 'f' : 'c';
    orderedLinearMap(siShape(tx.hostInfo), siStride(tx.hostInfo), siRank(tx.hostInfo), order, in.xm);
    if (siNumel(hy) == siNumel(hx)) {
        // a y laid out like x shares its TAD tables; any other layout gets tables of its own (which needs the
        // dimensions on the host, a small synchronous copy)
        ResolvedTad ty;
        bool sameLayout = siRank(hy) == siRank(hx) && siOrder(hy) == siOrder(hx);
        for (int d = 0; sameLayout && d < siRank(hx); d++)
            sameLayout = siShape(hy)[d] == siShape(hx)[d] && siStride(hy)[d] == siStride(hx)[d];
        if (sameLayout) ty = tx;
        else if (!resolveTad(nullptr, 0, 0, hy, dimension, dimLen, ty, s)) return;
        in.yOffsets = ty.devOffsets;
        orderedLinearMap(siShape(ty.hostInfo), siStride(ty.hostInfo), siRank(ty.hostInfo), order, in.ym);
    } else if (siNumel(hy) == tx.tadLength) {
        in.yOffsets = nullptr;
        orderedLinearMap(siShape(hy), siStride(hy), siRank(hy), order, in.ym);
    } else {
        std::printf("reduce3: y holds %lld elements, neither the %lld of x nor the %lld of one TAD\n", (long long)siNumel(hy),
                    (long long)siNumel(hx), (long long)tx.tadLength);
        return;
    }
    Scratch sc = scratchFor(s);
    if (!launchReduce3<T>(s, opNum, x, y, z, params, in, sc.rest)) { reportUnknownOp("reduce3", opNum); return; }
    checkLaunch("execReduce3", s);
}

// Every TAD of x against every TAD of y (reduce3.h:918-995): result[r * yTads + g].
template <typename T>
void reduce3All(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *params, T *y, Long *yInfo, T *z, int *dimension,
                int dimLen, const Long *xOffsetsDev, const Long *yOffsetsDev) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx, sy;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    const Long *hy = hostShapeInfo(extra, X_HOST_Y_SHAPE, yInfo, sy, s);
    if (hx == nullptr || hy == nullptr) return;
    ResolvedTad tx, ty;
    // What nd4j passes (blas/cuda/NativeOps.cu, execReduce3AllFloat): the device offset tables of both operands as
    // arguments and the host shapeInfo of x's TAD in extraPointers[9].  That describes y's TADs too when y is laid
    // out like x in every dimension but the first (the usual case: two batches of equally shaped rows); then nothing
    // has to be read back.  Otherwise the dimensions are fetched once and serve both operands.
    const Long *hostTad = reinterpret_cast<const Long *>(slotOf(extra, X_HOST_TAD_SHAPE));
    bool sameTads = hostTad != nullptr && xOffsetsDev != nullptr && yOffsetsDev != nullptr && siRank(hx) == siRank(hy) &&
                    siOrder(hx) == siOrder(hy) && siNumel(hostTad) > 0 && siNumel(hx) % siNumel(hostTad) == 0 &&
                    siNumel(hy) % siNumel(hostTad) == 0;
    for (int d = 0; sameTads && d < siRank(hx); d++)
        sameTads = siStride(hx)[d] == siStride(hy)[d] && (d == 0 || siShape(hx)[d] == siShape(hy)[d]);
    if (sameTads) {
        tx.hostInfo = ty.hostInfo = hostTad;
        tx.tadLength = ty.tadLength = siNumel(hostTad);
        tx.devOffsets = xOffsetsDev;
        ty.devOffsets = yOffsetsDev;
        tx.numTads = siNumel(hx) / tx.tadLength;
        ty.numTads = siNumel(hy) / ty.tadLength;
    } else {
        std::vector<int> dims;
        if (!hostInts(dimension, dimLen, dims, s)) return;
        if (!resolveTad(nullptr, 0, 0, hx, dims.data(), dimLen, tx, s)) return;
        if (!resolveTad(nullptr, 0, 0, hy, dims.data(), dimLen, ty, s)) return;
    }
    if (tx.tadLength != ty.tadLength) {
        std::printf("reduce3All: TAD lengths differ (%lld vs %lld)\n", (long long)tx.tadLength, (long long)ty.tadLength);
        return;
    }
    Reduce3Launch in;
    in.runLength = tx.tadLength;
    in.numOut = tx.numTads * ty.numTads;
    in.xDiv = ty.numTads > 0 ? ty.numTads : 1;
    in.yMod = in.xDiv;
    in.xOffsets = tx.devOffsets;
    in.yOffsets = ty.devOffsets;
    in.allPairs = true;
    orderedLinearMap(siShape(tx.hostInfo), siStride(tx.hostInfo), siRank(tx.hostInfo), siOrder(tx.hostInfo) == 'f' ? 'f' : 'c', in.xm);
    orderedLinearMap(siShape(ty.hostInfo), siStride(ty.hostInfo), siRank(ty.hostInfo), siOrder(ty.hostInfo) == 'f' ? 'f' : 'c', in.ym);
    Scratch sc = scratchFor(s);
    if (!launchReduce3<T>(s, opNum, x, y, z, params, in, sc.rest)) { reportUnknownOp("reduce3", opNum); return; }
    checkLaunch("execReduce3All", s);
}

// ---- special transforms (include/ops/special_ops.h:1422-2260) -------------------------------------------
namespace nd4j_amd {

// IsMax over a whole array, both operands dense with the same number of elements, on the same offset from a 16-byte
// boundary, and either the same array or two that do not overlap: the index reduction clears z while it reads x.
template <typename T>
bool specialTransform(Nd4jPointer *extra, int opNum, T *x, const Long *hx, T *z, const Long *hz, T *params, hipStream_t s) {
    if (opNum < 38 || opNum > 41) return false;
    const int rank = siRank(hx);
    const Long n = siNumel(hx);
    if (n <= 0) return true;
    if (opNum != 41) {
        // SoftMax family: over each row of a matrix, over a vector as a whole; other ranks are left alone, as in
        // the reference (special_ops.h:1483, 1533)
        SoftmaxPlan pl;
        const bool vector = rank <= 1 || (rank == 2 && (siShape(hx)[0] == 1 || siShape(hx)[1] == 1));
        int walked = 1;  // the dimension of x that a row runs along
        if (vector) {
            pl.numRows = 1;
            pl.length = n;
            pl.xRow = pl.zRow = 0;
            // the stride of the dimension that is walked (the EWS field says the same for a vector)
            const int xd = (rank == 2 && siShape(hx)[0] != 1) ? 0 : rank - 1;
            const int zd = (siRank(hz) == 2 && siShape(hz)[0] != 1) ? 0 : siRank(hz) - 1;
            walked = xd;
            pl.xEl = rank >= 1 ? siStride(hx)[xd] : 1;
            pl.zEl = siRank(hz) >= 1 ? siStride(hz)[zd] : 1;
        } else if (rank == 2 && siRank(hz) == 2) {
            pl.numRows = siShape(hx)[0];
            pl.length = siShape(hx)[1];
            pl.xRow = siStride(hx)[0];
            pl.xEl = siStride(hx)[1];
            pl.zRow = siStride(hz)[0];
            pl.zEl = siStride(hz)[1];
        } else {
            return true;
        }
        // Rows that do not fit the register-resident kernels.  A block (or a wave) per row would read the row three
        // times, and would leave most of the chip idle when the rows are few.  The row maxima and the row sums of
        // exp(x - max) come from one pass of the reduction kernels instead, which cut long rows into slices, and one
        // elementwise pass finishes: 12 bytes per element.  Measured against the per-row kernels this wins for rows of
        // 16384 elements or more, for shorter rows when they are few, and always for f-order matrices.
        if (rank >= 1 && pl.xRow == 1 && pl.zRow == 1 && pl.numRows >= 256) {
            // an f-order matrix with more columns than half a compute unit's registers hold of a group of rows: one
            // pass, the blocks that share the group's columns exchanging the rows' maxima and sums
            Scratch coop = scratchFor(s);
            if (launchSoftmaxColCooperative<T>(s, opNum, x, z, pl, coop.rest)) {
                checkLaunch("execTransform(softmax)", s);
                return true;
            }
        }
        const bool rowMajor = pl.xEl == 1 && pl.zEl == 1 && (pl.length >= 16384 || (pl.length >= 4096 && pl.numRows <= 512));
        const bool colMajor = pl.xRow == 1 && pl.zRow == 1 && pl.numRows >= 256 && pl.length >= 256;
        if (rank >= 1 && (rowMajor || colMajor) && !softmaxFitsRegisters<T>(x, z, pl)) {
            // (the rows' table is looked up before the one-pass kernel is tried, which does not need it: a stream under
            // capture, where that kernel is not available, then finds the table its eager calls left in the cache)
            ResolvedTad tx;
            if (!resolveTad(nullptr, 0, 0, hx, &walked, 1, tx, s)) return true;
            typedef typename Compute<T>::type C;  // the row sums stay in the compute type: those of half rows may exceed half
            const size_t perRow = ((size_t)pl.numRows * sizeof(C) + 255) / 256 * 256;
            Scratch sc = scratchFor(s, 2 * perRow + kWorkspaceBytes);  // (sized for the two-pass form in either case, for the same reason)
            if (rowMajor) {
                // aligned rows: one pass, the blocks of a row exchanging their maxima and sums
                if (launchSoftmaxCooperative<T>(s, opNum, x, z, pl, sc.rest)) {
                    checkLaunch("execTransform(softmax)", s);
                    return true;
                }
            }
            T *maxima = reinterpret_cast<T *>(sc.rest.ptr);
            C *sums = reinterpret_cast<C *>(reinterpret_cast<char *>(sc.rest.ptr) + perRow);
            Workspace rest;
            rest.ptr = reinterpret_cast<char *>(sc.rest.ptr) + 2 * perRow;
            rest.bytes = sc.rest.bytes - 2 * perRow;
            const TadPlan tp = tadPlanFrom(tx);
            if (!launchSoftmaxStats<T>(s, x, maxima, sums, tp, rest)) return false;
            if (!launchSoftmaxFinish<T>(s, opNum, x, z, maxima, sums, pl)) return false;
            checkLaunch("execTransform(softmax)", s);
            return true;
        }
        if (!launchSoftmax<T>(s, opNum, x, z, pl)) return false;
        checkLaunch("execTransform(softmax)", s);
        return true;
    }
    // IsMax.  Without extraParams (or with the "all dimensions" marker): one-hot of the first maximum of the whole
    // array.  With dimensions - extraPointers[15] / [18] hold the device dimension array and its length
    // (blas/cuda/NativeOps.cu:3280-3284): one-hot per TAD.
    int dimLen = 0;
    const int *devDims = nullptr;
    if (params != nullptr && extra != nullptr) {
        devDims = reinterpret_cast<const int *>(slotOf(extra, 15));
        dimLen = (int)reinterpret_cast<intptr_t>(slotOf(extra, 18));
        if (devDims == nullptr || dimLen <= 0 || dimLen >= rank) dimLen = 0;
    }
    if (dimLen == 0) {
        Scratch sc = scratchFor(s);
        T *slot = reinterpret_cast<T *>(sc.scalars);
        FlatPlan xp = flatIndexed(hx);
        FlatPlan zp = flatIndexed(hz);
        // (two passes - the index of the maximum, then a fill - take 83 us over 2^26 floats; one pass that cleared the
        // result while it looked for the maximum, and set the one element afterwards, took 96)
        if (!launchIndexReduceScalar<T>(s, 0, x, nullptr, slot, xp, sc.rest)) return false;
        launchIsMaxFill<T>(s, z, slot, zp);
        checkLaunch("execTransform(IsMax)", s);
        return true;
    }
    ResolvedTad tx, tz;
    if (!resolveTad(extra, X_HOST_TAD_SHAPE, X_DEV_TAD_OFFSETS, hx, devDims, dimLen, tx, s)) return true;
    // a result laid out like the input shares its TAD tables (the reference's fill kernel always assumes so,
    // blas/cuda/NativeOps.cu:3277-3290); any other layout gets tables of its own
    bool sameLayout = siRank(hz) == rank && siOrder(hz) == siOrder(hx);
    for (int d = 0; sameLayout && d < rank; d++)
        sameLayout = siShape(hz)[d] == siShape(hx)[d] && siStride(hz)[d] == siStride(hx)[d];
    if (sameLayout) tz = tx;
    else if (!resolveTad(nullptr, 0, 0, hz, devDims, dimLen, tz, s)) return true;
    Scratch sc = scratchFor(s, kScalarArea + (size_t)tx.numTads * sizeof(T) + (size_t)(4u << 20));
    T *index = reinterpret_cast<T *>(sc.rest.ptr);
    Workspace rest = sc.rest;
    size_t used = ((size_t)tx.numTads * sizeof(T) + 255) / 256 * 256;
    rest.ptr = reinterpret_cast<char *>(rest.ptr) + used;
    rest.bytes -= used;
    TadPlan xp = tadPlanFrom(tx);
    if (tx.numTads == 1) {
        FlatPlan fp = flatIndexed(hx);
        if (!launchIndexReduceScalar<T>(s, 0, x, nullptr, index, fp, rest)) return false;
    } else if (!launchIndexReduceTad<T>(s, 0, x, nullptr, index, xp, rest)) {
        return false;
    }
    TadPlan zp = tadPlanFrom(tz);
    if (tx.numTads == 1) {
        FlatPlan fz = flatIndexed(hz);
        launchIsMaxFill<T>(s, z, index, fz);
    } else {
        launchIsMaxTadFill<T>(s, z, index, zp);
    }
    checkLaunch("execTransform(IsMax)", s);
    return true;
}

#define INST(T) \
    template bool specialTransform<T>(Nd4jPointer *, int, T *, const Long *, T *, const Long *, T *, hipStream_t);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd

// ---- whole-array reduction that allocates nothing ---------------------------------------------------------
// No counterpart in the reference.  Same result as execReduceFloat without dimensions (result[0] on the device), for
// callers that may not allocate: the partial accumulators live in a file-scope device array (reduce.hip), the host
// shapeInfo must be at hand (extraPointers[0], or a host pointer as xShapeInfo), nothing is read back and nothing is
// synchronised.  Calls that overlap on one GPU race on the shared array.
namespace nd4j_amd {
static const Long kNoAllocMaxElements = (Long)1 << 36;  // 256 GiB of floats: beyond what one GPU's memory holds

void reduceFloatNoAlloc(Nd4jPointer *extra, int opNum, float *x, Long *xInfo, float *params, float *z) {
    hipStream_t s = streamOf(extra);
    const Long *hx = reinterpret_cast<const Long *>(slotOf(extra, X_HOST_X_SHAPE));
    if (hx == nullptr && xInfo != nullptr && !isDeviceMemory(xInfo)) hx = xInfo;
    if (hx == nullptr)
        throw std::invalid_argument("execReduceFloatNoAlloc: needs the host copy of xShapeInfo in extraPointers[0] "
                                    "(a device shapeInfo would have to be read back)");
    if (x == nullptr || z == nullptr) throw std::invalid_argument("execReduceFloatNoAlloc: null data pointer");
    const Long rank = hx[0];
    if (rank < 0 || rank > kMaxRank) throw std::invalid_argument("execReduceFloatNoAlloc: shapeInfo rank out of range");
    const Long n = siNumel(hx);
    if (n < 1) throw std::invalid_argument("execReduceFloatNoAlloc: empty array");
    if (n > kNoAllocMaxElements)
        throw std::invalid_argument("execReduceFloatNoAlloc: " + std::to_string(n) + " elements; at most 2^36 are accepted");
    FlatPlan pl = flatAnyOrder(hx);
    if (!launchReduceScalarNoAlloc(s, opNum, x, params, z, pl))
        throw std::invalid_argument("execReduceFloatNoAlloc: unknown opNum " + std::to_string(opNum));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) throw std::runtime_error(std::string("execReduceFloatNoAlloc: ") + hipGetErrorString(e));
}
}  // namespace nd4j_amd

#define ND4J_REDUCE3_MEMBERS(SUFFIX, T, R)                                                                          \
    void NativeOps::execReduce3##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,          \
                                        T *extraParamsVals, T *y, Nd4jLong *yShapeInfo, T *result,                  \
                                        Nd4jLong *resultShapeInfo) {                                                \
        (void)resultShapeInfo;                                                                                      \
        reduce3Full<T>(extraPointers, opNum, x, xShapeInfo, extraParamsVals, y, yShapeInfo, result);                \
    }                                                                                                               \
    R NativeOps::execReduce3Scalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,       \
                                           T *extraParamsVals, T *y, Nd4jLong *yShapeInfo) {                        \
        return reduce3Scalar<T>(extraPointers, opNum, x, xShapeInfo, extraParamsVals, y, yShapeInfo);               \
    }                                                                                                               \
    void NativeOps::execReduce3##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,          \
                                        T *extraParamsVals, T *y, Nd4jLong *yShapeInfo, T *result,                  \
                                        Nd4jLong *resultShapeInfoBuffer, int *dimension, int dimensionLength) {     \
        reduce3Dims<T>(extraPointers, opNum, x, xShapeInfo, extraParamsVals, y, yShapeInfo, result,                 \
                       resultShapeInfoBuffer, dimension, dimensionLength);                                          \
    }                                                                                                               \
    void NativeOps::execReduce3All##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xInfo,            \
                                           T *extraParamsVals, T *y, Nd4jLong *yInfo, T *result,                    \
                                           Nd4jLong *resultShapeInfoBuffer, int *dimension, int dimensionLength,    \
                                           Nd4jLong *xTadShapeInfo, Nd4jLong *xOffsets, Nd4jLong *yTadShapeInfo,    \
                                           Nd4jLong *yOffsets) {                                                    \
        (void)resultShapeInfoBuffer; (void)xTadShapeInfo; (void)yTadShapeInfo;                                      \
        reduce3All<T>(extraPointers, opNum, x, xInfo, extraParamsVals, y, yInfo, result, dimension,                 \
                      dimensionLength, xOffsets, yOffsets);                                                         \
    }

#define ND4J_REDUCE_MEMBERS(SUFFIX, T, R)                                                                            \
    R NativeOps::execReduceScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,         \
                                          T *extraParams) {                                                          \
        return reduceScalar<T>(extraPointers, opNum, x, xShapeInfo, extraParams);                                    \
    }                                                                                                                \
    void NativeOps::execReduce##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,            \
                                       T *extraParams, T *result, Nd4jLong *) {                                      \
        reduceFull<T>(extraPointers, opNum, x, xShapeInfo, extraParams, result);                                     \
    }                                                                                                                \
    void NativeOps::execReduce##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,            \
                                       T *extraParams, T *result, Nd4jLong *, int *dimension, int dimensionLength) { \
        reduceDims<T>(extraPointers, opNum, x, xShapeInfo, extraParams, result, dimension, dimensionLength);         \
    }                                                                                                                \
    R NativeOps::execIndexReduceScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,    \
                                               T *extraParams) {                                                     \
        return indexReduceScalar<T>(extraPointers, opNum, x, xShapeInfo, extraParams);                               \
    }                                                                                                                \
    void NativeOps::execIndexReduce##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,       \
                                            T *extraParams, T *result, Nd4jLong *resultShapeInfoBuffer,              \
                                            int *dimension, int dimensionLength) {                                   \
        indexReduceDims<T>(extraPointers, opNum, x, xShapeInfo, extraParams, result, resultShapeInfoBuffer,          \
                           dimension, dimensionLength);                                                              \
    }                                                                                                                \
    R NativeOps::execSummaryStatsScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,   \
                                                T *, bool biasCorrected) {                                           \
        return statsScalar<T>(extraPointers, opNum, x, xShapeInfo, biasCorrected);                                   \
    }                                                                                                                \
    void NativeOps::execSummaryStats##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *, \
                                             T *result, Nd4jLong *, bool biasCorrected) {                            \
        statsFull<T>(extraPointers, opNum, x, xShapeInfo, result, biasCorrected);                                    \
    }                                                                                                                \
    void NativeOps::execSummaryStats##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *, \
                                             T *result, Nd4jLong *resultShapeInfoBuffer, int *dimension,             \
                                             int dimensionLength, bool biasCorrected) {                              \
        statsDims<T>(extraPointers, opNum, x, xShapeInfo, result, resultShapeInfoBuffer, dimension,                  \
                     dimensionLength, biasCorrected);                                                                \
    }

ND4J_REDUCE_MEMBERS(Float, float, float)
ND4J_REDUCE_MEMBERS(Half, float16, float)
ND4J_REDUCE_MEMBERS(Double, double, double)
ND4J_REDUCE3_MEMBERS(Float, float, float)
ND4J_REDUCE3_MEMBERS(Half, float16, float)
ND4J_REDUCE3_MEMBERS(Double, double, double)
