// NativeOps boundary, part 1: lifecycle members and the elementwise families (transform, pairwise,
// broadcast).  Branch selection follows the reference's CPU loops, which are the parity oracle:
//   transform  include/loops/cpu/transform.cpp:28-89
//   pairwise   include/loops/pairwise_transform.h:154-366
//   broadcast  include/loops/cpu/broadcasting.cpp:42-156
// extraPointers are decoded as the reference's CUDA back end does (blas/cuda/NativeOps.cu:1813-1823,
// 3100-3131).
#include <atomic>
#include <cstdio>
#include <cstring>
#include <stdexcept>

#include "../../include/NativeOps.h"
#include "runtime.h"

using namespace nd4j_amd;

namespace {

inline bool sameShape(const Long *a, const Long *b) {
    if (siRank(a) != siRank(b)) return false;
    for (int i = 0; i < siRank(a); i++)
        if (siShape(a)[i] != siShape(b)[i]) return false;
    return true;
}

// true when the strides are those of a gap-free array in the given order (unit dimensions may carry any stride)
inline bool isDense(const Long *info, char order) {
    const int rank = siRank(info);
    Long expect = 1;
    for (int k = 0; k < rank; k++) {
        const int d = order == 'c' ? rank - 1 - k : k;
        if (siShape(info)[d] != 1 && siStride(info)[d] != expect) return false;
        expect *= siShape(info)[d];
    }
    return true;
}

// Index -> offset map of one operand walked by its own linear index, in C order or Fortran order.
void linearMap(const Long *shape, const Long *stride, int rank, char order, DimMap &out) {
    if (order == 'c') {
        ownCanon(rank, shape, stride, out);
        return;
    }
    Long rs[kMaxRank], rt[kMaxRank];
    for (int i = 0; i < rank; i++) { rs[i] = shape[rank - 1 - i]; rt[i] = stride[rank - 1 - i]; }
    ownCanon(rank, rs, rt, out);
}

// DropOut 43 / DropOutInverted 44 (include/ops/ops.h:3520-3562) draw from an unseeded generator in the reference; here
// every call takes the next value of a process-wide counter as its seed.
constexpr int kDropOut = 43, kDropOutInverted = 44;
unsigned long long nextDropoutSeed() {
    static std::atomic<unsigned long long> calls{0};
    return (calls.fetch_add(1) + 1) * 0x2545f4914f6cdd1dull;
}
template <typename T>
void dropoutTransform(hipStream_t s, int opNum, T *x, const DimMap &xm, T *z, const DimMap &zm, T *params, Long n) {
    if (params == nullptr) throw std::invalid_argument("DropOut: extraParams [probability] required");
    launchDropoutTransform<T>(s, opNum == kDropOutInverted, x, xm, z, zm, params, n, nextDropoutSeed());
    checkLaunch("execTransform(dropout)", s);
}
void stridedMap(Long n, Long stride, DimMap &m) {
    m.rank = 1;
    m.shape[0] = (unsigned)(n > 0xffffffffLL ? 0xffffffffu : n);
    m.stride[0] = stride;
}

template <typename T>
void transformStrided(Nd4jPointer *extra, int opNum, T *x, Long xs, T *z, Long zs, T *params, Long n) {
    hipStream_t s = streamOf(extra);
    if (opNum == kDropOut || opNum == kDropOutInverted) {
        DimMap xm, zm;
        stridedMap(n, xs, xm);
        stridedMap(n, zs, zm);
        dropoutTransform<T>(s, opNum, x, xm, z, zm, params, n);
        return;
    }
    if (!launchTransformStrided<T>(s, opNum, x, xs, z, zs, params, n)) { reportUnknownOp("transform", opNum); return; }
    checkLaunch("execTransform(strided)", s);
}

template <typename T>
void transformShaped(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *z, Long *zInfo, T *params) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx, sz;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    const Long *hz = hostShapeInfo(extra, X_HOST_Z_SHAPE, zInfo, sz, s);
    if (hx == nullptr || hz == nullptr) return;
    if (opNum >= 38 && opNum <= 41) {
        // whole-array special ops: SoftMax, SoftMaxDerivative, LogSoftMax, IsMax
        if (!specialTransform<T>(extra, opNum, x, hx, z, hz, params, s)) reportUnknownOp("transform", opNum);
        return;
    }
    if (wholeArrayTransform<T>(opNum, x, hx, z, hz, params, s)) {
        // Col2Im, Im2col, Histogram, Reverse, Pooling2D
        checkLaunch("execTransform(whole array)", s);
        return;
    }
    Long n = siNumel(hx);
    Long xe = siEws(hx), ze = siEws(hz);
    bool ok;
    if (xe >= 1 && ze >= 1 && siOrder(hx) == siOrder(hz)) {
        if (opNum == kDropOut || opNum == kDropOutInverted) {
            transformStrided<T>(extra, opNum, x, xe, z, ze, params, n);
            return;
        }
        ok = launchTransformStrided<T>(s, opNum, x, xe, z, ze, params, n);
    } else {
        // same logical coordinates on both sides (raw iteration over x's shape)
        const Long *strides[3] = {siStride(hx), nullptr, siStride(hz)};
        DimMap maps[3];
        jointCanon(siRank(hx), siShape(hx), strides, maps);
        if (opNum == kDropOut || opNum == kDropOutInverted) {
            dropoutTransform<T>(s, opNum, x, maps[0], z, maps[2], params, n);
            return;
        }
        ok = launchTransformGeneral<T>(s, opNum, x, maps[0], z, maps[2], params, n);
    }
    if (!ok) { reportUnknownOp("transform", opNum); return; }
    checkLaunch("execTransform", s);
}

template <typename T>
void pairwiseStrided(Nd4jPointer *extra, int opNum, T *x, Long xs, T *y, Long ys, T *z, Long zs, T *params, Long n) {
    hipStream_t s = streamOf(extra);
    bool ok;
    if (ys == 0) {
        // a literal zero stride is a valid (if unusual) request: every element pairs with y[0]
        DimMap xm, ym, zm;
        xm.rank = ym.rank = zm.rank = 1;
        xm.shape[0] = ym.shape[0] = zm.shape[0] = (unsigned)n;
        xm.stride[0] = xs; ym.stride[0] = 0; zm.stride[0] = zs;
        ok = launchPairwiseGeneral<T>(s, opNum, x, xm, y, ym, z, zm, params, n);
    } else {
        ok = launchPairwiseStrided<T>(s, opNum, x, xs, y, ys, z, zs, params, n);
    }
    if (!ok) { reportUnknownOp("pairwise", opNum); return; }
    checkLaunch("execPairwiseTransform(strided)", s);
}

template <typename T>
void pairwiseShaped(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *y, Long *yInfo, T *z, Long *zInfo, T *params) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx, sy, sz;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    const Long *hy = hostShapeInfo(extra, X_HOST_Y_SHAPE, yInfo, sy, s);
    const Long *hz = hostShapeInfo(extra, X_HOST_Z_SHAPE, zInfo, sz, s);
    if (hx == nullptr || hy == nullptr || hz == nullptr) return;
    Long n = siNumel(hx);
    Long xe = siEws(hx), ye = siEws(hy), ze = siEws(hz);
    bool ok;
    if (siIsScalar(hy)) {
        if (xe == 1 && ze == 1) {
            ok = launchPairwiseStrided<T>(s, opNum, x, 1, y, 0, z, 1, params, n);
        } else {
            DimMap xm, ym, zm;
            linearMap(siShape(hx), siStride(hx), siRank(hx), 'c', xm);
            linearMap(siShape(hz), siStride(hz), siRank(hz), 'c', zm);
            ym.rank = 1; ym.shape[0] = 1; ym.stride[0] = 0;
            ok = launchPairwiseGeneral<T>(s, opNum, x, xm, y, ym, z, zm, params, n);
        }
    } else {
        bool same = sameShape(hx, hy);
        bool ordersEqual = siOrder(hx) == siOrder(hy) && siOrder(hz) == siOrder(hx);
        bool ewsOk = xe >= 1 && ye >= 1 && ze >= 1 && xe == ye;
        if (ewsOk && ordersEqual) {
            // same shape: n elements; different shapes: length(y) elements (pairwise_transform.h:209-239)
            Long count = same ? n : siNumel(hy);
            ok = launchPairwiseStrided<T>(s, opNum, x, xe, y, ye, z, ze, params, count);
        } else if (same) {
            const Long *strides[3] = {siStride(hx), siStride(hy), siStride(hz)};
            DimMap maps[3];
            jointCanon(siRank(hx), siShape(hx), strides, maps);
            ok = launchPairwiseGeneral<T>(s, opNum, x, maps[0], y, maps[1], z, maps[2], params, n);
        } else {
            DimMap xm, ym, zm;
            linearMap(siShape(hx), siStride(hx), siRank(hx), 'c', xm);
            linearMap(siShape(hy), siStride(hy), siRank(hy), 'c', ym);
            if (x == z) zm = xm;
            else linearMap(siShape(hz), siStride(hz), siRank(hz), 'c', zm);
            ok = launchPairwiseGeneral<T>(s, opNum, x, xm, y, ym, z, zm, params, n);
        }
    }
    if (!ok) { reportUnknownOp("pairwise", opNum); return; }
    checkLaunch("execPairwiseTransform", s);
}

template <typename T>
void broadcastShaped(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *y, Long *yInfo, T *z, Long *zInfo,
                     int *dimension, int dimLen) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx, sy, sz, szt;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    const Long *hy = hostShapeInfo(extra, X_HOST_Y_SHAPE, yInfo, sy, s);
    const Long *hz = hostShapeInfo(extra, X_HOST_Z_SHAPE, zInfo, sz, s);
    if (hx == nullptr || hy == nullptr || hz == nullptr) return;

    ResolvedTad tx;
    if (!resolveTad(extra, X_HOST_TAD_SHAPE, X_DEV_TAD_OFFSETS, hx, dimension, dimLen, tx, s)) return;

    // TADs of the result: the caller's tables when given, else those of x (cpu/broadcasting.cpp:79-82).
    const Long *zTadInfo = tx.hostInfo;
    const Long *zOffsets = tx.devOffsets;
    const Long *devZTad = reinterpret_cast<const Long *>(slotOf(extra, X_DEV_TAD_SHAPE_Z));
    const Long *devZOff = reinterpret_cast<const Long *>(slotOf(extra, X_DEV_TAD_OFFSETS_Z));
    if (devZTad != nullptr && devZOff != nullptr) {
        zOffsets = devZOff;
        bool zLikeX = siRank(hx) == siRank(hz) &&
                      std::memcmp(hx, hz, sizeof(Long) * siLength(siRank(hx))) == 0;
        if (!zLikeX) {
            zTadInfo = hostShapeInfo(nullptr, 0, devZTad, szt, s);
            if (zTadInfo == nullptr) return;
        }
    }

    BroadcastPlan pl;
    pl.tadLength = tx.tadLength;
    pl.numTads = tx.numTads;
    pl.xOffsets = tx.devOffsets;
    pl.zOffsets = zOffsets;
    pl.tadEws = siEws(tx.hostInfo);
    pl.yEws = siEws(hy);
    pl.zEws = siEws(zTadInfo);
    // The reference takes its strided loop only for a single dimension whose TAD, y and result TAD all carry an
    // element-wise stride (cpu/broadcasting.cpp:95), and coordinate arithmetic per element otherwise.  Both visit element f
    // of every TAD with element f of y, so what decides the kernel here is the layout: TADs over several dimensions
    // (whose shapeInfo never carries an element-wise stride) that are one strided run all the same take the strided
    // kernels too.
    bool stridedWalk = pl.tadEws > 0 && pl.yEws > 0 && pl.zEws > 0 && dimLen == 1;
    if (!stridedWalk) {
        char xo = siOrder(tx.hostInfo) == 'c' ? 'c' : 'f';
        char zo = siOrder(zTadInfo) == 'c' ? 'c' : 'f';
        linearMap(siShape(tx.hostInfo), siStride(tx.hostInfo), siRank(tx.hostInfo), xo, pl.xm);
        linearMap(siShape(hy), siStride(hy), siRank(hy), xo, pl.ym);
        linearMap(siShape(zTadInfo), siStride(zTadInfo), siRank(zTadInfo), zo, pl.zm);
        if (pl.xm.rank == 1 && pl.ym.rank == 1 && pl.zm.rank == 1 && pl.xm.stride[0] > 0 && pl.ym.stride[0] > 0 &&
            pl.zm.stride[0] > 0 && siNumel(hy) >= tx.tadLength) {
            pl.tadEws = pl.xm.stride[0];
            pl.yEws = pl.ym.stride[0];
            pl.zEws = pl.zm.stride[0];
            stridedWalk = true;
        }
    }
    if (stridedWalk) {
        pl.kind = (pl.tadEws == 1 && pl.yEws == 1 && pl.zEws == 1) ? BroadcastPlan::ROW : BroadcastPlan::COL;
        // contiguous TADs of a dense array are its trailing (c order) or leading (f order) block, so they follow one
        // another without gaps;
        // when the result has the same dense layout the kernel needs no offset tables
        if (zTadInfo == tx.hostInfo && sameShape(hx, hz) && siNumel(hy) == tx.tadLength &&
            ((isDense(hx, 'c') && isDense(hz, 'c')) || (isDense(hx, 'f') && isDense(hz, 'f')))) {
            pl.consecutive = pl.kind == BroadcastPlan::ROW;
            // a single dimension of a dense array: its stride is the number of consecutive elements that share one y
            pl.denseAlike = pl.yEws == 1 && pl.zEws == pl.tadEws;
        }
    } else {
        pl.kind = BroadcastPlan::GENERAL;
        if (tx.tadLength > 0x7fffffffLL) throw std::invalid_argument("execBroadcast: a TAD without an element-wise stride holds 2^31 elements or more");
        // contiguous runs along the innermost dimension of all three walks: one 16-byte vector per thread.  Consecutive
        // runs of one TAD lie xm.stride[rank - 2] apart; when that leaves room for the same run of other TADs in between
        // (a dense array's TADs interleave), those are walked side by side.
        const DimMap *const maps[3] = {&pl.xm, &pl.ym, &pl.zm};
        const unsigned run = commonRunLength(maps);
        if (run >= 2 && siNumel(hy) >= tx.tadLength) {
            pl.runLength = run;
            const Long next = pl.xm.rank >= 2 && pl.xm.shape[pl.xm.rank - 1] == run ? pl.xm.stride[pl.xm.rank - 2] : (Long)run;
            pl.runMajor = tx.numTads > 1 && (next >= 2 * (Long)run || next < 0);
        }
    }
    // Contiguous TADs that the flat kernels do not take (gaps between them): their places follow from x's own
    // strides, so the call can be stated as one element-wise walk over x's shape in which y repeats along the dimensions
    // that are not the TAD's.  The reference pairs element f of every TAD, f counting in the TAD's order, with element f of
    // y; that is y[f * stride] here whenever y's own walk came out as one run (yLinear), and f counts in C order over the
    // TAD's dimensions when the TAD's order is 'c' (or it has one dimension).  The TAD's dimensions are found in x's by
    // extent and stride, in order (extents of 1 take no part); the result must be laid out over the same shape.
    const Long yLinear = pl.kind == BroadcastPlan::GENERAL ? (pl.ym.rank == 1 ? pl.ym.stride[0] : 0) : pl.yEws;
    if (!pl.consecutive && !pl.denseAlike && (pl.kind == BroadcastPlan::ROW || pl.kind == BroadcastPlan::GENERAL) && yLinear > 0 &&
        (siOrder(tx.hostInfo) == 'c' || dimLen == 1) && sameShape(hx, hz) && siNumel(hy) >= tx.tadLength &&
        siNumel(hx) <= 0x7fffffffLL && siRank(hx) <= kMaxDims) {
        const int rank = siRank(hx), tadRank = siRank(tx.hostInfo);
        // (without tables of its own the result is walked with x's, whatever its shapeInfo says: cpu/broadcasting.cpp:79-82;
        // with them, its TADs must be the ones its own strides give along the same dimensions)
        const bool ownTables = zOffsets != tx.devOffsets;
        const Long *xs = siShape(hx), *xst = siStride(hx), *zst = ownTables ? siStride(hz) : xst;
        const Long *ts = siShape(tx.hostInfo), *tst = siStride(tx.hostInfo);
        const Long *zts = siStride(zTadInfo);
        bool zNatural = siRank(zTadInfo) == tadRank;
        Long ystr[kMaxDims];
        bool inTad[kMaxDims];
        int k = 0;
        while (k < tadRank && ts[k] == 1) k++;
        for (int d = 0; d < rank; d++) {
            inTad[d] = xs[d] != 1 && k < tadRank && xs[d] == ts[k] && xst[d] == tst[k];
            if (inTad[d]) {
                if (zNatural && (siShape(zTadInfo)[k] != ts[k] || zts[k] != zst[d])) zNatural = false;
                k++;
                while (k < tadRank && ts[k] == 1) k++;
            }
        }
        if (k == tadRank && zNatural) {
            Long inner = yLinear;
            for (int d = rank - 1; d >= 0; d--) {
                ystr[d] = inTad[d] ? inner : 0;
                if (inTad[d]) inner *= xs[d];
            }
            const Long *strides[3] = {xst, ystr, zst};
            DimMap maps[3];
            jointCanon(rank, xs, strides, maps);
            const DimMap *const all[3] = {&maps[0], &maps[1], &maps[2]};
            const unsigned run = commonRunLength(all);
            if (run >= 2 && pl.kind == BroadcastPlan::ROW) {
                pl.wx = maps[0]; pl.wy = maps[1]; pl.wz = maps[2];
                pl.wholeN = siNumel(hx);
                pl.wholeRun = run;
            } else if (pl.kind == BroadcastPlan::GENERAL && maps[0].rank == 3) {
                // TADs over the outer and the inner part of a dense array ([A, B, C] along {0, 2}): x and z are plain vectors,
                // and position i takes y[(i / (B * C)) * C + i % C]
                const Long B = maps[0].shape[1], C = maps[0].shape[2];
                bool slab = yLinear == 1 && siNumel(hy) == tx.tadLength;
                for (int m = 0; m < 3 && slab; m += 2)
                    slab = maps[m].stride[0] == B * C && maps[m].stride[1] == C && maps[m].stride[2] == 1;
                if (slab && maps[1].stride[0] == C && maps[1].stride[1] == 0 && maps[1].stride[2] == 1) {
                    pl.slabInner = (unsigned)C;
                    pl.slabMid = (unsigned)B;
                }
            }
        }
    }
    if (!launchBroadcast<T>(s, opNum, x, y, z, pl)) { reportUnknownOp("broadcast", opNum); return; }
    checkLaunch("execBroadcast", s);
}

// ---- scalar family (include/loops/cpu/scalar.cpp) ---------------------------------------------------
template <typename T, typename S>
void scalarStrided(Nd4jPointer *extra, int opNum, T *x, Long xs, T *z, Long zs, S scalar, T *params, Long n) {
    hipStream_t s = streamOf(extra);
    if (!launchScalarStrided<T>(s, opNum, x, xs, z, zs, (typename Compute<T>::type)scalar, params, n)) {
        reportUnknownOp("scalar", opNum);
        return;
    }
    checkLaunch("execScalar(strided)", s);
}

template <typename T, typename S>
void scalarShaped(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *z, Long *zInfo, S scalar, T *params) {
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx, sz;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    const Long *hz = hostShapeInfo(extra, X_HOST_Z_SHAPE, zInfo, sz, s);
    if (hx == nullptr || hz == nullptr) return;
    Long n = siNumel(hx);
    Long xe = siEws(hx), ze = siEws(hz);
    const typename Compute<T>::type sv = (typename Compute<T>::type)scalar;
    bool ok;
    if (xe >= 1 && ze >= 1 && siOrder(hx) == siOrder(hz)) {
        // scalar.cpp:129-132, 187-191
        ok = launchScalarStrided<T>(s, opNum, x, xe, z, ze, sv, params, n);
    } else {
        // raw iteration over x's shape with both stride sets (scalar.cpp:135-181)
        const Long *strides[3] = {siStride(hx), nullptr, siStride(hz)};
        DimMap maps[3];
        jointCanon(siRank(hx), siShape(hx), strides, maps);
        ok = launchScalarGeneral<T>(s, opNum, x, maps[0], z, maps[2], sv, params, n);
    }
    if (!ok) { reportUnknownOp("scalar", opNum); return; }
    checkLaunch("execScalar", s);
}

// one scalar per TAD along `dimension` (scalar.cpp:14-62)
template <typename T>
void scalarAlongDimension(Nd4jPointer *extra, int opNum, T *x, Long *xInfo, T *z, Long *zInfo, T *scalars, T *params,
                          int *dimension, int dimLen) {
    (void)zInfo;
    hipStream_t s = streamOf(extra);
    std::vector<Long> sx;
    const Long *hx = hostShapeInfo(extra, X_HOST_X_SHAPE, xInfo, sx, s);
    if (hx == nullptr) return;
    ResolvedTad tx;
    if (!resolveTad(extra, X_HOST_TAD_SHAPE, X_DEV_TAD_OFFSETS, hx, dimension, dimLen, tx, s)) return;
    const Long *devZOff = reinterpret_cast<const Long *>(slotOf(extra, X_DEV_TAD_OFFSETS_Z));
    BroadcastPlan pl;
    pl.tadLength = tx.tadLength;
    pl.numTads = tx.numTads;
    pl.xOffsets = tx.devOffsets;
    pl.zOffsets = devZOff != nullptr ? devZOff : tx.devOffsets;
    pl.tadEws = siEws(tx.hostInfo);
    pl.yEws = 0;
    pl.zEws = pl.tadEws;  // the reference takes z's stride from the x TAD as well (scalar.cpp:22-23)
    if (pl.tadEws < 1) {
        // the only branch the reference has for such TADs (scalar.cpp:56-58)
        std::printf("Super-bad loop visited. Shouldn't ever happen\n");
        return;
    }
    pl.kind = pl.tadEws == 1 ? BroadcastPlan::ROW : BroadcastPlan::COL;
    // Dense x, z laid out like it, and TADs whose numbering follows memory order: the arrays can be walked as plain
    // vectors, the TAD index falling out of the position (rows of a c-order array: i / tadLength; its columns, or whatever
    // lies along its leading dimension: i % numTads).  For f-order arrays that holds in two dimensions only (the
    // reference numbers TADs in C order over the remaining dimensions).
    const Long *hz = reinterpret_cast<const Long *>(slotOf(extra, X_HOST_Z_SHAPE));
    const bool zLikeX = devZOff == nullptr || (hz != nullptr && siRank(hz) == siRank(hx) &&
                                               std::memcmp(hx, hz, sizeof(Long) * siLength(siRank(hx))) == 0);
    const bool numbered = isDense(hx, 'c') || (siRank(hx) <= 2 && isDense(hx, 'f'));
    if (zLikeX && numbered && tx.numTads * tx.tadLength == siNumel(hx)) {
        if (pl.kind == BroadcastPlan::ROW) { pl.flatInner = pl.tadLength; pl.flatExtent = pl.numTads; }
        else if (pl.tadEws == pl.numTads) { pl.flatInner = 1; pl.flatExtent = pl.numTads; }
    }
    if (!launchScalarTad<T>(s, opNum, x, scalars, z, params, pl)) { reportUnknownOp("scalar", opNum); return; }
    checkLaunch("execScalar(dimension)", s);
}

}  // namespace

// ---- per-type members ---------------------------------------------------------------------------------
#define ND4J_SCALAR_MEMBERS(SUFFIX, T, S)                                                                        \
    void NativeOps::execScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong xStride, T *result, \
                                       Nd4jLong resultStride, S scalar, T *extraParams, Nd4jLong n) {            \
        scalarStrided<T, S>(extraPointers, opNum, x, xStride, result, resultStride, scalar, extraParams, n);     \
    }                                                                                                            \
    void NativeOps::execScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,        \
                                       T *result, Nd4jLong *resultShapeInfo, S scalar, T *extraParams) {         \
        scalarShaped<T, S>(extraPointers, opNum, x, xShapeInfo, result, resultShapeInfo, scalar, extraParams);   \
    }                                                                                                            \
    void NativeOps::execScalar##SUFFIX(Nd4jPointer *, int, T *, Nd4jLong *, T *, Nd4jLong *, S, T *, Nd4jLong *, \
                                       Nd4jLong *) {                                                             \
        /* indexed variant: launches nothing in the reference's CUDA back end (blas/cuda/NativeOps.cu:2788-2816) */ \
    }                                                                                                            \
    void NativeOps::execScalar##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo, T *z,  \
                                       Nd4jLong *zShapeInfo, T *scalars, T *extraParams, int *dimension,         \
                                       int dimensionLength) {                                                    \
        scalarAlongDimension<T>(extraPointers, opNum, x, xShapeInfo, z, zShapeInfo, scalars, extraParams,        \
                                dimension, dimensionLength);                                                     \
    }
ND4J_SCALAR_MEMBERS(Float, float, float)
ND4J_SCALAR_MEMBERS(Half, float16, float)
ND4J_SCALAR_MEMBERS(Double, double, double)
#undef ND4J_SCALAR_MEMBERS
// the reference's indexed Double variant carries an extra element count (blas/NativeOps.h:419-430); like the others
// it launches nothing
void NativeOps::execScalarDouble(Nd4jPointer *, int, double *, Nd4jLong *, double *, Nd4jLong *, double, double *, Nd4jLong,
                                 Nd4jLong *, Nd4jLong *) {}

#define ND4J_ELEMENTWISE_MEMBERS(SUFFIX, T)                                                                      \
    void NativeOps::execTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong xStride,        \
                                          T *result, Nd4jLong resultStride, T *extraParams, Nd4jLong n) {        \
        transformStrided<T>(extraPointers, opNum, dx, xStride, result, resultStride, extraParams, n);            \
    }                                                                                                            \
    void NativeOps::execTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx, Nd4jLong *xShapeInfo,    \
                                          T *result, Nd4jLong *resultShapeInfo, T *extraParams) {                \
        transformShaped<T>(extraPointers, opNum, dx, xShapeInfo, result, resultShapeInfo, extraParams);          \
    }                                                                                                            \
    void NativeOps::execTransform##SUFFIX(Nd4jPointer *, int, T *, Nd4jLong *, T *, Nd4jLong *, T *, Nd4jLong *, \
                                          Nd4jLong *) {                                                          \
        /* indexed variant: empty in the reference too (blas/cuda/NativeOps.cu:3598-3612) */                     \
    }                                                                                                            \
    void NativeOps::execPairwiseTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx,                  \
                                                  Nd4jLong xStride, T *y, Nd4jLong yStride, T *result,           \
                                                  Nd4jLong resultStride, T *extraParams, Nd4jLong n) {           \
        pairwiseStrided<T>(extraPointers, opNum, dx, xStride, y, yStride, result, resultStride, extraParams, n); \
    }                                                                                                            \
    void NativeOps::execPairwiseTransform##SUFFIX(Nd4jPointer *, int, T *, Nd4jLong *, T *, Nd4jLong *, T *,     \
                                                  Nd4jLong *, T *, Nd4jLong *, Nd4jLong *, Nd4jLong *) {         \
        /* indexed variant: empty in the reference's CUDA back end (blas/cuda/NativeOps.cu:1928-1960) */         \
    }                                                                                                            \
    void NativeOps::execPairwiseTransform##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *dx,                  \
                                                  Nd4jLong *xShapeInfo, T *y, Nd4jLong *yShapeInfo, T *result,   \
                                                  Nd4jLong *resultShapeInfo, T *extraParams) {                   \
        pairwiseShaped<T>(extraPointers, opNum, dx, xShapeInfo, y, yShapeInfo, result, resultShapeInfo,          \
                          extraParams);                                                                          \
    }                                                                                                            \
    void NativeOps::execBroadcast##SUFFIX(Nd4jPointer *extraPointers, int opNum, T *x, Nd4jLong *xShapeInfo,     \
                                          T *y, Nd4jLong *yShapeInfo, T *result, Nd4jLong *resultShapeInfo,      \
                                          int *dimension, int dimensionLength) {                                 \
        broadcastShaped<T>(extraPointers, opNum, x, xShapeInfo, y, yShapeInfo, result, resultShapeInfo,          \
                           dimension, dimensionLength);                                                          \
    }

ND4J_ELEMENTWISE_MEMBERS(Float, float)
ND4J_ELEMENTWISE_MEMBERS(Half, float16)
ND4J_ELEMENTWISE_MEMBERS(Double, double)

// ---- shape service -------------------------------------------------------------------------------------
void NativeOps::tadOnlyShapeInfo(Nd4jLong *xShapeInfo, int *dimension, int dimensionLength, Nd4jLong *targetBuffer,
                                 Nd4jLong *offsetsBuffer) {
    TadPack pack;
    computeTad(xShapeInfo, dimension, dimensionLength, pack, offsetsBuffer != nullptr);
    std::memcpy(targetBuffer, pack.shapeInfo.data(), pack.shapeInfo.size() * sizeof(Long));
    if (offsetsBuffer != nullptr) std::memcpy(offsetsBuffer, pack.offsets.data(), pack.offsets.size() * sizeof(Long));
}

// ---- lifecycle (reference: blas/cuda/NativeOps.cu:3946-4390) ---------------------------------------------
static int deviceIdOf(Nd4jPointer p) { return (int)(intptr_t)p; }

void NativeOps::initializeDevicesAndFunctions() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return; }
    // the address of the no-allocation entry point's scratch array on the current device (other devices: looked up
    // by the first call that runs on them)
    if (n > 0) {
        try { prepareNoAllocScratch(); } catch (const std::exception &) { (void)hipGetLastError(); }
    }
}

Nd4jPointer NativeOps::mallocHost(Nd4jLong memorySize, int) {
    void *p = nullptr;
    if (hipHostMalloc(&p, (size_t)memorySize, hipHostMallocDefault) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    return p;
}
Nd4jPointer NativeOps::mallocDevice(Nd4jLong memorySize, Nd4jPointer, int) {
    void *p = nullptr;
    if (hipMalloc(&p, (size_t)memorySize) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    return p;
}
int NativeOps::freeHost(Nd4jPointer pointer) { return hipHostFree(pointer) == hipSuccess ? 1 : 0; }
int NativeOps::freeDevice(Nd4jPointer pointer, Nd4jPointer) { return hipFree(pointer) == hipSuccess ? 1 : 0; }

int NativeOps::ompGetMaxThreads() { return environment().maxThreads.load(); }
int NativeOps::ompGetNumThreads() { return environment().maxThreads.load(); }
void NativeOps::setOmpNumThreads(int threads) {
    // on the GPU back end this is the maximum block size, clamped to 32..1024 (blas/cuda/NativeOps.cu:4380-4390)
    if (threads < 32) threads = 32;
    if (threads > 1024) threads = 1024;
    environment().maxThreads.store(threads);
}
void NativeOps::setOmpMinThreads(int) {}
Nd4jPointer NativeOps::createContext() { return nullptr; }
Nd4jPointer NativeOps::createStream() {
    hipStream_t s = nullptr;
    if (hipStreamCreate(&s) != hipSuccess) throw std::runtime_error("createStream failed");
    return reinterpret_cast<Nd4jPointer>(s);  // the handle itself (blas/cuda/NativeOps.cu:4166-4177)
}
Nd4jPointer NativeOps::createEvent() {
    hipEvent_t e = nullptr;
    if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) throw std::runtime_error("createEvent failed");
    return reinterpret_cast<Nd4jPointer>(e);
}
int NativeOps::registerEvent(Nd4jPointer event, Nd4jPointer stream) {
    if (hipEventRecord(reinterpret_cast<hipEvent_t>(event), reinterpret_cast<hipStream_t>(stream)) != hipSuccess)
        throw std::runtime_error("registerEvent failed");
    return 1;
}
int NativeOps::destroyEvent(Nd4jPointer event) {
    if (hipEventDestroy(reinterpret_cast<hipEvent_t>(event)) != hipSuccess) throw std::runtime_error("destroyEvent failed");
    return 1;
}
int NativeOps::setDevice(Nd4jPointer ptrToDeviceId) {
    if (hipSetDevice(deviceIdOf(ptrToDeviceId)) != hipSuccess) throw std::runtime_error("setDevice failed");
    return 1;
}
int NativeOps::getDevice() {
    int d = 0;
    (void)hipGetDevice(&d);
    return d;
}
int NativeOps::streamSynchronize(Nd4jPointer stream) {
    if (hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream)) != hipSuccess)
        throw std::runtime_error("streamSynchronize failed");
    return 1;
}
int NativeOps::eventSynchronize(Nd4jPointer event) {
    if (hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)) != hipSuccess)
        throw std::runtime_error("eventSynchronize failed");
    return 1;
}
Nd4jLong NativeOps::getDeviceFreeMemory(Nd4jPointer ptrToDeviceId) {
    int prev = getDevice(), want = deviceIdOf(ptrToDeviceId);
    if (want >= 0 && want != prev) (void)hipSetDevice(want);
    size_t f = 0, t = 0;
    (void)hipMemGetInfo(&f, &t);
    if (want >= 0 && want != prev) (void)hipSetDevice(prev);
    return (Nd4jLong)f;
}
Nd4jLong NativeOps::getDeviceTotalMemory(Nd4jPointer ptrToDeviceId) {
    int prev = getDevice(), want = deviceIdOf(ptrToDeviceId);
    if (want >= 0 && want != prev) (void)hipSetDevice(want);
    size_t f = 0, t = 0;
    (void)hipMemGetInfo(&f, &t);
    if (want >= 0 && want != prev) (void)hipSetDevice(prev);
    return (Nd4jLong)t;
}
static int attributeOf(Nd4jPointer ptrToDeviceId, hipDeviceAttribute_t attr) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, attr, deviceIdOf(ptrToDeviceId)) != hipSuccess) { (void)hipGetLastError(); return 0; }
    return v;
}
int NativeOps::getDeviceMajor(Nd4jPointer ptrToDeviceId) { return attributeOf(ptrToDeviceId, hipDeviceAttributeComputeCapabilityMajor); }
int NativeOps::getDeviceMinor(Nd4jPointer ptrToDeviceId) { return attributeOf(ptrToDeviceId, hipDeviceAttributeComputeCapabilityMinor); }
const char *NativeOps::getDeviceName(Nd4jPointer ptrToDeviceId) {
    static char names[64][256];
    int dev = deviceIdOf(ptrToDeviceId);
    if (dev < 0 || dev >= 64) dev = 0;
    if (names[dev][0] == 0 && hipDeviceGetName(names[dev], 255, dev) != hipSuccess) { (void)hipGetLastError(); names[dev][0] = 0; }
    return names[dev];
}

static hipMemcpyKind kindOf(int flags) {
    switch (flags) {
        case 0: return hipMemcpyHostToHost;
        case 1: return hipMemcpyHostToDevice;
        case 2: return hipMemcpyDeviceToHost;
        case 3: return hipMemcpyDeviceToDevice;
        default: return hipMemcpyDefault;
    }
}
int NativeOps::memcpy(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer) {
    return hipMemcpy(dst, src, (size_t)size, kindOf(flags)) == hipSuccess ? 1 : 0;
}
int NativeOps::memcpyAsync(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved) {
    return hipMemcpyAsync(dst, src, (size_t)size, kindOf(flags), reinterpret_cast<hipStream_t>(reserved)) == hipSuccess ? 1 : 0;
}
int NativeOps::memset(Nd4jPointer dst, int value, Nd4jLong size, int, Nd4jPointer) {
    return hipMemset(dst, value, (size_t)size) == hipSuccess ? 1 : 0;
}
int NativeOps::memsetAsync(Nd4jPointer dst, int value, Nd4jLong size, int, Nd4jPointer reserved) {
    return hipMemsetAsync(dst, value, (size_t)size, reinterpret_cast<hipStream_t>(reserved)) == hipSuccess ? 1 : 0;
}

// The reference keeps a 48 KiB __constant__ arena that ND4J fills with shapeInfo buffers
// (blas/cuda/NativeOps.cu:87, 4793-4835).  Plain device memory serves the same purpose here.
static void *constantSpace() {
    static void *space = nullptr;
    if (space == nullptr && hipMalloc(&space, 49152) != hipSuccess) { (void)hipGetLastError(); space = nullptr; }
    return space;
}
int NativeOps::memcpyConstantAsync(Nd4jLong dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved) {
    char *base = reinterpret_cast<char *>(constantSpace());
    if (base == nullptr || dst < 0 || dst + size > 49152) return 0;
    hipMemcpyKind k = flags == 3 ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice;
    return hipMemcpyAsync(base + dst, src, (size_t)size, k, reinterpret_cast<hipStream_t>(reserved)) == hipSuccess ? 1 : 0;
}
Nd4jPointer NativeOps::getConstantSpace() { return constantSpace(); }
int NativeOps::getAvailableDevices() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; }
    return n;
}
void NativeOps::enableDebugMode(bool reallyEnable) { environment().debug.store(reallyEnable); }
void NativeOps::enableVerboseMode(bool reallyEnable) { environment().verbose.store(reallyEnable); }
void NativeOps::setGridLimit(int gridSize) {
    if (gridSize > 8192) gridSize = 8192;
    if (gridSize < 1) gridSize = 1;
    environment().gridLimit.store(gridSize);
}
void NativeOps::setElementThreshold(int num) { if (num > 0) environment().elementThreshold.store(num); }
void NativeOps::setTADThreshold(int num) { if (num > 0) environment().tadThreshold.store(num); }
