// NativeOps boundary, part 5: the whole-array transforms with a routine of their own that travel through
// execTransform*(shapeInfo form) - Col2Im 36, Im2col 37, Histogram 48, Reverse 70, Pooling2D 71.  Branch selection
// follows the reference's CPU routines, which are the parity oracle (include/ops/special_ops.h: Pooling2D 227-359,
// Im2col 530-663, Histogram 811-882, Col2Im 997-1129, Reverse 1317-1414); extraParams stays on the device and is
// read by the kernels, as in the reference's CUDA back end.
#include <stdexcept>
#include <string>

#include "runtime.h"

namespace nd4j_amd {

namespace {

// offsets of the elements of one array walked by its own linear index, in its own order
void ownOrderMap(const Long *info, DimMap &out) {
    const int rank = siRank(info);
    if (siOrder(info) != 'f') {
        ownCanon(rank, siShape(info), siStride(info), out);
        return;
    }
    Long rs[kMaxRank], rt[kMaxRank];
    for (int i = 0; i < rank; i++) { rs[i] = siShape(info)[rank - 1 - i]; rt[i] = siStride(info)[rank - 1 - i]; }
    ownCanon(rank, rs, rt, out);
}

void stridedMap(Long n, Long stride, DimMap &out) {
    out.rank = 1;
    out.shape[0] = (unsigned)(n > 0xffffffffLL ? 0xffffffffu : n);
    out.stride[0] = stride;
}

// shape::strideDescendingCAscendingF (include/helpers/shape.h)
bool stridesDescend(const Long *info) {
    const int rank = siRank(info);
    const Long *st = siStride(info);
    for (int i = 1; i < rank; i++) {
        if (siOrder(info) == 'c' ? st[i - 1] <= st[i] : st[i - 1] >= st[i]) return false;
    }
    return true;
}

void requireRank(const Long *info, int rank, const char *op, const char *which) {
    if (siRank(info) != rank)
        throw std::invalid_argument(std::string(op) + ": " + which + " must have rank " + std::to_string(rank));
}

void requireSmall(Long elements, const char *op) {
    if (elements >= 0x7fffffffLL) throw std::invalid_argument(std::string(op) + ": more than 2^31 - 1 elements");
}

// the largest offset any element of the view has, plus one
Long spanOf(const Long *info) {
    Long span = 1;
    for (int d = 0; d < siRank(info); d++) {
        if (siShape(info)[d] > 0) span += (siShape(info)[d] - 1) * (siStride(info)[d] < 0 ? -siStride(info)[d] : siStride(info)[d]);
    }
    return span;
}

template <typename T> void reverseWhole(const T *x, const Long *hx, T *z, const Long *hz, hipStream_t s) {
    ReversePlan p;
    p.n = siNumel(hx);
    if (p.n <= 0) return;
    const Long xe = siEws(hx);
    if (x == z) {
        if (xe >= 1) {
            p.swap = true;
            p.contiguous = xe == 1;
            p.count = p.n / 2;
            stridedMap(p.n, xe, p.xm);
            p.zm = p.xm;
        } else {
            // without an element-wise stride the reference only copies the first half onto the mirrored positions
            p.count = p.n / 2;
            ownOrderMap(hx, p.xm);
            p.zm = p.xm;
        }
    } else {
        const Long ze = siEws(hz);
        p.count = p.n;
        if (xe >= 1 && ze >= 1 && siOrder(hx) == siOrder(hz)) {
            p.contiguous = xe == 1 && ze == 1;
            stridedMap(p.n, xe, p.xm);
            stridedMap(p.n, ze, p.zm);
        } else {
            ownOrderMap(hx, p.xm);
            ownOrderMap(hz, p.zm);
        }
    }
    launchReverse<T>(s, x, z, p);
}

template <typename T> void histogramWhole(const T *x, const Long *hx, T *z, const Long *hz, const T *params, hipStream_t s) {
    if (params == nullptr) throw std::invalid_argument("Histogram: extraParams [numBins, min, max] required");
    // the reference reads the first length(x) elements of the buffer (an int count) and writes the first numBins of z
    const Long n = siNumel(hx);
    requireSmall(n, "Histogram");
    const Long capacity = siNumel(hz);
    requireSmall(capacity, "Histogram");
    if (capacity <= 0) return;
    Workspace w = workspaceFor(s, histogramScratchBytes(n, (int)sizeof(T), (int)capacity));
    launchHistogram<T>(s, x, n, z, (int)capacity, params, reinterpret_cast<unsigned *>(w.ptr));
}

void fillImage(ConvGeometry &g, const Long *img) {
    g.bS = (int)siShape(img)[0];
    g.iC = (int)siShape(img)[1];
    g.iH = (int)siShape(img)[2];
    g.iW = (int)siShape(img)[3];
    for (int d = 0; d < 4; d++) g.imS[d] = siStride(img)[d];
    g.dIC = FastDiv((unsigned)g.iC);
    g.dIH = FastDiv((unsigned)g.iH);
    g.dIW = FastDiv((unsigned)g.iW);
}

// col: [bS, iC, kH, kW, oH, oW].  When both arrays are c-order with descending strides the reference walks a batch
// entry of the column array as one run whose step is the last stride (1 for the result of Im2col, which it writes
// through a plain pointer), whatever the strides in between say.
void fillColumns(ConvGeometry &g, const Long *col, bool asOneRun, bool unitStep) {
    g.kH = (int)siShape(col)[2];
    g.kW = (int)siShape(col)[3];
    g.oH = (int)siShape(col)[4];
    g.oW = (int)siShape(col)[5];
    for (int d = 0; d < 6; d++) g.colS[d] = siStride(col)[d];
    if (asOneRun) {
        if (unitStep) g.colS[5] = 1;
        g.colS[4] = g.oW * g.colS[5];
        g.colS[3] = g.oH * g.colS[4];
        g.colS[2] = g.kW * g.colS[3];
        g.colS[1] = g.kH * g.colS[2];
    }
    g.dOW = FastDiv((unsigned)g.oW);
    g.dOH = FastDiv((unsigned)g.oH);
    g.dKW = FastDiv((unsigned)g.kW);
    g.dKH = FastDiv((unsigned)g.kH);
}

template <typename T> void im2colWhole(const T *x, const Long *hx, T *z, const Long *hz, const T *params, hipStream_t s) {
    if (params == nullptr) throw std::invalid_argument("Im2col: extraParams required");
    requireRank(hx, 4, "Im2col", "x");
    requireRank(hz, 6, "Im2col", "z");
    requireSmall(spanOf(hx), "Im2col");
    requireSmall(spanOf(hz), "Im2col");
    requireSmall(siNumel(hz), "Im2col");
    ConvGeometry g;
    fillImage(g, hx);
    const bool oneRun = siOrder(hx) == 'c' && siOrder(hz) == 'c' && stridesDescend(hx) && stridesDescend(hz);
    fillColumns(g, hz, oneRun, true);
    launchIm2col<T>(s, x, z, params, g);
}

template <typename T> void col2imWhole(const T *x, const Long *hx, T *z, const Long *hz, const T *params, hipStream_t s) {
    if (params == nullptr) throw std::invalid_argument("Col2Im: extraParams required");
    requireRank(hx, 6, "Col2Im", "x");
    requireRank(hz, 4, "Col2Im", "z");
    requireSmall(spanOf(hx), "Col2Im");
    requireSmall(spanOf(hz), "Col2Im");
    ConvGeometry g;
    fillImage(g, hz);
    // batch and channel counts are read from the column array (special_ops.h:1006, 1011-1012)
    g.bS = (int)siShape(hx)[0];
    g.iC = (int)siShape(hx)[1];
    g.dIC = FastDiv((unsigned)g.iC);
    const bool oneRun = siOrder(hx) == 'c' && siOrder(hz) == 'c' && stridesDescend(hx) && stridesDescend(hz);
    fillColumns(g, hx, oneRun, false);
    // The reference clears length(z) leading elements of z's buffer and adds onto whatever lies beyond.  When every
    // element of the view sits inside that stretch (a dense result) the sums simply start from zero.
    const Long zn = siNumel(hz);
    const bool inside = spanOf(hz) <= zn;
    launchCol2im<T>(s, x, z, params, g, inside ? 0 : zn);
}

template <typename T> void pooling2dWhole(const T *x, const Long *hx, T *z, const Long *hz, const T *params, hipStream_t s) {
    if (params == nullptr) throw std::invalid_argument("Pooling2D: extraParams required");
    requireRank(hx, 4, "Pooling2D", "x");
    requireRank(hz, 4, "Pooling2D", "z");
    requireSmall(spanOf(hx), "Pooling2D");
    requireSmall(spanOf(hz), "Pooling2D");
    ConvGeometry g;
    fillImage(g, hx);
    g.kH = g.kW = 0;  // read from extraParams by the kernel
    g.oH = (int)siShape(hz)[2];
    g.oW = (int)siShape(hz)[3];
    for (int d = 0; d < 4; d++) g.colS[d] = siStride(hz)[d];
    g.colS[4] = g.colS[5] = 0;
    if (siOrder(hz) != 'f') {
        // a c-order result is written densely behind each (batch, channel) start (special_ops.h:350-351)
        g.colS[3] = 1;
        g.colS[2] = g.oW;
    }
    g.dOW = FastDiv((unsigned)g.oW);
    g.dOH = FastDiv((unsigned)g.oH);
    launchPooling2d<T>(s, x, z, params, g);
}

}  // namespace

template <typename T>
bool wholeArrayTransform(int opNum, T *x, const Long *hx, T *z, const Long *hz, T *params, hipStream_t s) {
    switch (opNum) {
        case 36: col2imWhole<T>(x, hx, z, hz, params, s); return true;
        case 37: im2colWhole<T>(x, hx, z, hz, params, s); return true;
        case 48: histogramWhole<T>(x, hx, z, hz, params, s); return true;
        case 70: reverseWhole<T>(x, hx, z, hz, s); return true;
        case 71: pooling2dWhole<T>(x, hx, z, hz, params, s); return true;
        default: return false;
    }
}

#define INST(T) template bool wholeArrayTransform<T>(int, T *, const Long *, T *, const Long *, T *, hipStream_t);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
