// Host-side shapeInfo / TAD (tensor-along-dimension) logic.
//
// A shapeInfo buffer is [rank, shape[rank], stride[rank], offset, elementWiseStride, order], 2*rank+4
// 64-bit integers (reference: include/helpers/shape.h:2558-2683).  Everything here runs on the host:
// kernels never parse shapeInfo buffers, they receive small by-value descriptors built from them.
//
// The TAD part restates shape::TAD (reference: include/helpers/TAD.h:325-352 init, 577-611 tadOffset,
// 714-721 createOffsets, 723-895 shapeInfoOnlyShapeAndStride) for tadIndex 0, including the reference's
// conventions that callers can observe: a 1-dimensional TAD of a matrix is reported as [1, L] with
// strides [1, s], permuted buffers get elementWiseStride -1, and the order character is recomputed by
// the contiguity test of shape::getOrder (shape.h:2195-2241).
#pragma once

#include <cstdint>
#include <cstring>
#include <vector>

namespace nd4j_amd {

typedef long long Long;
static const int kMaxRank = 32;
static const int kMaxDimension = 0x7fffffff;

inline int siRank(const Long *si) { return (int)si[0]; }
inline const Long *siShape(const Long *si) { return si + 1; }
inline const Long *siStride(const Long *si) { return si + 1 + siRank(si); }
inline int siLength(int rank) { return 2 * rank + 4; }
inline Long siOffset(const Long *si) { return si[2 * siRank(si) + 1]; }
inline Long siEws(const Long *si) { return si[2 * siRank(si) + 2]; }
inline char siOrder(const Long *si) { return (char)si[2 * siRank(si) + 3]; }

inline Long prodOf(const Long *v, int n) {
    Long p = 1;
    for (int i = 0; i < n; i++) p *= v[i];
    return p;
}

// shape::length (shape.h:2628-2637)
inline Long siNumel(const Long *si) {
    int r = siRank(si);
    if (r == 0) return 1;
    if (r == 1) return si[1];
    return prodOf(siShape(si), r);
}

// shape::isVector (shape.h:2310-2324): rank 1, or rank 2 with a unit dimension.
inline bool shapeIsVector(const Long *shape, int rank) {
    if (rank == 0) return false;
    if (rank == 1) return true;
    if (rank > 2) return false;
    return shape[0] == 1 || shape[1] == 1;
}
inline bool siIsVector(const Long *si) { return shapeIsVector(siShape(si), siRank(si)); }

// shape::isMatrix (shape.h:2389-2398).  Note: no rank guard below 2 in the reference either; callers
// only reach it with rank >= 2 here.
inline bool siIsMatrix(const Long *si) {
    int r = siRank(si);
    if (r > 2) return false;
    if (r < 2) return !(siShape(si)[0] == 1);
    return !(siShape(si)[0] == 1 || siShape(si)[1] == 1);
}

// shape::isScalar (shape.h:2765-2779)
inline bool siIsScalar(const Long *si) {
    int r = siRank(si);
    if (r > 2) return false;
    if (r == 0) return true;
    if (r == 1) return siShape(si)[0] == 1;
    return siShape(si)[0] == 1 && siShape(si)[1] == 1;
}
inline bool siIsRowVector(const Long *si) { return siIsVector(si) && siShape(si)[0] == 1; }

// shape::getOrder (shape.h:2195-2241): contiguity test deciding the order character.
inline char orderOf(int rank, const Long *shape, const Long *stride, int elementStride) {
    bool cContig = true, fContig = true;
    int sd = 1;
    for (int i = rank - 1; i >= 0; --i) {
        int dim = (int)shape[i];
        if (stride[i] != sd) { cContig = false; break; }
        if (dim == 0) break;
        sd *= dim;
    }
    sd = elementStride;
    for (int i = 0; i < rank; ++i) {
        int dim = (int)shape[i];
        if (stride[i] != sd) fContig = false;
        if (dim == 0) break;
        sd *= dim;
    }
    if (fContig && cContig) return 'a';
    if (fContig) return 'f';
    return 'c';
}

// shape::computeElementWiseStride (shape.h:1461-1608): the stride with which the whole array can be
// walked as [1, length] in C order (isFOrder == 0), or -1 when dimensions cannot be merged.
inline int computeEws(int rank, const Long *shape, const Long *stride, int isFOrder) {
    if (rank == 0) return 1;
    if (shapeIsVector(shape, rank)) return (int)stride[rank - 1];
    Long dims[kMaxRank], strs[kMaxRank];
    int nd = 0;
    for (int i = 0; i < rank; i++)
        if (shape[i] != 1) { dims[nd] = shape[i]; strs[nd] = stride[i]; nd++; }
    // The reference compares the products as 32-bit ints (np, op are int).
    int np = (int)prodOf(shape, rank);
    int op = 1;
    for (int i = 0; i < nd; i++) op *= (int)dims[i];
    if (np != op || np == 0) return -1;
    if (nd == 0) {
        // all dimensions are 1 (rank > 2, otherwise isVector): no old axis is consumed, the new strides
        // are filled from stride[rank-1] (times newShape[0] == 1 in f mode)
        return (int)stride[rank - 1];
    }
    for (int k = 0; k < nd - 1; k++) {
        if (isFOrder) {
            if (strs[k + 1] != dims[k] * strs[k]) return -1;
        } else {
            if (strs[k] != dims[k + 1] * strs[k + 1]) return -1;
        }
    }
    if (isFOrder) {
        // new shape is [1, len]: newStrides = {s0, s0}; the trailing fix-up multiplies by newShape[1]
        int last = (int)strs[0];
        last *= np;
        return last;
    }
    return (int)strs[nd - 1];
}

// shape::shapeBuffer / shapeBufferFortran (shape.h:1617-1710): EWS is always computed in C mode.
inline void makeShapeInfo(int rank, const Long *shape, char order, Long *out) {
    out[0] = rank;
    Long *shp = out + 1, *str = out + 1 + rank;
    for (int i = 0; i < rank; i++) shp[i] = shape[i];
    if (order == 'f') {
        Long st = 1;
        for (int i = 0; i < rank; i++) { str[i] = st; st *= shape[i]; }
    } else {
        Long st = 1;
        for (int i = rank - 1; i >= 0; i--) { str[i] = st; st *= shape[i]; }
    }
    // shape::calcStrides* give stride 1 (the start number) to unit dimensions of vectors; for the dense
    // buffers produced here the plain running product is what both variants yield except for that case.
    if (shapeIsVector(shape, rank)) {
        // calcStrides (shape.h:1322-1377) / calcStridesFortran (1270-1320): a [1,n] or [n,1] vector gets
        // strides {1,1}.
        for (int i = 0; i < rank; i++) str[i] = 1;
    }
    out[2 * rank + 1] = 0;
    out[2 * rank + 2] = computeEws(rank, shp, str, 0);
    out[2 * rank + 3] = order;
}

namespace detail {

typedef std::vector<Long> Buf;

inline Buf scalarInfoRank1() { return Buf{1, 1, 1, 0, 1, 99}; }

// shape::doPermuteSwap (shape.h:1960-2004): identity when already in order or when the product is < 2;
// for length 2 the two entries are swapped whatever the rearrangement says.
inline void permuteSwap(int n, Long *v, const int *rearrange) {
    if (n == 1) return;
    if (prodOf(v, n) < 2) return;
    bool inOrder = true;
    for (int i = 0; i < n - 1; i++) inOrder = inOrder && (rearrange[i] + 1 == rearrange[i + 1]);
    if (inOrder) return;
    if (n == 2) { Long t = v[0]; v[0] = v[1]; v[1] = t; return; }
    Long tmp[kMaxRank];
    for (int i = 0; i < n; i++) tmp[i] = v[i];
    for (int i = 0; i < n; i++) v[i] = tmp[rearrange[i]];
}

// shape::doPermuteShapeBuffer(Nd4jLong*, int*) (shape.h:2100-2118), used by permuteShapeBuffer.
inline void permuteInfo(Buf &b, const int *rearrange) {
    if (siIsScalar(b.data())) return;
    int r = siRank(b.data());
    Long *shp = b.data() + 1, *str = b.data() + 1 + r;
    permuteSwap(r, shp, rearrange);
    permuteSwap(r, str, rearrange);
    b[2 * r + 2] = -1;
    b[2 * r + 3] = orderOf(r, shp, str, 1);
}

// shape::doPermuteShapeBuffer(int rank, buffer, rearrange, tmp) (shape.h:2154-2168), used by
// permuteShapeBufferInPlace: same as above without the scalar early-out.
inline void permuteInfoInPlace(Buf &b, const int *rearrange) {
    int r = siRank(b.data());
    Long *shp = b.data() + 1, *str = b.data() + 1 + r;
    permuteSwap(r, shp, rearrange);
    permuteSwap(r, str, rearrange);
    b[2 * r + 2] = -1;
    b[2 * r + 3] = orderOf(r, shp, str, 1);
}

// shape::sliceOfShapeBuffer (shape.h:2483-2548) for slice index 0.
inline Buf sliceZero(const Buf &b) {
    const Long *si = b.data();
    int rank = siRank(si);
    int newRank = rank - 1 < 2 ? 2 : rank - 1;
    const Long *shp = siShape(si), *str = siStride(si);
    if (siIsVector(si)) {
        if (shp[0] == 1) return b;  // row vector: slice 0 is the vector itself
        Buf s = scalarInfoRank1();
        // the reference stores offset+sliceIdx at index shapeInfoLength(2)-3 == 5 of this rank-1 buffer,
        // which is its order slot
        s[5] = siOffset(si) + 0;
        return s;
    }
    Buf out(siLength(newRank));
    out[0] = newRank;
    Long *nshp = out.data() + 1, *nstr = out.data() + 1 + newRank;
    bool matrix = siIsMatrix(si);
    if (matrix) {
        nshp[0] = 1; nshp[1] = shp[1];
        nstr[0] = 1; nstr[1] = str[1];
    } else {
        for (int i = 0; i < newRank; i++) { nshp[i] = shp[i + 1]; nstr[i] = str[i + 1]; }
    }
    out[2 * newRank + 1] = 0;  // getOffset with all-zero indices
    out[2 * newRank + 2] = matrix ? str[1] : siEws(si);
    out[2 * newRank + 3] = orderOf(newRank, nshp, nstr, 1);
    return out;
}

inline void reversePermuteInPlace(Buf &b) {
    int r = siRank(b.data());
    int rev[kMaxRank];
    for (int i = 0; i < r; i++) rev[i] = r - 1 - i;
    permuteInfoInPlace(b, rev);
}
inline void reversePermuteCopy(Buf &b) {
    int r = siRank(b.data());
    int rev[kMaxRank];
    for (int i = 0; i < r; i++) rev[i] = r - 1 - i;
    permuteInfo(b, rev);
}

}  // namespace detail

// Result of a TAD decomposition of `x` along `dimension[0..dimLen)`.
struct TadPack {
    std::vector<Long> shapeInfo;  // TAD-only shapeInfo
    std::vector<Long> offsets;    // one element offset per TAD
    Long numTads = 0;
    bool wholeThing = false;
};

// shape::TAD::tadLength semantics as used by init (TAD.h:898-913).
inline Long tadLengthOf(const Long *xsi, const int *dim, int dimLen) {
    if (dimLen == 1) return siShape(xsi)[dim[0]];
    Long ret = 1;
    for (int i = 0; i < siRank(xsi); i++)
        for (int j = 0; j < dimLen; j++)
            if (i == dim[j]) ret *= siShape(xsi)[dim[j]];
    return ret;
}

inline void buildTadShapeInfo(const Long *xsi, const int *dim, int dimLen, Long numTads, bool wholeThing,
                              std::vector<Long> &outInfo) {
    using namespace detail;
    int rank = siRank(xsi);
    const Long *shp = siShape(xsi);
    Buf x(xsi, xsi + siLength(rank));

    if ((wholeThing && (dimLen == 1 && dim[0] == kMaxDimension)) || siIsScalar(xsi)) { outInfo = scalarInfoRank1(); return; }
    if (dimLen > 1 && siIsVector(xsi)) { outInfo = x; return; }
    if (numTads == 1 && (rank == dimLen || dimLen == 0)) {
        bool permuted = false;
        for (int i = 0; i < dimLen - 1; i++) if (dim[i] > dim[i + 1]) permuted = true;
        if (permuted) permuteInfo(x, dim);
        outInfo = x;
        return;
    }
    if (dimLen == 1) {
        if (dim[0] == 0 && siIsVector(xsi) && shp[1] == 1) {
            int p[2] = {1, 0};
            permuteInfo(x, p);
            outInfo = x;
            return;
        } else if (dim[0] == 1 && siIsVector(xsi) && shp[0] == 1) {
            outInfo = x;
            return;
        } else if (shp[dim[0]] == 1) {
            outInfo = scalarInfoRank1();
            outInfo[3] = 0;  // offset slot <- tadIndex
            return;
        }
    }

    // permutation: untouched dimensions first (ascending), then the TAD dimensions in reverse
    int perm[kMaxRank];
    int np = 0;
    for (int i = 0; i < rank; i++) {
        bool inDim = false;
        for (int j = 0; j < dimLen; j++) if (dim[j] == i) inDim = true;
        if (!inDim) perm[np++] = i;
    }
    for (int j = dimLen - 1; j >= 0; j--) perm[np++] = dim[j];

    Long tensorLength = 1;
    int tensorLengthInt = 1;  // shape::prod works in 32-bit ints
    for (int j = 0; j < dimLen; j++) { tensorLength *= shp[dim[j]]; tensorLengthInt *= (int)shp[dim[j]]; }

    Buf permuted = x;
    permuteInfo(permuted, perm);
    Buf ret = sliceZero(permuted);

    Long compLength = siIsVector(ret.data()) ? siNumel(ret.data()) : (Long)tensorLengthInt;
    if (compLength == siNumel(ret.data())) {
        if (dimLen == 1 && siIsVector(ret.data()) && siShape(ret.data())[0] == 1) {
            // row vectors are returned as they are
        } else if (dimLen > 1) {
            reversePermuteInPlace(ret);
        }
    } else {
        Long lengthPerSlice = prodOf(siShape(ret.data()) + 1, siRank(ret.data()) - 1);
        if (lengthPerSlice < 1) { outInfo = ret; return; }
        if (tensorLength == lengthPerSlice) {
            ret = sliceZero(ret);
            if (!siIsRowVector(ret.data())) reversePermuteInPlace(ret);
        } else {
            while (siNumel(ret.data()) > tensorLength) ret = sliceZero(ret);
            if (dimLen == 1 && siIsVector(ret.data()) && siShape(ret.data())[0] == 1) {
                // unchanged
            } else if (dimLen > 1) {
                reversePermuteCopy(ret);
            }
        }
    }
    outInfo = ret;
}

// Element offset of TAD `index` (TAD.h:577-611 with tad2Sub 613-712): C-order coordinates over the
// dimensions that are not part of the TAD, applied to the strides of x (unit dimensions contribute 0).
inline Long tadOffsetOf(const Long *xsi, const int *dim, int dimLen, bool wholeThing, Long index) {
    if (wholeThing) return index;
    int rank = siRank(xsi);
    const Long *shp = siShape(xsi), *str = siStride(xsi);
    int left[kMaxRank];
    int nl = 0;
    int len = 1;  // 32-bit like the reference
    for (int i = 0; i < rank; i++) {
        bool inDim = false;
        for (int j = 0; j < dimLen; j++) if (dim[j] == i) { inDim = true; break; }
        if (!inDim) { left[nl++] = i; len *= (int)shp[i]; }
    }
    Long off = 0;
    int denom = len;
    int idx = (int)index;
    for (int k = 0; k < nl; k++) {
        denom /= (int)shp[left[k]];
        Long c = 0;
        if (denom > 0) { c = idx / denom; idx %= denom; }
        if (shp[left[k]] != 1) off += c * str[left[k]];
    }
    return off;
}

// shape::TAD::init + createTadOnlyShapeInfo + createOffsets, i.e. what NativeOps::tadOnlyShapeInfo
// exports (reference: blas/cpu/NativeOps.cpp:2022-2032).
inline void computeTad(const Long *xsi, const int *dim, int dimLen, TadPack &out, bool wantOffsets = true) {
    int rank = siRank(xsi);
    Long numTads = dimLen == 0 ? 1 : siNumel(xsi) / tadLengthOf(xsi, dim, dimLen);
    Long ews = siEws(xsi);
    bool whole = false;
    if (!siIsVector(xsi)) {
        whole = numTads == 1 ||
                ((dimLen == rank || (numTads == siNumel(xsi) && siOrder(xsi) == 'c')) && ews == 1);
    } else if (siIsScalar(xsi)) {
        whole = true;
    }
    out.numTads = numTads;
    out.wholeThing = whole;
    buildTadShapeInfo(xsi, dim, dimLen, numTads, whole, out.shapeInfo);
    out.offsets.clear();
    if (wantOffsets) {
        out.offsets.resize((size_t)numTads);
        // The coordinates tadOffsetOf derives from the index by division are those of an odometer over the dimensions
        // outside the TAD (last one fastest), as long as their product stays within the reference's 32-bit arithmetic:
        // then the offsets are stepped instead of divided out (a million TADs in a few milliseconds instead of fifty).
        int left[kMaxRank];
        int nl = 0;
        Long product = 1;
        const Long *shp = siShape(xsi), *str = siStride(xsi);
        for (int i = 0; i < rank; i++) {
            bool inDim = false;
            for (int j = 0; j < dimLen; j++) if (dim[j] == i) { inDim = true; break; }
            if (!inDim) { left[nl++] = i; product *= shp[i]; }
        }
        if (whole) {
            for (Long i = 0; i < numTads; i++) out.offsets[(size_t)i] = i;
        } else if (nl > 0 && product == numTads && product <= 0x7fffffffLL) {
            Long coord[kMaxRank] = {0};
            Long off = 0;
            for (Long i = 0; i < numTads; i++) {
                out.offsets[(size_t)i] = off;
                for (int k = nl - 1; k >= 0; k--) {
                    const Long extent = shp[left[k]], stride = extent != 1 ? str[left[k]] : 0;
                    coord[k]++;
                    off += stride;
                    if (coord[k] < extent) break;
                    off -= coord[k] * stride;
                    coord[k] = 0;
                }
            }
        } else {
            for (Long i = 0; i < numTads; i++) out.offsets[(size_t)i] = tadOffsetOf(xsi, dim, dimLen, whole, i);
        }
    }
}

}  // namespace nd4j_amd
