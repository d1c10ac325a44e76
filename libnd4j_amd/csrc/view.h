// Stride canonicalisation: turns shapeInfo views into the small by-value descriptors the kernels take.
//
// Two situations occur in the reference's loops:
//  * all operands are walked with the SAME logical coordinates (raw iteration in cpu/transform.cpp:50-87
//    and pairwise_transform.h:241-313).  The visiting order is irrelevant for an elementwise op, so the
//    dimensions may be dropped (size 1), sorted by the output stride and merged wherever every operand
//    is contiguous across the pair: a dense f-order array paired with a dense f-order output collapses
//    to one contiguous run and takes the vector path.
//  * every operand is walked by ITS OWN C-order linear index (ind2subC branches,
//    pairwise_transform.h:315-365).  Only C-order merging of adjacent dimensions is allowed then.
#pragma once

#include <algorithm>
#include <cstdlib>
#include <stdexcept>

#include "shape_host.h"

namespace nd4j_amd {

static const int kMaxDims = kMaxRank;

// One operand's index -> element offset map: offset = sum(coord[d] * stride[d]) with coord the C-order
// decomposition of the linear index over `shape`.
struct DimMap {
    int rank;
    unsigned shape[kMaxDims];
    Long stride[kMaxDims];
};

// n / d and n % d for 0 <= n < 2^31 and 1 <= d < 2^31 through one high multiplication: with s = ceil(log2 d) and
// m = ceil(2^(31 + s) / d) (which fits 32 bits), floor(n * m / 2^(31 + s)) == floor(n / d) because the excess
// n * (m * d - 2^(31 + s)) / (d * 2^(31 + s)) stays below 1 / d.
struct FastDiv {
    unsigned d = 1, m = 0, shift = 0;
    FastDiv() {}
    explicit FastDiv(unsigned divisor) : d(divisor < 1 ? 1 : divisor) {
        unsigned s = 0;
        while (((unsigned long long)1 << s) < d) s++;
        if (s == 0) { m = 0; shift = 0; return; }  // d == 1
        m = (unsigned)((((unsigned long long)1 << (31 + s)) + d - 1) / d);
        shift = s - 1;
    }
#if defined(__HIPCC__)
    __host__ __device__
#endif
    inline unsigned div(unsigned n) const {
        const unsigned q = (unsigned)(((unsigned long long)n * m) >> 32) >> shift;
        return d == 1 ? n : q;
    }
    // returns n / d and leaves n % d in rem
#if defined(__HIPCC__)
    __host__ __device__
#endif
    inline unsigned divmod(unsigned n, unsigned &rem) const {
        const unsigned q = div(n);
        rem = n - q * d;
        return q;
    }
};

// An extent as a DimMap stores it.  A map of one dimension is walked by multiplying the index with the stride and never
// looks at its extent (which may exceed 32 bits: whole arrays of more than 2^32 elements); with two dimensions or more the
// kernels divide by the extents in 32-bit arithmetic, so one that does not fit is refused instead of wrapping round.
inline unsigned mapExtent(Long extent, int rank) {
    if (extent > 0xffffffffLL) {
        if (rank > 1) throw std::invalid_argument("a view with a (merged) dimension of 2^32 elements or more next to other dimensions is not supported");
        return 0xffffffffu;
    }
    return (unsigned)extent;
}

// C-order merge of one operand (drop unit dims, fuse dims d,d+1 when stride[d] == shape[d+1]*stride[d+1]).
inline void ownCanon(int rank, const Long *shape, const Long *stride, DimMap &out) {
    Long shp[kMaxDims], str[kMaxDims];
    int n = 0;
    for (int i = 0; i < rank; i++)
        if (shape[i] != 1) { shp[n] = shape[i]; str[n] = stride[i]; n++; }
    int m = 0;
    for (int i = 0; i < n; i++) {
        if (m > 0 && str[m - 1] == shp[i] * str[i]) {
            shp[m - 1] *= shp[i];
            str[m - 1] = str[i];
        } else {
            shp[m] = shp[i]; str[m] = str[i]; m++;
        }
    }
    if (m == 0) { shp[0] = 1; str[0] = 1; m = 1; }
    out.rank = m;
    for (int i = 0; i < m; i++) { out.shape[i] = mapExtent(shp[i], m); out.stride[i] = str[i]; }
}

// Joint canonicalisation of up to three operands sharing one shape.  `strides[k]` may be null for an
// absent operand.  On return every present operand has the same rank/shape in `out[k]`.
inline void jointCanon(int rank, const Long *shape, const Long *const strides[3], DimMap out[3]) {
    struct D { Long shp; Long s[3]; };
    D d[kMaxDims];
    int n = 0;
    for (int i = 0; i < rank; i++) {
        if (shape[i] == 1) continue;
        d[n].shp = shape[i];
        for (int k = 0; k < 3; k++) d[n].s[k] = strides[k] ? strides[k][i] : 0;
        n++;
    }
    int key = strides[2] ? 2 : (strides[1] ? 1 : 0);
    std::stable_sort(d, d + n, [key](const D &a, const D &b) { return std::llabs(a.s[key]) > std::llabs(b.s[key]); });
    int m = 0;
    for (int i = 0; i < n; i++) {
        bool fuse = m > 0;
        if (fuse)
            for (int k = 0; k < 3; k++)
                if (strides[k] && d[m - 1].s[k] != d[i].shp * d[i].s[k]) fuse = false;
        if (fuse) {
            d[m - 1].shp *= d[i].shp;
            for (int k = 0; k < 3; k++) d[m - 1].s[k] = d[i].s[k];
        } else {
            d[m++] = d[i];
        }
    }
    if (m == 0) { d[0].shp = 1; for (int k = 0; k < 3; k++) d[0].s[k] = 1; m = 1; }
    for (int k = 0; k < 3; k++) {
        out[k].rank = m;
        for (int i = 0; i < m; i++) { out[k].shape[i] = mapExtent(d[i].shp, m); out[k].stride[i] = d[i].s[k]; }
    }
}

// Largest run length the contiguous-run kernel can use for these maps: the greatest common divisor of the innermost
// extents when every present map ends in a stride of 1, else 0.  (A run of that many elements starting at a multiple of
// it lies inside the innermost dimension of every operand.)
inline unsigned commonRunLength(const DimMap *const maps[3]) {
    unsigned long long g = 0;
    for (int k = 0; k < 3; k++) {
        const DimMap *m = maps[k];
        if (m == nullptr) continue;
        if (m->rank < 1 || m->stride[m->rank - 1] != 1) return 0;
        unsigned long long a = m->shape[m->rank - 1], b = g;
        while (b != 0) { const unsigned long long t = a % b; a = b; b = t; }
        g = a;
    }
    return (unsigned)g;
}

}  // namespace nd4j_amd
