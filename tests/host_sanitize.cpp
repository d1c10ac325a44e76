// Host-only exercise of the code that decodes caller-shaped buffers - the shapeInfo / TAD logic (shape_host.h), the
// stride canonicalisation and the division-by-multiplication helper (view.h) - for a build with
// -fsanitize=address,undefined (tests/test_host_sanitizers.py compiles and runs it; no GPU involved).
// Inputs are generated shapes, strides (dense, permuted, padded, with unit dimensions) and dimension lists; checked are
// the invariants a kernel launch relies on: every TAD offset plus every TAD element offset lies inside the view's
// span, the TADs partition the array, canonicalised maps address the same elements as the original strides.
#include <cstdio>
#include <cstdlib>
#include <set>
#include <stdexcept>
#include <vector>

typedef long long Long;
#include "../libnd4j_amd/csrc/view.h"

using namespace nd4j_amd;

static unsigned long long state = 88172645463325252ULL;
static unsigned rnd(unsigned n) {
    state ^= state << 13; state ^= state >> 7; state ^= state << 17;
    return (unsigned)((state >> 11) % n);
}
static int fail(const char *what, int it) {
    std::printf("FAILED %s (case %d)\n", what, it);
    return 1;
}

static Long mapOffset(const DimMap &m, Long idx) {
    Long off = 0;
    for (int d = m.rank - 1; d >= 0; d--) { off += (idx % m.shape[d]) * m.stride[d]; idx /= m.shape[d]; }
    return off;
}

int main() {
    const int sizes[] = {1, 2, 3, 4, 5, 7, 8, 16};
    for (int it = 0; it < 4000; it++) {
        const int rank = 1 + (int)rnd(5);
        std::vector<Long> shape(rank), stride(rank);
        for (int d = 0; d < rank; d++) shape[d] = sizes[rnd(8)];
        const char order = rnd(2) ? 'c' : 'f';
        const int kind = (int)rnd(3);  // dense, permuted dense, permuted with padding
        std::vector<int> perm(rank);
        for (int d = 0; d < rank; d++) perm[d] = order == 'c' ? rank - 1 - d : d;
        if (kind > 0) for (int d = rank - 1; d > 0; d--) std::swap(perm[d], perm[rnd(d + 1)]);
        Long run = kind == 2 ? 1 + rnd(3) : 1;
        for (int k = 0; k < rank; k++) { stride[perm[k]] = run; run *= shape[perm[k]] + (kind == 2 ? rnd(3) : 0); }
        Long n = 1, span = 1;
        for (int d = 0; d < rank; d++) { n *= shape[d]; span += (shape[d] - 1) * stride[d]; }
        // shapeInfo: [rank, shape.., stride.., offset, ews, order]
        std::vector<Long> info(siLength(rank));
        info[0] = rank;
        for (int d = 0; d < rank; d++) { info[1 + d] = shape[d]; info[1 + rank + d] = stride[d]; }
        info[2 * rank + 1] = 0;
        info[2 * rank + 2] = (kind == 0 && rank > 0) ? 1 : -1;
        info[2 * rank + 3] = order;
        if (siNumel(info.data()) != n) return fail("siNumel", it);

        // TADs along a random non-empty proper subset of the dimensions (or all of them)
        const int dimLen = 1 + (int)rnd(rank);
        std::vector<int> dims;
        while ((int)dims.size() < dimLen) {
            int d = (int)rnd(rank);
            bool have = false;
            for (int v : dims) have = have || v == d;
            if (!have) dims.push_back(d);
        }
        for (size_t a = 0; a + 1 < dims.size(); a++)
            for (size_t b = a + 1; b < dims.size(); b++)
                if (dims[b] < dims[a]) std::swap(dims[a], dims[b]);
        TadPack pack;
        computeTad(info.data(), dims.data(), dimLen, pack, true);
        const Long tadLength = tadLengthOf(info.data(), dims.data(), dimLen);
        if (tadLength <= 0 || n % tadLength != 0) return fail("tad length", it);
        if (pack.numTads != n / tadLength || (Long)pack.offsets.size() != pack.numTads) return fail("tad count", it);
        const Long *ti = pack.shapeInfo.data();
        if (siNumel(ti) != tadLength) return fail("tad shapeInfo length", it);
        DimMap tm;
        ownCanon(siRank(ti), siShape(ti), siStride(ti), tm);
        std::set<Long> seen;
        for (Long t = 0; t < pack.numTads; t++) {
            for (Long f = 0; f < tadLength; f++) {
                const Long off = pack.offsets[t] + mapOffset(tm, f);
                if (off < 0 || off >= span) return fail("tad element outside the view", it);
                seen.insert(off);
            }
        }
        if ((Long)seen.size() != n) return fail("TADs do not partition the array", it);

        // canonical maps address the elements the strides address
        DimMap own;
        ownCanon(rank, shape.data(), stride.data(), own);
        Long total = 1;
        for (int d = 0; d < own.rank; d++) total *= own.shape[d];
        if (total != n) return fail("ownCanon element count", it);
        std::set<Long> viaOwn;
        for (Long i = 0; i < n; i++) viaOwn.insert(mapOffset(own, i));
        if (viaOwn != seen) return fail("ownCanon addresses other elements", it);
        const Long *strides[3] = {stride.data(), nullptr, stride.data()};
        DimMap joint[3];
        jointCanon(rank, shape.data(), strides, joint);
        std::set<Long> viaJoint;
        for (Long i = 0; i < n; i++) {
            if (mapOffset(joint[0], i) != mapOffset(joint[2], i)) return fail("jointCanon operands disagree", it);
            viaJoint.insert(mapOffset(joint[0], i));
        }
        if (viaJoint != seen) return fail("jointCanon addresses other elements", it);
    }
    // FastDiv against the division it stands for
    for (int it = 0; it < 500000; it++) {
        const unsigned d = 1 + (it & 1 ? rnd(5000) : rnd(0x7ffffffe));
        const unsigned v = (unsigned)(((unsigned long long)rnd(0x7fffffff) << 1 | rnd(2)) & 0x7fffffffu);
        const FastDiv f(d);
        unsigned rem;
        if (f.div(v) != v / d || f.divmod(v, rem) != v / d || rem != v % d) return fail("FastDiv", it);
    }
    // Extents that do not fit 32 bits: a map of one dimension clamps its extent (the kernels never divide by it), one of
    // several dimensions refuses instead of wrapping round
    {
        const Long big = (Long)1 << 33;
        Long shape1[1] = {big}, stride1[1] = {1};
        DimMap m1;
        ownCanon(1, shape1, stride1, m1);
        if (m1.rank != 1 || m1.shape[0] != 0xffffffffu) return fail("one long dimension", 0);
        Long shape2[2] = {big, 3}, dense2[2] = {3, 1}, padded2[2] = {4, 1};
        ownCanon(2, shape2, dense2, m1);  // merges into one run of 3 * 2^33 elements
        if (m1.rank != 1 || m1.shape[0] != 0xffffffffu || m1.stride[0] != 1) return fail("merged long dimension", 0);
        bool threw = false;
        try { ownCanon(2, shape2, padded2, m1); } catch (const std::invalid_argument &) { threw = true; }
        if (!threw) return fail("a long dimension beside another one was not refused", 0);
        const Long *strides[3] = {padded2, nullptr, padded2};
        DimMap joint[3];
        threw = false;
        try { jointCanon(2, shape2, strides, joint); } catch (const std::invalid_argument &) { threw = true; }
        if (!threw) return fail("jointCanon: a long dimension beside another one was not refused", 0);
    }
    // the common run length of up to three maps
    {
        DimMap a, b, c;
        a.rank = 2; a.shape[0] = 7; a.shape[1] = 24; a.stride[0] = 100; a.stride[1] = 1;
        b.rank = 1; b.shape[0] = 7 * 24; b.stride[0] = 1;
        c.rank = 3; c.shape[0] = 7; c.shape[1] = 2; c.shape[2] = 12; c.stride[0] = 50; c.stride[1] = 20; c.stride[2] = 1;
        const DimMap *abc[3] = {&a, &b, &c}, *ab[3] = {&a, &b, nullptr};
        if (commonRunLength(abc) != 12 || commonRunLength(ab) != 24) return fail("commonRunLength", 0);
        c.stride[2] = 2;
        if (commonRunLength(abc) != 0) return fail("commonRunLength with a strided innermost dimension", 0);
    }
    std::printf("host sanitize run: ok\n");
    return 0;
}
