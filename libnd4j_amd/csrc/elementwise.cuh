// Elementwise kernels shared by the transform, pairwise and broadcast families.
//
//   ewVecKernel      all operands contiguous: one 16-byte vector per operand and thread.
//   ewGeneralKernel  arbitrary views: each operand has its own index -> offset map (DimMap).
//   bcRowKernel      broadcast over contiguous TADs: one 16-byte vector of x / z per thread, y through the
//                    caches; a block spans as many neighbouring TADs as fill it.
//   bcColKernel      broadcast over strided TADs: one thread per TAD, neighbouring TADs coalesce.
//   bcGeneralKernel  broadcast with per-element coordinate maps.
//
// All of them are HBM-bound: algorithmic bytes are (inputs + 1) * sizeof(T) per element.
#pragma once

#include <hip/hip_runtime.h>

#include <utility>

#include "launch.h"
#include "ops_elementwise.cuh"
#include "types.h"
#include "view.h"

namespace nd4j_amd {

static constexpr int kBlock = 256;
static constexpr int kUnroll = 4;

template <typename T> struct alignas(16) Pack {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};

// 16-byte accesses with the streaming (non-temporal) cache policy.  The vector kernels touch every operand
// element exactly once per call, and marking the accesses so raises the sustained HBM rate of a three-stream
// kernel from about 5.5 to 6.5 TB/s.  (A run-time switch between the two policies is not possible in one
// kernel: the optimiser merges the two otherwise identical accesses and drops the hint.)
typedef unsigned int U32x4 __attribute__((ext_vector_type(4)));
template <typename T> __device__ __forceinline__ Pack<T> loadPack(const Pack<T> *p) {
    return __builtin_bit_cast(Pack<T>, __builtin_nontemporal_load(reinterpret_cast<const U32x4 *>(p)));
}
template <typename T> __device__ __forceinline__ void storePack(Pack<T> *p, const Pack<T> &v) {
    __builtin_nontemporal_store(__builtin_bit_cast(U32x4, v), reinterpret_cast<U32x4 *>(p));
}

// 16 bytes at an address that is only aligned to the element size: the hardware serves misaligned global accesses
// (slower than aligned ones where they straddle cache lines, far faster than element-wise accesses).
typedef U32x4 U32x4A2 __attribute__((aligned(2)));
typedef U32x4 U32x4A4 __attribute__((aligned(4)));
typedef U32x4 U32x4A8 __attribute__((aligned(8)));
template <typename T> __device__ __forceinline__ Pack<T> loadPackAnywhere(const T *p) {
    U32x4 v;
    if (sizeof(T) == 2) v = *reinterpret_cast<const U32x4A2 *>(p);
    else if (sizeof(T) == 4) v = *reinterpret_cast<const U32x4A4 *>(p);
    else v = *reinterpret_cast<const U32x4A8 *>(p);
    return __builtin_bit_cast(Pack<T>, v);
}
template <typename T> __device__ __forceinline__ void storePackAnywhere(T *p, const Pack<T> &a) {
    const U32x4 v = __builtin_bit_cast(U32x4, a);
    if (sizeof(T) == 2) *reinterpret_cast<U32x4A2 *>(p) = v;
    else if (sizeof(T) == 4) *reinterpret_cast<U32x4A4 *>(p) = v;
    else *reinterpret_cast<U32x4A8 *>(p) = v;
}
// the same with the streaming cache policy of loadPack / storePack
template <typename T> __device__ __forceinline__ Pack<T> streamPackAnywhere(const T *p) {
    U32x4 v;
    if (sizeof(T) == 2) v = __builtin_nontemporal_load(reinterpret_cast<const U32x4A2 *>(p));
    else if (sizeof(T) == 4) v = __builtin_nontemporal_load(reinterpret_cast<const U32x4A4 *>(p));
    else v = __builtin_nontemporal_load(reinterpret_cast<const U32x4A8 *>(p));
    return __builtin_bit_cast(Pack<T>, v);
}
template <typename T> __device__ __forceinline__ void streamPackAnywhere(T *p, const Pack<T> &a) {
    const U32x4 v = __builtin_bit_cast(U32x4, a);
    if (sizeof(T) == 2) __builtin_nontemporal_store(v, reinterpret_cast<U32x4A2 *>(p));
    else if (sizeof(T) == 4) __builtin_nontemporal_store(v, reinterpret_cast<U32x4A4 *>(p));
    else __builtin_nontemporal_store(v, reinterpret_cast<U32x4A8 *>(p));
}

// Functor adapters: apply(a, b, params)
template <int OP> struct TransformF {
    static constexpr int nin = 1;
    static constexpr bool tables = !transformIsPlain(OP);
    template <typename C, typename P> static __device__ __forceinline__ C apply(C a, C, P p) {
        return TransformOp<OP>::template op<C, P>(a, p);
    }
};
template <int KIND> struct Pairwise3F {
    static constexpr int nin = 2;
    static constexpr bool tables = !binaryIsPlain(KIND);
    template <typename C, typename P> static __device__ __forceinline__ C apply(C a, C b, P p) {
        return BinaryOp<KIND>::template op3<C, P>(a, b, p);
    }
};
// scalar family: z = op(x, scalar, params) (scalar.h: OpType::op(x, scalar, extra)).  The scalar is loop-invariant
// in the reference's loops, and its release flags (-freciprocal-math) turn every division by it into a
// multiplication by 1 / scalar: Divide, SafeDivide and FloorDiv are evaluated that way here too (the compiled
// reference agrees with x * (1 / s) on all of 200000 random operands, with x / s on 60 % of them).
template <int KIND, typename C, typename P> __device__ __forceinline__ C scalarOp(C a, C s, P p) {
    if (KIND == B_Divide) return a * ((C)1 / s);
    if (KIND == B_SafeDivide) return s == (C)0 ? (C)0 : a * ((C)1 / s);
    if (KIND == B_FloorDiv) return m::floor_(a * ((C)1 / s));
    return BinaryOp<KIND>::template op3<C, P>(a, s, p);
}
// one scalar for the whole array, carried by value in Params
template <int KIND> struct Scalar3F {
    static constexpr int nin = 1;
    static constexpr bool tables = !binaryIsPlain(KIND);
    template <typename C, typename P> static __device__ __forceinline__ C apply(C a, C, P p) {
        return scalarOp<KIND, C, P>(a, p.scalarValue(), p);
    }
};
// one scalar per TAD, passed as the second operand
template <int KIND> struct ScalarTad3F {
    static constexpr int nin = 2;
    static constexpr bool tables = !binaryIsPlain(KIND);
    template <typename C, typename P> static __device__ __forceinline__ C apply(C a, C b, P p) {
        return scalarOp<KIND, C, P>(a, b, p);
    }
};
template <int KIND> struct Broadcast2F {
    static constexpr int nin = 2;
    static constexpr bool tables = !binaryIsPlain(KIND);
    template <typename C, typename P> static __device__ __forceinline__ C apply(C a, C b, P) {
        return BinaryOp<KIND>::template op2<C>(a, b);
    }
};

// ---------------------------------------------------------------------------------------------------
// z[i] = F(x[i], y[i or 0]) over n contiguous elements.  `head` leading elements are done one by one so
// that the vector part starts on a 16-byte boundary (the host guarantees all operands share the same
// misalignment); yScalar selects y[0] for every element.  Launched with kBlock threads or fewer (the kernel goes by
// blockDim.x; the lookup-table staging wants all kBlock).
template <typename T, typename F>
__global__ void __launch_bounds__(kBlock) ewVecKernel(const T *x, const T *y, T *z, Params<T> p, Long n, int head,
                                                      int yScalar) {
    typedef typename Compute<T>::type C;
    constexpr int VEC = Pack<T>::N;
    const Long body = n - head;
    const Long nvec = body / VEC;
    const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x + head);
    const Pack<T> *yv = reinterpret_cast<const Pack<T> *>(y + head);
    Pack<T> *zv = reinterpret_cast<Pack<T> *>(z + head);
    C ys = (C)0;
    if (F::nin == 2 && yScalar) ys = toCompute(y[0]);

    // one vector per thread and pass (the launcher gives one-operand calls two passes per thread): many short blocks
    // sustain a higher HBM rate on this chip than fewer blocks with several vectors in flight per thread
    if (F::tables) {
        // the first vectors are requested before the lookup tables are staged, so the two waits overlap
        Long j = (Long)blockIdx.x * blockDim.x + threadIdx.x;
        bool have = j < nvec;
        Pack<T> a, b;
        if (have) {
            a = loadPack(xv + j);
            if (F::nin == 2 && !yScalar) b = loadPack(yv + j);
        }
        lm::loadTables();
        while (have) {
            Pack<T> r;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                C bv = (F::nin == 2) ? (yScalar ? ys : toCompute(b.v[e])) : (C)0;
                r.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a.v[e]), bv, p));
            }
            storePack(zv + j, r);
            j += (Long)gridDim.x * blockDim.x;
            have = j < nvec;
            if (have) {
                a = loadPack(xv + j);
                if (F::nin == 2 && !yScalar) b = loadPack(yv + j);
            }
        }
    } else {
        for (Long j = (Long)blockIdx.x * blockDim.x + threadIdx.x; j < nvec; j += (Long)gridDim.x * blockDim.x) {
            Pack<T> a = loadPack(xv + j), b;
            if (F::nin == 2 && !yScalar) b = loadPack(yv + j);
            Pack<T> r;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                C bv = (F::nin == 2) ? (yScalar ? ys : toCompute(b.v[e])) : (C)0;
                r.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a.v[e]), bv, p));
            }
            storePack(zv + j, r);
        }
    }
    // head and tail elements
    const Long gtid = (Long)blockIdx.x * blockDim.x + threadIdx.x;
    const Long tailStart = head + nvec * VEC;
    const Long nScalar = head + (n - tailStart);
    if (gtid < nScalar) {
        Long i = gtid < head ? gtid : tailStart + (gtid - head);
        C bv = (F::nin == 2) ? (yScalar ? ys : toCompute(y[i])) : (C)0;
        z[i] = fromCompute<T>(F::template apply<C>(toCompute(x[i]), bv, p));
    }
}

// C-order linear index -> element offset through a DimMap.
__device__ __forceinline__ Long mapOffset32(const DimMap &m, unsigned idx) {
    if (m.rank == 1) return (Long)idx * m.stride[0];
    Long off = 0;
    for (int d = m.rank - 1; d > 0; d--) {
        unsigned q = idx / m.shape[d];
        unsigned c = idx - q * m.shape[d];
        off += (Long)c * m.stride[d];
        idx = q;
    }
    return off + (Long)idx * m.stride[0];
}
__device__ __forceinline__ Long mapOffset64(const DimMap &m, unsigned long long idx) {
    if (m.rank == 1) return (Long)idx * m.stride[0];
    Long off = 0;
    for (int d = m.rank - 1; d > 0; d--) {
        unsigned long long q = idx / m.shape[d];
        unsigned long long c = idx - q * m.shape[d];
        off += (Long)c * m.stride[d];
        idx = q;
    }
    return off + (Long)idx * m.stride[0];
}

// for walks over whole arrays, which may hold more than 2^32 elements: 32-bit divisions while the index allows them
__device__ __forceinline__ Long mapOffsetAny(const DimMap &m, Long idx) {
    return idx <= 0xffffffffLL ? mapOffset32(m, (unsigned)idx) : mapOffset64(m, (unsigned long long)idx);
}

template <typename T, typename F>
__global__ void __launch_bounds__(kBlock) ewGeneralKernel(const T *x, DimMap xm, const T *y, DimMap ym, T *z,
                                                          DimMap zm, Params<T> p, Long n) {
    typedef typename Compute<T>::type C;
    if (F::tables) lm::loadTables();
    const Long stride = (Long)gridDim.x * kBlock;
    if (n <= 0xffffffffLL) {
        for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
            Long ox = mapOffset32(xm, (unsigned)i);
            Long oz = mapOffset32(zm, (unsigned)i);
            C bv = (C)0;
            if (F::nin == 2) bv = toCompute(y[mapOffset32(ym, (unsigned)i)]);
            z[oz] = fromCompute<T>(F::template apply<C>(toCompute(x[ox]), bv, p));
        }
    } else {
        for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
            Long ox = mapOffset64(xm, (unsigned long long)i);
            Long oz = mapOffset64(zm, (unsigned long long)i);
            C bv = (C)0;
            if (F::nin == 2) bv = toCompute(y[mapOffset64(ym, (unsigned long long)i)]);
            z[oz] = fromCompute<T>(F::template apply<C>(toCompute(x[ox]), bv, p));
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Broadcast over contiguous TADs (tadEWS == yEWS == zEWS == 1).  A block covers colThreads (a power of two)
// column vectors of kBlock / colThreads neighbouring TADs and walks kBcRows such TAD groups per pass, so the
// TAD offsets and the x vectors of all of them are in flight together; blockIdx.x walks the TADs, blockIdx.y
// the column chunks.  y comes through the caches, x and z are streamed.  TADs whose offsets (or the base
// pointers) are not 16-byte aligned fall back to scalar accesses for that TAD only.
static constexpr int kBcRows = 4;

// BYTAD: y holds one value per TAD (the scalar family's per-TAD scalars) instead of one per TAD element.
template <typename T, typename F, bool BYTAD>
__global__ void __launch_bounds__(kBlock) bcRowKernel(const T *x, const T *y, T *z, const Long *xOffsets,
                                                      const Long *zOffsets, Long tadLength, Long numTads,
                                                      int basesAligned, int colShift, Params<T> p) {
    typedef typename Compute<T>::type C;
    if (F::tables) lm::loadTables();
    constexpr int VEC = Pack<T>::N;
    const int colThreads = 1 << colShift;
    const int rowsPerBlock = kBlock >> colShift;
    const int cIdx = threadIdx.x & (colThreads - 1);
    const int rIdx = threadIdx.x >> colShift;
    const bool yAligned = (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    for (Long col = ((Long)blockIdx.y * colThreads + cIdx) * VEC; col < tadLength; col += (Long)gridDim.y * colThreads * VEC) {
        const bool full = col + VEC <= tadLength;
        C yv[VEC];
        if (BYTAD) {
#pragma unroll
            for (int e = 0; e < VEC; e++) yv[e] = (C)0;
        } else if (full && yAligned) {
            const Pack<T> yp = *reinterpret_cast<const Pack<T> *>(y + col);  // through the caches: every TAD re-reads it
#pragma unroll
            for (int e = 0; e < VEC; e++) yv[e] = toCompute(yp.v[e]);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; e++) yv[e] = (col + e < tadLength) ? toCompute(y[col + e]) : (C)0;
        }
        const Long rowsPerPass = (Long)rowsPerBlock * kBcRows;
        for (Long r0 = (Long)blockIdx.x * rowsPerPass + rIdx; r0 < numTads; r0 += (Long)gridDim.x * rowsPerPass) {
            Long xo[kBcRows], zo[kBcRows];
            bool live[kBcRows], vec[kBcRows];
            Pack<T> a[kBcRows];
            C ys[kBcRows];
#pragma unroll
            for (int u = 0; u < kBcRows; u++) {
                const Long r = r0 + (Long)u * rowsPerBlock;
                live[u] = r < numTads;
                xo[u] = live[u] ? xOffsets[r] : 0;
                zo[u] = live[u] ? zOffsets[r] : 0;
                ys[u] = (BYTAD && live[u]) ? toCompute(y[r]) : (C)0;
            }
#pragma unroll
            for (int u = 0; u < kBcRows; u++) {
                vec[u] = live[u] && full && basesAligned && ((xo[u] | zo[u]) % VEC) == 0;
                if (vec[u]) a[u] = loadPack(reinterpret_cast<const Pack<T> *>(x + xo[u] + col));
            }
#pragma unroll
            for (int u = 0; u < kBcRows; u++) {
                if (vec[u]) {
                    Pack<T> o;
#pragma unroll
                    for (int e = 0; e < VEC; e++)
                        o.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a[u].v[e]), BYTAD ? ys[u] : yv[e], p));
                    storePack(reinterpret_cast<Pack<T> *>(z + zo[u] + col), o);
                } else if (live[u]) {
                    const T *xr = x + xo[u] + col;
                    T *zr = z + zo[u] + col;
#pragma unroll
                    for (int e = 0; e < VEC; e++)
                        if (col + e < tadLength)
                            zr[e] = fromCompute<T>(F::template apply<C>(toCompute(xr[e]), BYTAD ? ys[u] : yv[e], p));
                }
            }
        }
    }
}

// Broadcast over contiguous TADs that follow one another without gaps in x and in z (the rows of a dense c-order
// matrix): the array is walked as one long vector, one 16-byte vector per thread as in ewVecKernel, and the only
// trace of the TADs is the position inside the row, which selects the vector of y (read through the caches).  No
// offset tables are read.  Needs tadLength % VEC == 0 and 16-byte aligned x, y, z.
template <typename T, typename F>
__global__ void __launch_bounds__(kBlock) bcFlatKernel(const T *x, const T *y, T *z, Long nvec, unsigned vecsPerTad,
                                                       Params<T> p) {
    typedef typename Compute<T>::type C;
    if (F::tables) lm::loadTables();
    constexpr int VEC = Pack<T>::N;
    const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x);
    const Pack<T> *yv = reinterpret_cast<const Pack<T> *>(y);
    Pack<T> *zv = reinterpret_cast<Pack<T> *>(z);
    const bool pow2 = (vecsPerTad & (vecsPerTad - 1)) == 0;
    for (Long j = (Long)blockIdx.x * blockDim.x + threadIdx.x; j < nvec; j += (Long)gridDim.x * blockDim.x) {
        const Pack<T> a = loadPack(xv + j);
        unsigned col;
        if (pow2) col = (unsigned)j & (vecsPerTad - 1);  // the usual case: no division
        else col = (j >> 32) == 0 ? (unsigned)j % vecsPerTad : (unsigned)((unsigned long long)j % vecsPerTad);
        const Pack<T> b = yv[col];
        Pack<T> r;
#pragma unroll
        for (int e = 0; e < VEC; e++) r.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a.v[e]), toCompute(b.v[e]), p));
        storePack(zv + j, r);
    }
}

// TADs over the outer and the inner part of a dense array [A, B, C] (dimensions {0, 2}): x and z are still one vector after
// the other; vector j lies in row j / (C / VEC) of the [A * B, C] matrix, whose y row is that of a = row / B.  Two divisions
// by multiplication per vector, no tables.  Needs C % VEC == 0, 16-byte aligned x, y, z and fewer than 2^31 vectors.
template <typename T, typename F>
__global__ void __launch_bounds__(kBlock) bcFlatSlabKernel(const T *x, const T *y, T *z, unsigned nvec, FastDiv vecsPerRow,
                                                           FastDiv mid, Params<T> p) {
    typedef typename Compute<T>::type C;
    if (F::tables) lm::loadTables();
    constexpr int VEC = Pack<T>::N;
    const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x);
    const Pack<T> *yv = reinterpret_cast<const Pack<T> *>(y);
    Pack<T> *zv = reinterpret_cast<Pack<T> *>(z);
    const unsigned step = gridDim.x * blockDim.x;
    for (unsigned j = blockIdx.x * blockDim.x + threadIdx.x; j < nvec;) {
        const Pack<T> a = loadPack(xv + j);
        unsigned col;
        const unsigned row = vecsPerRow.divmod(j, col);
        const Pack<T> b = yv[(size_t)mid.div(row) * vecsPerRow.d + col];
        Pack<T> r;
#pragma unroll
        for (int e = 0; e < VEC; e++) r.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a.v[e]), toCompute(b.v[e]), p));
        storePack(zv + j, r);
        const unsigned before = j;
        j += step;
        if (j < before) break;
    }
}

// The same walk when the TAD length is not a multiple of the vector width (rows of odd length: only every fourth row
// of a float matrix then starts on a 16-byte boundary): x and z are still one aligned vector after the other, and a
// vector's elements take their y one by one, from the position inside the row where the vector begins, wrapping into
// the next row.  The last n % VEC elements are done singly.
template <typename T, typename F>
__global__ void __launch_bounds__(kBlock) bcFlatAnyKernel(const T *x, const T *y, T *z, Long n, Long tadLength, Params<T> p) {
    typedef typename Compute<T>::type C;
    if (F::tables) lm::loadTables();
    constexpr int VEC = Pack<T>::N;
    const Long nvec = n / VEC;
    const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x);
    Pack<T> *zv = reinterpret_cast<Pack<T> *>(z);
    const bool small = n <= 0xffffffffLL;
    for (Long j = (Long)blockIdx.x * kBlock + threadIdx.x; j < nvec; j += (Long)gridDim.x * kBlock) {
        const Pack<T> a = loadPack(xv + j);
        const Long i0 = j * VEC;
        Long f = small ? (Long)((unsigned)i0 % (unsigned)tadLength) : i0 % tadLength;
        Pack<T> r;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            r.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a.v[e]), toCompute(y[f]), p));
            f = f + 1 == tadLength ? 0 : f + 1;
        }
        storePack(zv + j, r);
    }
    const Long gtid = (Long)blockIdx.x * kBlock + threadIdx.x;
    if (gtid < n - nvec * VEC) {
        const Long i = nvec * VEC + gtid;
        z[i] = fromCompute<T>(F::template apply<C>(toCompute(x[i]), toCompute(y[i % tadLength]), p));
    }
}

// Broadcast along one dimension of a dense array, whatever its position (a column vector added to the rows of a c-order
// matrix, a per-channel bias in the middle of a rank-3 array): in memory order, `inner` consecutive elements share one
// y (inner is the dimension's stride) and the y index then steps through the dimension's `extent` values.  x and z are
// walked as aligned vectors; a vector finds its run by two divisions and steps on from there.
template <typename T, typename F>
__global__ void __launch_bounds__(kBlock) bcFlatInnerKernel(const T *x, const T *y, T *z, Long n, Long inner, Long extent, Params<T> p) {
    typedef typename Compute<T>::type C;
    if (F::tables) lm::loadTables();
    constexpr int VEC = Pack<T>::N;
    const Long nvec = n / VEC;
    const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x);
    Pack<T> *zv = reinterpret_cast<Pack<T> *>(z);
    const bool small = n <= 0xffffffffLL;
    for (Long j = (Long)blockIdx.x * kBlock + threadIdx.x; j < nvec; j += (Long)gridDim.x * kBlock) {
        const Pack<T> a = loadPack(xv + j);
        const Long i0 = j * VEC;
        Long q, yi;
        if (small) {
            q = (Long)((unsigned)i0 / (unsigned)inner);
            yi = (Long)((unsigned)q % (unsigned)extent);
        } else {
            q = i0 / inner;
            yi = q % extent;
        }
        Long rem = i0 - q * inner;
        C yv = toCompute(y[yi]);
        Pack<T> r;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            r.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a.v[e]), yv, p));
            if (++rem == inner) {
                rem = 0;
                yi = yi + 1 == extent ? 0 : yi + 1;
                yv = toCompute(y[yi]);
            }
        }
        storePack(zv + j, r);
    }
    const Long gtid = (Long)blockIdx.x * kBlock + threadIdx.x;
    if (gtid < n - nvec * VEC) {
        const Long i = nvec * VEC + gtid;
        z[i] = fromCompute<T>(F::template apply<C>(toCompute(x[i]), toCompute(y[(i / inner) % extent]), p));
    }
}

// Broadcast over strided TADs: thread <-> TAD, loop over the TAD's elements.  When neighbouring TADs
// are neighbours in memory (a column of a c-order matrix) each wave reads and writes full lines.
// MAPPED: TADs over several dimensions without contiguous runs: element f of a TAD (of y, of the result's TAD) lies where
// the operand's coordinate map puts it; f is the same for all lanes of a wave, so the maps are worked out once per wave.
template <typename T, typename F, bool BYTAD, bool MAPPED = false>
__global__ void __launch_bounds__(kBlock) bcColKernel(const T *x, const T *y, T *z, const Long *xOffsets,
                                                      const Long *zOffsets, Long tadLength, Long numTads,
                                                      Long tadEws, Long yEws, Long zEws, Params<T> p, DimMap xm = DimMap(),
                                                      DimMap ym = DimMap(), DimMap zm = DimMap()) {
    typedef typename Compute<T>::type C;
    if (F::tables) lm::loadTables();
    const Long t = (Long)blockIdx.x * kBlock + threadIdx.x;
    if (t >= numTads) return;
    const T *xr = x + xOffsets[t];
    T *zr = z + zOffsets[t];
    const C yt = BYTAD ? toCompute(y[t]) : (C)0;
    const Long f0 = (Long)blockIdx.y;
    for (Long f = f0; f < tadLength; f += gridDim.y) {
        if (MAPPED) {
            const unsigned ff = (unsigned)f;
            zr[mapOffset32(zm, ff)] = fromCompute<T>(F::template apply<C>(toCompute(xr[mapOffset32(xm, ff)]), toCompute(y[mapOffset32(ym, ff)]), p));
        } else {
            C bv = BYTAD ? yt : toCompute(y[f * yEws]);
            zr[f * zEws] = fromCompute<T>(F::template apply<C>(toCompute(xr[f * tadEws]), bv, p));
        }
    }
}

template <typename T, typename F>
__global__ void __launch_bounds__(kBlock) bcGeneralKernel(const T *x, DimMap xm, const T *y, DimMap ym, T *z,
                                                          DimMap zm, const Long *xOffsets, const Long *zOffsets,
                                                          Long tadLength, Long numTads) {
    typedef typename Compute<T>::type C;
    if (F::tables) lm::loadTables();
    Params<T> p{nullptr};
    for (Long r = blockIdx.x; r < numTads; r += gridDim.x) {
        const Long xo = xOffsets[r];
        const Long zo = zOffsets[r];
        for (Long f = threadIdx.x; f < tadLength; f += kBlock) {
            Long ox = xo + mapOffset32(xm, (unsigned)f);
            Long oz = zo + mapOffset32(zm, (unsigned)f);
            Long oy = mapOffset32(ym, (unsigned)f);
            z[oz] = fromCompute<T>(F::template apply<C>(toCompute(x[ox]), toCompute(y[oy]), p));
        }
    }
}

// Offset of the vector that starts `inner` elements into run m (runs of runLength elements, numbered in C order) of a
// map whose innermost dimension is contiguous and holds whole runs.  When a run is that whole dimension - the usual case -
// m counts the outer dimensions directly and the first of them costs no division.
__device__ __forceinline__ Long runOffset(const DimMap &mp, unsigned m, unsigned inner, unsigned runLength) {
    const int last = mp.rank - 1;
    if (last > 0 && mp.shape[last] == runLength) {
        Long off = inner;
        for (int d = last - 1; d > 0; d--) {
            const unsigned q = m / mp.shape[d];
            off += (Long)(m - q * mp.shape[d]) * mp.stride[d];
            m = q;
        }
        return off + (Long)m * mp.stride[0];
    }
    return mapOffset32(mp, m * runLength + inner);
}

// Views that are made of contiguous runs: every operand's index -> offset map ends in a dimension of stride 1 whose extent
// is a multiple of runLength (the padded rows of a view with a pitch; the TADs of a broadcast over several dimensions).
// The element space is cut into units of one 16-byte vector inside a run (the last unit of a run is shorter when
// runLength is not a multiple of the vector width); a thread takes a unit, finds its place through each operand's map
// once - divisions per vector, not per element - and moves it with 16-byte accesses that need no alignment beyond the
// element's own; the next unit's loads are issued before the current one is worked on.  xOffsets / zOffsets (null: one
// "TAD" at offset 0) add a per-TAD offset, y is shared by all TADs.  Units are numbered run by run inside a TAD
// (runMajor 0), or with the same run of all TADs side by side (runMajor 1): whichever makes neighbouring threads touch
// neighbouring memory.  perRun divides by the units of a run, second by the TAD count (runMajor) or the runs of a TAD;
// both serve totals below 2^31 units, larger ones take 64-bit divisions.
template <typename T, typename F, int U>
__global__ void __launch_bounds__(kBlock) ewRunsKernel(const T *x, DimMap xm, const T *y, DimMap ym, T *z, DimMap zm,
                                                       const Long *xOffsets, const Long *zOffsets, Params<T> p, unsigned total,
                                                       unsigned runLength, int runMajor, FastDiv perRun, FastDiv second,
                                                       unsigned unitStep, unsigned runStep) {
    typedef typename Compute<T>::type C;
    constexpr int VEC = Pack<T>::N;
    constexpr bool two = F::nin == 2;
    // (everything that numbers units is 32-bit - the host sends calls of 2^31 units or more elsewhere: with 64-bit
    // counters and the divisions they bring, a wave spent 200 instructions of its compute unit's one scalar unit on a
    // single vector)
    const unsigned step = gridDim.x * kBlock;
    const unsigned unitsPerRun = perRun.d;
    // A thread's units lie `step` apart: the first one's run t (counted over all TADs) and place c in it come from a
    // division, the later ones from adding step / unitsPerRun and step % unitsPerRun (unitStep, runStep: from the host).
    unsigned g = blockIdx.x * kBlock + threadIdx.x;
    unsigned c, t;
    t = perRun.divmod(g, c);
    auto advance = [&]() {
        g += step;
        c += unitStep;
        t += runStep;
        if (c >= unitsPerRun) { c -= unitsPerRun; t++; }
    };
    // run t -> (TAD r, run m of the TAD)
    auto split = [&](unsigned run, unsigned &r, unsigned &m) {
        unsigned rem;
        const unsigned q = second.divmod(run, rem);
        if (runMajor) { m = q; r = rem; }
        else { r = q; m = rem; }
    };
    if constexpr (U > 1) {
        // With offset tables a unit costs two trips to memory, one after the other (its TAD's offsets, then its vectors): U
        // units per thread go through each stage together, so that what is in flight stays ahead of the memory's latency.
        if (F::tables) lm::loadTables();
        const bool shortRuns = runLength % VEC != 0;  // some units hold fewer elements than a vector
        while (g < total) {
            unsigned m[U], first[U];
            Long xo[U], zo[U];
            bool live[U];
            // (a unit beyond the end is placed on the array's first one, so that no load sits in a branch of its own - the
            // compiler would make each such load wait for those before it - and is neither worked on nor stored)
#pragma unroll
            for (int k = 0; k < U; k++) {
                live[k] = g < total;
                unsigned r;
                split(live[k] ? t : 0, r, m[k]);
                first[k] = live[k] ? c * VEC : 0;
                xo[k] = xOffsets != nullptr ? xOffsets[r] : 0;
                zo[k] = zOffsets != nullptr ? zOffsets[r] : 0;
                const unsigned before = g;
                advance();
                if (g < before) g = total;  // (the 32-bit sum wrapped round: past the end)
            }
            const T *xp[U], *yp[U];
            T *zp[U];
            Pack<T> a[U], b[U];
            bool whole[U];
#pragma unroll
            for (int k = 0; k < U; k++) {
                xp[k] = x + xo[k] + runOffset(xm, m[k], first[k], runLength);
                zp[k] = z + zo[k] + runOffset(zm, m[k], first[k], runLength);
                if (two) yp[k] = y + runOffset(ym, m[k], first[k], runLength);
                whole[k] = !shortRuns || runLength - first[k] >= (unsigned)VEC;
                if (!shortRuns) {
                    a[k] = streamPackAnywhere(xp[k]);
                    if (two) b[k] = loadPackAnywhere(yp[k]);
                } else if (whole[k]) {
                    a[k] = streamPackAnywhere(xp[k]);
                    if (two) b[k] = loadPackAnywhere(yp[k]);
                }
                whole[k] = whole[k] && live[k];
            }
#pragma unroll
            for (int k = 0; k < U; k++) {
                if (whole[k]) {
                    Pack<T> o;
#pragma unroll
                    for (int e = 0; e < VEC; e++)
                        o.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a[k].v[e]), two ? toCompute(b[k].v[e]) : (C)0, p));
                    streamPackAnywhere(zp[k], o);
                } else if (live[k]) {
                    const unsigned count = runLength - first[k];
                    for (unsigned e = 0; e < count; e++)
                        zp[k][e] = fromCompute<T>(F::template apply<C>(toCompute(xp[k][e]), two ? toCompute(yp[k][e]) : (C)0, p));
                }
            }
        }
        return;
    }
    const T *xp = nullptr, *yp = nullptr;
    T *zp = nullptr;
    unsigned count = 0;
    Pack<T> a, b;
    // the three addresses of the unit the walk stands on; requests the unit's vectors
    auto fetch = [&](const T *&ux, const T *&uy, T *&uz, unsigned &ucount, Pack<T> &ua, Pack<T> &ub) {
        unsigned r, m;
        split(t, r, m);
        ucount = runLength - c * VEC;  // elements left in the run from the unit's first one on
        ux = x + (xOffsets != nullptr ? xOffsets[r] : 0) + runOffset(xm, m, c * VEC, runLength);
        uz = z + (zOffsets != nullptr ? zOffsets[r] : 0) + runOffset(zm, m, c * VEC, runLength);
        if (two) uy = y + runOffset(ym, m, c * VEC, runLength);
        if (ucount >= (unsigned)VEC) {
            ua = streamPackAnywhere(ux);
            if (two) ub = loadPackAnywhere(uy);  // through the caches: every TAD reads it again
        }
    };
    bool have = g < total;
    if (have) fetch(xp, yp, zp, count, a, b);
    if (F::tables) lm::loadTables();  // staged while the first vectors are on their way
    while (have) {
        const unsigned before = g;
        advance();
        const bool haveNext = g < total && g > before;
        const T *nxp = nullptr, *nyp = nullptr;
        T *nzp = nullptr;
        unsigned ncount = 0;
        Pack<T> na, nb;
        if (haveNext) fetch(nxp, nyp, nzp, ncount, na, nb);
        if (count >= (unsigned)VEC) {
            Pack<T> o;
#pragma unroll
            for (int e = 0; e < VEC; e++)
                o.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a.v[e]), two ? toCompute(b.v[e]) : (C)0, p));
            streamPackAnywhere(zp, o);
        } else {
            for (unsigned e = 0; e < count; e++)
                zp[e] = fromCompute<T>(F::template apply<C>(toCompute(xp[e]), two ? toCompute(yp[e]) : (C)0, p));
        }
        have = haveNext;
        xp = nxp; yp = nyp; zp = nzp; count = ncount; a = na; b = nb;
    }
}

// The plainest of those views: a matrix whose rows lie a pitch apart, one run per row, the same for every operand (a
// pitch of 0 repeats y's one row).  Unit g is vector g % unitsPerRun of row g / unitsPerRun: one multiplication in place of
// a division and three pointer sums, a third of the instructions the general walk spends on a unit.
template <typename T, typename F>
__global__ void __launch_bounds__(kBlock) ewPitchKernel(const T *x, Long px, const T *y, Long py, T *z, Long pz, Params<T> p,
                                                        unsigned total, unsigned runLength, FastDiv perRun) {
    typedef typename Compute<T>::type C;
    constexpr int VEC = Pack<T>::N;
    constexpr bool two = F::nin == 2;
    if (F::tables) lm::loadTables();
    const unsigned step = gridDim.x * kBlock;
    const bool shortRuns = runLength % VEC != 0;  // some units hold fewer elements than a vector
    for (unsigned g = blockIdx.x * kBlock + threadIdx.x; g < total;) {
        unsigned c;
        const unsigned r = perRun.divmod(g, c);
        const unsigned first = c * VEC, count = runLength - first;
        const T *xp = x + (Long)r * px + first;
        const T *yp = two ? y + (Long)r * py + first : nullptr;
        T *zp = z + (Long)r * pz + first;
        if (!shortRuns || count >= (unsigned)VEC) {
            const Pack<T> a = streamPackAnywhere(xp);
            Pack<T> b;
            if (two) b = loadPackAnywhere(yp);  // through the caches: a repeated row is read again and again
            Pack<T> o;
#pragma unroll
            for (int e = 0; e < VEC; e++)
                o.v[e] = fromCompute<T>(F::template apply<C>(toCompute(a.v[e]), two ? toCompute(b.v[e]) : (C)0, p));
            streamPackAnywhere(zp, o);
        } else {
            for (unsigned e = 0; e < count; e++)
                zp[e] = fromCompute<T>(F::template apply<C>(toCompute(xp[e]), two ? toCompute(yp[e]) : (C)0, p));
        }
        const unsigned before = g;
        g += step;
        if (g < before) break;  // (the 32-bit sum wrapped round: past the end)
    }
}

// ---------------------------------------------------------------------------------------------------
// Host-side launch helpers.

inline int gridFor(Long work, Long perBlock, int cap) {
    Long g = (work + perBlock - 1) / perBlock;
    if (g < 1) g = 1;
    if (g > cap) g = cap;
    return (int)g;
}

static constexpr int kGridCap = 256 * 32;  // 32 blocks of 256 threads per CU
// Blocks of the contiguous element-wise kernel when the functor stages lookup tables (every block stages them once and
// then walks its share in passes): exp over 2^26 floats 90 us with 8192 blocks, 86.5 with 16384, 90 with 32768, 108 with
// a block per pass.
static constexpr int kTableGridCap = 256 * 64;
static constexpr int kMaxGrid = (1 << 24) - 1;  // blocks of 256 threads: a launch may not exceed 2^32 threads in all

// Returns the number of leading scalar elements that brings every pointer to a 16-byte boundary, or -1
// when the pointers do not share one misalignment.
template <typename T> inline int commonHead(const void *a, const void *b, const void *c) {
    uintptr_t pa = (uintptr_t)a, pb = b ? (uintptr_t)b : pa, pc = c ? (uintptr_t)c : pa;
    if ((pa & 15) != (pb & 15) || (pa & 15) != (pc & 15)) return -1;
    if ((pa & (sizeof(T) - 1)) != 0) return -1;
    return (int)(((16 - (pa & 15)) & 15) / sizeof(T));
}

// The most units (vectors inside runs) a call of ewRunsKernel may have, and their number for `numTads` TADs of tadLength
// elements in runs of runLength; callers send larger calls to the element-wise kernels.
static constexpr Long kMaxRunUnits = 0x7fffffffLL;
template <typename T> inline Long runUnits(Long numTads, Long tadLength, unsigned runLength) {
    const Long perTad = tadLength / runLength * ((runLength + Pack<T>::N - 1) / Pack<T>::N);
    if (perTad <= 0 || numTads > kMaxRunUnits / perTad) return kMaxRunUnits + 1;
    return numTads * perTad;
}
// grid and divisors of ewRunsKernel; OFFSETS: the call carries per-TAD offset tables (a compile-time choice, so that each
// family builds only the form it launches)
template <typename T, typename F, bool OFFSETS, int UNITS = 0>
inline void launchRuns(hipStream_t s, const T *x, const DimMap &xm, const T *y, const DimMap &ym, T *z, const DimMap &zm,
                       const Long *xOffsets, const Long *zOffsets, Params<T> p, Long numTads, Long tadLength, unsigned runLength,
                       bool runMajor) {
    const unsigned unitsPerRun = (runLength + Pack<T>::N - 1) / Pack<T>::N;
    const Long runsPerTad = tadLength / runLength;
    const Long units = runUnits<T>(numTads, tadLength, runLength);
    const FastDiv perRun(unitsPerRun);
    const FastDiv second((unsigned)(runMajor ? numTads : runsPerTad));
    // with offset tables: two units per thread and round (one: 54-63 % of the HBM peak on a [256,1024,256] array broadcast
    // along dimensions {0,2}, two: 68 %, four: 60 %), and so for functors with lookup tables, whose capped grid gives a
    // thread several rounds (exp over rows with a pitch: 56 -> 62 %); otherwise one unit per thread
    constexpr int U = UNITS > 0 ? UNITS : ((OFFSETS || F::tables) ? 2 : 1);
    if (!OFFSETS && numTads == 1 && xOffsets == nullptr && zOffsets == nullptr) {
        // rows with a pitch, y (if any) one repeated row: the plain kernel (a row added to [65536, 1024] floats with a pitch of
        // 1032: 69 -> 74 % of the HBM peak, exp over them 61 -> 71.5 %; with a y of rows of its own the general walk is
        // ahead, 79 % against 77 %, and keeps the call)
        auto pitched = [&](const DimMap &m) { return m.rank == 2 && m.shape[1] == runLength && m.stride[1] == 1; };
        if (pitched(xm) && pitched(zm) && (F::nin != 2 || (pitched(ym) && ym.stride[0] == 0))) {
            // (functors with lookup tables on up to 24576 blocks, a thread going round for the rest: exp over the 2^26 floats
            // of such rows 71.5 % of the HBM peak; 65 / 70 / 71.4 / 68.5 / 66 % on 8192 / 16384 / 32768 / 40960 / 49152 blocks,
            // 58 % uncapped, 64-67 % with two units per thread and round)
            const unsigned grid = gridFor(units, kBlock, F::tables ? 256 * 96 : kMaxGrid);
            ND4J_LAUNCH((ewPitchKernel<T, F>), dim3(grid), dim3(kBlock), 0, s, x, xm.stride[0], y, (Long)0, z, zm.stride[0], p,
                        (unsigned)units, runLength, perRun);
            return;
        }
    }
    const unsigned grid = gridFor(units, kBlock * U, F::tables ? kGridCap : kMaxGrid);
    const unsigned long long step = (unsigned long long)grid * kBlock;  // at most 2^32 - 256
    const unsigned unitStep = (unsigned)(step % unitsPerRun), runStep = (unsigned)(step / unitsPerRun);
    ND4J_LAUNCH((ewRunsKernel<T, F, U>), dim3(grid), dim3(kBlock), 0, s, x, xm, y, ym, z, zm, xOffsets, zOffsets, p,
                       (unsigned)units, runLength, runMajor ? 1 : 0, perRun, second, unitStep, runStep);
}

template <typename T, typename F>
inline void launchStrided(hipStream_t s, const T *x, Long xs, const T *y, Long ys, T *z, Long zs, const T *extra, Long n,
                          typename Compute<T>::type scalar = 0) {
    if (n <= 0) return;
    Params<T> p{extra};
    p.scalar = scalar;
    const bool two = F::nin == 2;
    const bool contig = xs == 1 && zs == 1 && (!two || ys == 1 || ys == 0);
    if (contig) {
        int head = commonHead<T>(x, (two && ys == 1) ? (const void *)y : nullptr, z);
        if (head >= 0) {
            if (head > n) head = (int)n;
            Long nvec = (n - head) / Pack<T>::N;
            // kernels that stage the lookup tables run several passes per block, so the staging is paid less often
            int grid = gridFor(nvec > 0 ? nvec : 1, (Long)kBlock, F::tables ? kTableGridCap : kMaxGrid);
            // one operand: two passes per thread (a little better for the functors with some arithmetic to overlap - tanh
            // 89 -> 82 us per 2^26 - and no worse for copies); with two operands one pass per thread stays the faster
            if (!two && !F::tables && grid > 2) grid = (grid + 1) / 2;
            // Two operands: blocks of 128 threads (z = x + y over 2^26 floats 123.6 -> 119.1 us against 256, the same with 64,
            // 124.4 with 192; one-operand calls measure the same with either).  The kernel takes its block size from the
            // launch; the functors that stage lookup tables keep the 256 threads their staging is written for.
            int blk = kBlock;
            if (two && !F::tables) {
                blk = kBlock / 2;
                grid = gridFor(nvec > 0 ? nvec : 1, (Long)blk, kMaxGrid);
            }
            ND4J_LAUNCH((ewVecKernel<T, F>), dim3(grid), dim3(blk), 0, s, x, two ? y : x, z, p, n, head,
                               (two && ys == 0) ? 1 : 0);
            return;
        }
    }
    DimMap xm, ym, zm;
    xm.rank = ym.rank = zm.rank = 1;
    xm.shape[0] = ym.shape[0] = zm.shape[0] = (unsigned)(n > 0xffffffffLL ? 0xffffffffu : n);
    xm.stride[0] = xs; ym.stride[0] = ys; zm.stride[0] = zs;
    int grid = gridFor(n, kBlock * 4, kGridCap);
    ND4J_LAUNCH((ewGeneralKernel<T, F>), dim3(grid), dim3(kBlock), 0, s, x, xm, two ? y : x, ym, z, zm, p, n);
}

// Dense matrices in mixed orders (z = op(x, y) with x or y laid out the other way round than z: a + b.transpose()): in
// z's frame z[r * cols + c]; an operand of z's order is read where z is written, a transposed one, t[r + c * rows], goes
// through an LDS tile - read with the lanes along r, where it is contiguous, used with the lanes along c.  Tiles and
// block order as in the transposing copy (32 x 64, neighbouring blocks on neighbouring column tiles); ACC elements per
// access (a 16-byte vector, or 1 when shapes or alignment do not allow vectors).
template <typename T, typename F, int ACC, bool XT, bool YT>
__global__ void __launch_bounds__(kBlock) ewMixedOrderKernel(const T *x, const T *y, T *z, Long rows, Long cols, Params<T> p) {
    typedef typename Compute<T>::type C;
    constexpr int TR = 32, TC = 64;
    constexpr bool two = F::nin == 2;
    __shared__ T tileX[XT ? TC : 1][TR + 1];
    __shared__ T tileY[(two && YT) ? TC : 1][TR + 1];
    if (F::tables) lm::loadTables();
    constexpr int LANES_R = TR / ACC, STEP_R = kBlock / LANES_R;
    constexpr int LANES_C = TC / ACC, STEP_C = kBlock / LANES_C;
    const int rFast = (threadIdx.x % LANES_R) * ACC, rSlow = threadIdx.x / LANES_R;
    const int cFast = (threadIdx.x % LANES_C) * ACC, cSlow = threadIdx.x / LANES_C;
    const Long colTiles = (cols + TC - 1) / TC, rowTiles = (rows + TR - 1) / TR;
    for (Long tile_ = blockIdx.x; tile_ < colTiles * rowTiles; tile_ += gridDim.x) {
        const Long rt = tile_ / colTiles, ct = tile_ - rt * colTiles;
        const Long r0 = rt * TR, c0 = ct * TC;
        if (XT || (two && YT)) {
#pragma unroll
            for (int lc = rSlow; lc < TC; lc += STEP_R) {
                const Long r = r0 + rFast, c = c0 + lc;
                if (r < rows && c < cols) {
                    if (XT) {
                        if (ACC > 1) {
                            const Pack<T> v = loadPack(reinterpret_cast<const Pack<T> *>(x + r + c * rows));
#pragma unroll
                            for (int k = 0; k < ACC; k++) tileX[lc][rFast + k] = v.v[k % Pack<T>::N];
                        } else {
                            tileX[lc][rFast] = x[r + c * rows];
                        }
                    }
                    if (two && YT) {
                        if (ACC > 1) {
                            const Pack<T> v = loadPack(reinterpret_cast<const Pack<T> *>(y + r + c * rows));
#pragma unroll
                            for (int k = 0; k < ACC; k++) tileY[lc][rFast + k] = v.v[k % Pack<T>::N];
                        } else {
                            tileY[lc][rFast] = y[r + c * rows];
                        }
                    }
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int lr = cSlow; lr < TR; lr += STEP_C) {
            const Long r = r0 + lr, c = c0 + cFast;
            if (r < rows && c < cols) {
                const Long at = r * cols + c;
                if (ACC > 1) {
                    Pack<T> xa, ya, o;
                    if (!XT) xa = loadPack(reinterpret_cast<const Pack<T> *>(x + at));
                    if (two && !YT) ya = loadPack(reinterpret_cast<const Pack<T> *>(y + at));
#pragma unroll
                    for (int k = 0; k < ACC; k++) {
                        const C a = toCompute(XT ? tileX[cFast + k][lr] : xa.v[k % Pack<T>::N]);
                        const C b = two ? toCompute(YT ? tileY[cFast + k][lr] : ya.v[k % Pack<T>::N]) : (C)0;
                        o.v[k % Pack<T>::N] = fromCompute<T>(F::template apply<C>(a, b, p));
                    }
                    storePack(reinterpret_cast<Pack<T> *>(z + at), o);
                } else {
                    const C a = toCompute(XT ? tileX[cFast][lr] : x[at]);
                    const C b = two ? toCompute(YT ? tileY[cFast][lr] : y[at]) : (C)0;
                    z[at] = fromCompute<T>(F::template apply<C>(a, b, p));
                }
            }
        }
        if (XT || (two && YT)) __syncthreads();
    }
}

// 0: contiguous along dimension 1 (c-like), 1: along dimension 0 (f-like), -1: neither, for a rank-2 map
inline int denseClass2D(const DimMap &m) {
    if (m.rank != 2) return -1;
    if (m.stride[1] == 1 && m.stride[0] == (Long)m.shape[1]) return 0;
    if (m.stride[0] == 1 && m.stride[1] == (Long)m.shape[0]) return 1;
    return -1;
}

template <typename T, typename F, int ACC>
inline void launchMixedOrder(hipStream_t s, const T *x, const T *y, T *z, Long rows, Long cols, bool xt, bool yt, Params<T> p) {
    const Long tiles = ((rows + 31) / 32) * ((cols + 63) / 64);
    const dim3 grid((unsigned)(tiles < kMaxGrid ? tiles : kMaxGrid));
    if constexpr (F::nin == 2) {
        if (xt && yt) ND4J_LAUNCH((ewMixedOrderKernel<T, F, ACC, true, true>), grid, dim3(kBlock), 0, s, x, y, z, rows, cols, p);
        else if (xt) ND4J_LAUNCH((ewMixedOrderKernel<T, F, ACC, true, false>), grid, dim3(kBlock), 0, s, x, y, z, rows, cols, p);
        else ND4J_LAUNCH((ewMixedOrderKernel<T, F, ACC, false, true>), grid, dim3(kBlock), 0, s, x, y, z, rows, cols, p);
    } else {
        (void)yt;  // one input: it is the transposed one
        ND4J_LAUNCH((ewMixedOrderKernel<T, F, ACC, true, false>), grid, dim3(kBlock), 0, s, x, y, z, rows, cols, p);
    }
}

template <typename T, typename F>
inline void launchGeneral(hipStream_t s, const T *x, const DimMap &xm, const T *y, const DimMap &ym, T *z,
                          const DimMap &zm, const T *extra, Long n, typename Compute<T>::type scalar = 0) {
    if (n <= 0) return;
    const bool two = F::nin == 2;
    if (xm.rank == 1 && zm.rank == 1 && (!two || ym.rank == 1)) {
        launchStrided<T, F>(s, x, xm.stride[0], y, two ? ym.stride[0] : 0, z, zm.stride[0], extra, n, scalar);
        return;
    }
    // dense matrices of one shape whose orders differ
    const int zc = denseClass2D(zm), xc = denseClass2D(xm), yc = two ? denseClass2D(ym) : zc;
    if (zc >= 0 && xc >= 0 && yc >= 0 && xm.shape[0] == zm.shape[0] && xm.shape[1] == zm.shape[1] &&
        (!two || (ym.shape[0] == zm.shape[0] && ym.shape[1] == zm.shape[1])) && (xc != zc || yc != zc) &&
        (Long)zm.shape[0] * zm.shape[1] == n) {
        // z's frame: c runs along z's contiguous dimension
        const Long cols = zm.shape[zc == 0 ? 1 : 0], rows = zm.shape[zc == 0 ? 0 : 1];
        Params<T> p{extra};
        p.scalar = scalar;
        constexpr int N = Pack<T>::N;
        const bool vec = rows % N == 0 && cols % N == 0 &&
                         ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(z) | (two ? reinterpret_cast<uintptr_t>(y) : 0)) & 15) == 0;
        if (vec) launchMixedOrder<T, F, N>(s, x, two ? y : x, z, rows, cols, xc != zc, two && yc != zc, p);
        else launchMixedOrder<T, F, 1>(s, x, two ? y : x, z, rows, cols, xc != zc, two && yc != zc, p);
        return;
    }
    Params<T> p{extra};
    p.scalar = scalar;
    // rows with a pitch and the like: contiguous runs along the innermost dimension of every operand
    const DimMap *const maps[3] = {&xm, two ? &ym : nullptr, &zm};
    const unsigned run = commonRunLength(maps);
    if (run >= (unsigned)Pack<T>::N && n <= 0x7fffffffLL && runUnits<T>(1, n, run) <= kMaxRunUnits) {
        launchRuns<T, F, false>(s, x, xm, two ? y : x, two ? ym : xm, z, zm, nullptr, nullptr, p, 1, n, run, false);
        return;
    }
    int grid = gridFor(n, kBlock * 4, kGridCap);
    ND4J_LAUNCH((ewGeneralKernel<T, F>), dim3(grid), dim3(kBlock), 0, s, x, xm, two ? y : x, two ? ym : xm, z, zm,
                       p, n);
}

// Compile-time opNum dispatch: calls Body<I>::run(args...) for I == op, returns false if no I matches
// or the op has no functor.
template <template <int> class Body, int... Is, typename... A>
inline bool dispatchSeq(int op, std::integer_sequence<int, Is...>, A &&...a) {
    return ((op == Is ? Body<Is>::run(std::forward<A>(a)...) : false) || ...);
}

}  // namespace nd4j_amd
