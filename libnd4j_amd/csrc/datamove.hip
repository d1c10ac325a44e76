// Data-movement specials: concat, pullRows, tear, shuffle and the float-type conversions.  (flatten needs no
// kernel of its own: the host turns it into an Identity transform between two index maps.)
// Reference: include/loops/special_kernels.h:140-360 (concat), 579-625 (pullRows), 824-874 (tear), 890-967
// (shuffle), include/loops/type_conversions.h:38-49 (convert); CPU counterparts include/ops/impl/specials.cpp:17-200
// and blas/cpu/NativeOps.cpp:2045-2160, 2266-2325.
//
// As in the reference's CUDA back end every pointer these calls receive - data, shapeInfo, TAD tables, and the
// tables of such pointers - is a device pointer, so the kernels decode shapeInfo themselves.  All of them are pure
// copies: 16-byte streaming accesses wherever source and destination runs are contiguous and equally aligned.
#include <type_traits>

#include "elementwise.cuh"
#include "launch.h"
#include "reduce_engine.cuh"

namespace nd4j_amd {

// ---- shapeInfo on the device: [rank, shape.., stride.., offset, ews, order] --------------------------------
__device__ __forceinline__ int dRank(const Long *si) { return (int)si[0]; }
__device__ __forceinline__ const Long *dShape(const Long *si) { return si + 1; }
__device__ __forceinline__ const Long *dStride(const Long *si) { return si + 1 + si[0]; }
__device__ __forceinline__ Long dEws(const Long *si) { return si[2 * si[0] + 2]; }
__device__ __forceinline__ char dOrder(const Long *si) { return (char)si[2 * si[0] + 3]; }
__device__ __forceinline__ Long dLength(const Long *si) {
    Long n = 1;
    for (int i = 0; i < (int)si[0]; i++) n *= si[1 + i];
    return n;
}
// element offset of linear index i decomposed over the shape in C order / in F order (shape::ind2subC / ind2sub
// followed by shape::getOffset)
__device__ __forceinline__ Long dOffsetC(const Long *si, Long i) {
    const int rank = dRank(si);
    const Long *shape = dShape(si), *stride = dStride(si);
    Long off = 0;
    for (int d = rank - 1; d >= 0; d--) {
        const Long q = i / shape[d];
        off += (i - q * shape[d]) * stride[d];
        i = q;
    }
    return off;
}
__device__ __forceinline__ Long dOffsetF(const Long *si, Long i) {
    const int rank = dRank(si);
    const Long *shape = dShape(si), *stride = dStride(si);
    Long off = 0;
    for (int d = 0; d < rank; d++) {
        const Long q = i / shape[d];
        off += (i - q * shape[d]) * stride[d];
        i = q;
    }
    return off;
}

template <typename T> __device__ __forceinline__ bool sameAlignment(const T *a, const T *b) {
    const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
    return (pa & 15) == (pb & 15) && (pa & (sizeof(T) - 1)) == 0;
}

// `lanes` cooperating lanes copy len elements from src to dst.  se / de: element-wise strides (>= 1) or, when
// either is < 1, offsets come from the coordinate decomposition of the two shapeInfos (FORDER: ind2sub, else ind2subC).
template <typename T, bool FORDER>
__device__ __forceinline__ void copyRun(const T *src, Long se, const Long *sInfo, T *dst, Long de, const Long *dInfo, Long len,
                                        int lane, int lanes) {
    if (se == 1 && de == 1) {
        constexpr int N = Pack<T>::N;
        if (sameAlignment(src, dst)) {
            Long head = (Long)(((16 - (reinterpret_cast<uintptr_t>(src) & 15)) & 15) / sizeof(T));
            if (head > len) head = len;
            for (Long i = lane; i < head; i += lanes) dst[i] = src[i];
            const Long nvec = (len - head) / N;
            const Pack<T> *sv = reinterpret_cast<const Pack<T> *>(src + head);
            Pack<T> *dv = reinterpret_cast<Pack<T> *>(dst + head);
            Long v = lane;
            for (; v + 3 * (Long)lanes < nvec; v += 4 * (Long)lanes) {
                Pack<T> p0 = loadPack(sv + v), p1 = loadPack(sv + v + lanes), p2 = loadPack(sv + v + 2 * lanes),
                        p3 = loadPack(sv + v + 3 * lanes);
                storePack(dv + v, p0);
                storePack(dv + v + lanes, p1);
                storePack(dv + v + 2 * lanes, p2);
                storePack(dv + v + 3 * lanes, p3);
            }
            for (; v < nvec; v += lanes) storePack(dv + v, loadPack(sv + v));
            for (Long i = head + nvec * N + lane; i < len; i += lanes) dst[i] = src[i];
        } else {
            for (Long i = lane; i < len; i += lanes) dst[i] = src[i];
        }
    } else if (se >= 1 && de >= 1) {
        for (Long i = lane; i < len; i += lanes) dst[i * de] = src[i * se];
    } else {
        for (Long i = lane; i < len; i += lanes)
            dst[FORDER ? dOffsetF(dInfo, i) : dOffsetC(dInfo, i)] = src[FORDER ? dOffsetF(sInfo, i) : dOffsetC(sInfo, i)];
    }
}

// A block works on one long TAD, on four shorter ones (a wave each) or on sixteen short ones, sized so that a lane
// keeps about four 16-byte vectors in flight
template <typename T> __device__ __forceinline__ int lanesPerTad(Long tadLength, bool wide = false) {
    const Long vectors = tadLength / Pack<T>::N;
    // (wide: a vector per lane from 256 vectors on - rows of 1024 floats torn into buffers of their own: 88 -> 85 us;
    // the same rows gathered or swapped in place: 95 -> 127 us, so those keep a wave per row)
    if (wide) return vectors >= 256 ? kBlock : (vectors >= 64 ? kWave : 16);
    return vectors >= 1024 ? kBlock : (vectors >= 256 ? kWave : 16);
}

// ---- pullRows: z TAD idx <- x TAD indexes[idx] ---------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(kBlock) pullRowsKernel(const T *x, T *z, Long n, const Long *indexes, const Long *tadInfo,
                                                         const Long *tadOffsets, const Long *zTadInfo, const Long *zTadOffsets) {
    const Long tadLength = dLength(tadInfo);
    const Long xe = dEws(tadInfo), ze = dEws(zTadInfo);
    const int lanes = lanesPerTad<T>(tadLength), groups = kBlock / lanes;
    const int g = threadIdx.x / lanes, lane = threadIdx.x % lanes;
    if (lanes == kBlock && xe == 1 && ze == 1) {
        // long contiguous TADs are cut into pieces of four vectors per lane, so that a few long rows still fill the chip
        const Long piece = (Long)kBlock * 4 * Pack<T>::N;
        const Long pieces = (tadLength + piece - 1) / piece;
        for (Long u = blockIdx.x; u < n * pieces; u += gridDim.x) {
            const Long idx = u / pieces, f0 = (u - idx * pieces) * piece;
            const Long len = tadLength - f0 < piece ? tadLength - f0 : piece;
            copyRun<T, false>(x + tadOffsets[indexes[idx]] + f0, 1, tadInfo, z + zTadOffsets[idx] + f0, 1, zTadInfo, len, lane, lanes);
        }
        return;
    }
    for (Long idx = (Long)blockIdx.x * groups + g; idx < n; idx += (Long)gridDim.x * groups)
        copyRun<T, false>(x + tadOffsets[indexes[idx]], xe, tadInfo, z + zTadOffsets[idx], ze, zTadInfo, tadLength, lane, lanes);
}

// ---- tear: target[r] <- x TAD r (the stride-less branch decomposes in F order, as both reference back ends do) ----
template <typename T>
__global__ void __launch_bounds__(kBlock) tearKernel(const T *x, const Long *xInfo, T *const *targets, const Long *zInfo,
                                                     const Long *tadInfo, const Long *tadOffsets) {
    const Long tadLength = dLength(tadInfo);
    const Long numTads = dLength(xInfo) / tadLength;
    const Long xe = dEws(tadInfo), ze = dEws(zInfo);
    const int lanes = lanesPerTad<T>(tadLength, true), groups = kBlock / lanes;
    const int g = threadIdx.x / lanes, lane = threadIdx.x % lanes;
    if (lanes == kBlock && xe == 1 && ze == 1) {
        // long contiguous TADs are cut into pieces of four vectors per lane, so that a few long TADs still fill the chip
        const Long piece = (Long)kBlock * 4 * Pack<T>::N;
        const Long pieces = (tadLength + piece - 1) / piece;
        for (Long u = blockIdx.x; u < numTads * pieces; u += gridDim.x) {
            const Long r = u / pieces, f0 = (u - r * pieces) * piece;
            const Long len = tadLength - f0 < piece ? tadLength - f0 : piece;
            copyRun<T, true>(x + tadOffsets[r] + f0, 1, tadInfo, reinterpret_cast<T *>(targets[r]) + f0, 1, zInfo, len, lane, lanes);
        }
        return;
    }
    for (Long r = (Long)blockIdx.x * groups + g; r < numTads; r += (Long)gridDim.x * groups)
        copyRun<T, true>(x + tadOffsets[r], xe, tadInfo, targets[r], ze, zInfo, tadLength, lane, lanes);
}

// ---- shuffle: TAD r and TAD map[r] of every array trade places (map[r] < 0: leave r alone) -----------------------
// The pairs of one map are disjoint (each TAD appears in at most one pair), which is what makes the reference's
// sequential loop and a parallel one agree.  Values are read from x and written to z; the callers pass z == x.
template <typename T>
__global__ void __launch_bounds__(kBlock) shuffleKernel(T *const *xs, const Long *const *xInfos, T *const *zs, int N,
                                                        const int *map, const Long *const *tadInfos,
                                                        const Long *const *tadOffsets) {
    constexpr int VEC = Pack<T>::N;
    for (int f = blockIdx.y; f < N; f += gridDim.y) {
        const T *x = xs[f];
        T *z = zs[f];
        const Long *ti = tadInfos[f], *off = tadOffsets[f];
        const Long tadLength = dLength(ti);
        const Long numTads = dLength(xInfos[f]) / tadLength;
        const Long ews = dEws(ti);
        const int lanes = lanesPerTad<T>(tadLength), groups = kBlock / lanes;
        const int g = threadIdx.x / lanes, lane = threadIdx.x % lanes;
        for (Long r = (Long)blockIdx.x * groups + g; r < numTads; r += (Long)gridDim.x * groups) {
            const int m = map[r];
            if (m < 0) continue;
            const Long oa = off[r], ob = off[m];
            if (ews == 1 && tadLength % VEC == 0 && (reinterpret_cast<uintptr_t>(x + oa) & 15) == 0 &&
                (reinterpret_cast<uintptr_t>(x + ob) & 15) == 0 && (reinterpret_cast<uintptr_t>(z + oa) & 15) == 0 &&
                (reinterpret_cast<uintptr_t>(z + ob) & 15) == 0) {
                const Pack<T> *xa = reinterpret_cast<const Pack<T> *>(x + oa), *xb = reinterpret_cast<const Pack<T> *>(x + ob);
                Pack<T> *za = reinterpret_cast<Pack<T> *>(z + oa), *zb = reinterpret_cast<Pack<T> *>(z + ob);
                const Long nv = tadLength / VEC;
                Long v = lane;
                for (; v + 3 * (Long)lanes < nv; v += 4 * (Long)lanes) {  // eight loads in flight: a 4 KiB float row per wave in one go
                    Pack<T> a[4], b[4];
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        a[k] = loadPack(xa + v + k * lanes);
                        b[k] = loadPack(xb + v + k * lanes);
                    }
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        storePack(za + v + k * lanes, b[k]);
                        storePack(zb + v + k * lanes, a[k]);
                    }
                }
                for (; v + lanes < nv; v += 2 * (Long)lanes) {  // four loads in flight
                    const Pack<T> a0 = loadPack(xa + v), b0 = loadPack(xb + v), a1 = loadPack(xa + v + lanes), b1 = loadPack(xb + v + lanes);
                    storePack(za + v, b0);
                    storePack(zb + v, a0);
                    storePack(za + v + lanes, b1);
                    storePack(zb + v + lanes, a1);
                }
                for (; v < nv; v += lanes) {
                    const Pack<T> a = loadPack(xa + v), b = loadPack(xb + v);
                    storePack(za + v, b);
                    storePack(zb + v, a);
                }
            } else if (ews >= 1) {
                for (Long i = lane; i < tadLength; i += lanes) {
                    const T a = x[oa + i * ews], b = x[ob + i * ews];
                    z[oa + i * ews] = b;
                    z[ob + i * ews] = a;
                }
            } else {
                for (Long i = lane; i < tadLength; i += lanes) {
                    const Long o = dOffsetC(ti, i);
                    const T a = x[oa + o], b = x[ob + o];
                    z[oa + o] = b;
                    z[ob + o] = a;
                }
            }
        }
    }
}

// ---- concat ----------------------------------------------------------------------------------------------------
// What the copy kernel needs to know about one input, prepared by a one-block kernel so that the copy blocks start
// with a single small load instead of a chain of dependent ones through the tables of pointers and shapeInfos.
struct ConcatDesc {
    const void *data;
    Long length;  // elements of the input
    Long start;   // sum of shape[dim] of the inputs before it
    Long run;     // shape[dim] * inner: elements that stay together in the result
    Long fast;    // 1: C-contiguous input of the result's rank going into a C-contiguous result
};

__global__ void __launch_bounds__(kBlock) concatPrepareKernel(const void *const *data, const Long *const *infos, int n,
                                                              ConcatView v, ConcatDesc *desc) {
    __shared__ Long part[kBlock];
    const int chunk = (n + kBlock - 1) / kBlock;
    const int lo = threadIdx.x * chunk, hi = lo + chunk < n ? lo + chunk : n;
    Long sum = 0;
    for (int f = lo; f < hi; f++) sum += dShape(infos[f])[v.dim];
    part[threadIdx.x] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        Long run = 0;
        for (int t = 0; t < kBlock; t++) {
            const Long p = part[t];
            part[t] = run;
            run += p;
        }
    }
    __syncthreads();
    Long run = part[threadIdx.x];
    for (int f = lo; f < hi; f++) {
        const Long *si = infos[f];
        ConcatDesc d;
        d.data = data[f];
        d.length = dLength(si);
        d.start = run;
        d.run = dShape(si)[v.dim] * v.inner;
        d.fast = (dRank(si) == v.rank && v.zContig && dOrder(si) == 'c' && dEws(si) == 1) ? 1 : 0;
        desc[f] = d;
        run += dShape(si)[v.dim];
    }
}

// Input r (blockIdx.y) is copied into the slab [start, start + shape[dim]) of dimension `dim` of z.  C-contiguous
// inputs into a C-contiguous result move as 16-byte vectors, one per thread: vector j of the input belongs to run
// j / runV and lands zRunV vectors further on for every run.  Other layouts are walked in the input's logical C order.
template <typename T>
__global__ void __launch_bounds__(kBlock) concatKernel(const Long *const *infos, T *z, ConcatView v, const ConcatDesc *desc, int n,
                                                       int inputFastest) {
    constexpr int VEC = Pack<T>::N;
    // inputFastest: neighbouring blocks take the same stretch of different inputs, whose short runs are neighbours in z
    const Long bx = inputFastest ? blockIdx.y : blockIdx.x, gdx = inputFastest ? gridDim.y : gridDim.x;
    const int by = inputFastest ? blockIdx.x : blockIdx.y, gdy = inputFastest ? gridDim.x : gridDim.y;
    for (int r = by; r < n; r += gdy) {
        const ConcatDesc d = desc[r];
        const T *x = reinterpret_cast<const T *>(d.data);
        if (d.fast) {
            const Long zRun = v.dimTotal * v.inner;  // distance between consecutive runs in z
            T *zb = z + d.start * v.inner;
            if (d.run % VEC == 0 && zRun % VEC == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                (reinterpret_cast<uintptr_t>(zb) & 15) == 0) {
                const Long runV = d.run / VEC, zRunV = zRun / VEC, nv = d.length / VEC;
                const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x);
                Pack<T> *zv = reinterpret_cast<Pack<T> *>(zb);
                const bool small = (nv >> 32) == 0;
                // a block moves two vectors per thread, both loads in flight before the first store (eight inputs of 2^23 floats
                // each: 90.1 us; 90.9 with four, 106.9 with one)
                constexpr int STEPS = 2;
                for (Long j0 = bx * (kBlock * STEPS) + threadIdx.x; j0 < nv; j0 += gdx * (kBlock * STEPS)) {
                    Pack<T> a[STEPS];
#pragma unroll
                    for (int k = 0; k < STEPS; k++)
                        if (j0 + k * kBlock < nv) a[k] = loadPack(xv + j0 + k * kBlock);
#pragma unroll
                    for (int k = 0; k < STEPS; k++) {
                        const Long j = j0 + k * kBlock;
                        if (j >= nv) break;
                        const Long o = runV >= nv ? 0 : (small ? (Long)((unsigned)j / (unsigned)runV) : j / runV);
                        storePack(zv + o * zRunV + (j - o * runV), a[k]);
                    }
                }
            } else {
                for (Long i = bx * kBlock + threadIdx.x; i < d.length; i += gdx * kBlock) {
                    const Long o = i / d.run;
                    zb[o * zRun + (i - o * d.run)] = x[i];
                }
            }
        } else {
            const Long *si = infos[r];
            const int rank = dRank(si);
            if (rank != v.rank) continue;
            const Long *shape = dShape(si), *stride = dStride(si);
            for (Long i = bx * kBlock + threadIdx.x; i < d.length; i += gdx * kBlock) {
                Long rem = i, xo = 0, zo = 0;
                for (int dd = rank - 1; dd >= 0; dd--) {
                    const Long q = rem / shape[dd], c = rem - q * shape[dd];
                    xo += c * stride[dd];
                    zo += (c + (dd == v.dim ? d.start : 0)) * v.zStride[dd];
                    rem = q;
                }
                z[zo] = x[xo];
            }
        }
    }
}

// ---- strided copy whose destination stride is the EWS field of a device shapeInfo ---------------------------------
// (flatten with equal orders: the result's shapeInfo is only known on the device, and reading one field of it here
// spares the host a stream synchronisation)
template <typename T>
__global__ void __launch_bounds__(kBlock) copyToEwsKernel(const T *x, Long xe, T *z, const Long *zInfo, Long n) {
    Long ze = dEws(zInfo);
    if (ze < 1) ze = 1;
    // the grid holds one thread per two 16-byte vectors: a plain streaming copy is fastest as very many short blocks
    copyRun<T, false>(x, xe, nullptr, z, ze, nullptr, n, (int)(blockIdx.x * kBlock + threadIdx.x), (int)(gridDim.x * kBlock));
}
template <typename T> void launchCopyToEws(hipStream_t s, const T *x, Long xe, T *z, const Long *zInfo, Long n) {
    if (n <= 0) return;
    // (two vectors per thread, one after the other: 2^26 floats in 83 us against 87 with one and 100 with four)
    ND4J_LAUNCH((copyToEwsKernel<T>), dim3(gridFor(n, (Long)kBlock * Pack<T>::N * 2, 1 << 22)), dim3(kBlock), 0, s, x, xe, z,
                       zInfo, n);
}

// ---- transposing copy: z[r * zRowStride + c] = x[r + c * xColStride] --------------------------------------------
// x is contiguous along r, z along c (an f-order matrix read out in C order, or the other way round).  A block moves
// a TR x TC tile through LDS: it is read with the lanes running along r and written with the lanes running along c,
// so both sides see full-width accesses; ACC elements per access (a 16-byte vector, or 1 when shapes or alignment
// do not allow vectors).  The tile rows are padded by one element, which spreads both access patterns over the banks.
template <typename T, int ACC, int TR, int TC>
__global__ void __launch_bounds__(kBlock) transposeCopyKernel(const T *x, T *z, Long rows, Long cols, Long xColStride,
                                                              Long zRowStride) {
    __shared__ T tile[TC][TR + 1];  // tile[c][r]
    constexpr int LANES_R = TR / ACC, STEP_R = kBlock / LANES_R;  // reading: threads along r, lines of c per pass
    constexpr int LANES_C = TC / ACC, STEP_C = kBlock / LANES_C;  // writing: threads along c, lines of r per pass
    const int rFast = (threadIdx.x % LANES_R) * ACC, rSlow = threadIdx.x / LANES_R;
    const int cFast = (threadIdx.x % LANES_C) * ACC, cSlow = threadIdx.x / LANES_C;
    // Neighbouring blocks take neighbouring column tiles of the same rows: together they complete whole stretches of the
    // result (its rows are contiguous along c) while these are still open in the memory controllers.
    const Long colTiles = (cols + TC - 1) / TC, rowTiles = (rows + TR - 1) / TR;
    for (Long tile_ = blockIdx.x; tile_ < colTiles * rowTiles; tile_ += gridDim.x) {
        const Long rt = tile_ / colTiles, ct = tile_ - rt * colTiles;
        const Long r0 = rt * TR, c0 = ct * TC;
#pragma unroll
        for (int lc = rSlow; lc < TC; lc += STEP_R) {
            const Long r = r0 + rFast, c = c0 + lc;
            if (r < rows && c < cols) {
                const T *src = x + r + c * xColStride;
                if (ACC > 1) {
                    const Pack<T> p = loadPack(reinterpret_cast<const Pack<T> *>(src));
#pragma unroll
                    for (int k = 0; k < ACC; k++) tile[lc][rFast + k] = p.v[k % Pack<T>::N];
                } else {
                    tile[lc][rFast] = src[0];
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int lr = cSlow; lr < TR; lr += STEP_C) {
            const Long r = r0 + lr, c = c0 + cFast;
            if (r < rows && c < cols) {
                T *dst = z + r * zRowStride + c;
                if (ACC > 1) {
                    Pack<T> p;
#pragma unroll
                    for (int k = 0; k < ACC; k++) p.v[k % Pack<T>::N] = tile[cFast + k][lr];
                    storePack(reinterpret_cast<Pack<T> *>(dst), p);
                } else {
                    dst[0] = tile[cFast][lr];
                }
            }
        }
        __syncthreads();
    }
}
template <typename T>
void launchTransposeCopy(hipStream_t s, const T *x, T *z, Long rows, Long cols, Long xColStride, Long zRowStride) {
    if (rows <= 0 || cols <= 0) return;
    constexpr int N = Pack<T>::N;
    // Tile extents in elements: 32 along r (where x is contiguous), 64 along c (where z is).  With neighbouring blocks on
    // neighbouring column tiles, small tiles (8.4 KB of LDS, many blocks per CU) measured best for a [65536,1024] float
    // matrix: 5.8 TB/s, against 5.5 for 64 x 64, 5.4 for 128 x 64, 5.3 for 64 x 128 and 5.2 for 256 x 32.
    constexpr int TR = 32, TC = 64;
    const Long rowTiles = (rows + TR - 1) / TR, colTiles = (cols + TC - 1) / TC;
    const Long tiles = rowTiles * colTiles;
    const dim3 grid((unsigned)(tiles < kMaxGrid ? tiles : kMaxGrid));
    const bool vec = rows % N == 0 && cols % N == 0 && xColStride % N == 0 && zRowStride % N == 0 &&
                     (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(z) & 15) == 0;
    if (vec) ND4J_LAUNCH((transposeCopyKernel<T, N, TR, TC>), grid, dim3(kBlock), 0, s, x, z, rows, cols, xColStride, zRowStride);
    else ND4J_LAUNCH((transposeCopyKernel<T, 1, TR, TC>), grid, dim3(kBlock), 0, s, x, z, rows, cols, xColStride, zRowStride);
}

template <typename T>
void launchPullRows(hipStream_t s, const T *x, T *z, Long n, const Long *indexes, const Long *tadInfo, const Long *tadOffsets,
                    const Long *zTadInfo, const Long *zTadOffsets) {
    if (n <= 0) return;
    // (a launch with few rows gets the full grid: the kernel cuts long rows into pieces, and idle blocks leave at once)
    ND4J_LAUNCH((pullRowsKernel<T>), dim3(n >= kGridCap ? gridFor(n, 1, kGridCap * 4) : kGridCap), dim3(kBlock), 0, s, x, z, n,
                       indexes, tadInfo, tadOffsets, zTadInfo, zTadOffsets);
}
template <typename T>
void launchTear(hipStream_t s, const T *x, const Long *xInfo, T *const *targets, const Long *zInfo, const Long *tadInfo,
                const Long *tadOffsets, Long numTadsHint) {
    ND4J_LAUNCH((tearKernel<T>), dim3(gridFor(numTadsHint > 0 ? numTadsHint : kGridCap, 1, kGridCap * 4)), dim3(kBlock), 0, s,
                       x, xInfo, targets, zInfo, tadInfo, tadOffsets);
}
template <typename T>
void launchShuffle(hipStream_t s, T *const *xs, const Long *const *xInfos, T *const *zs, int N, const int *map,
                   const Long *const *tadInfos, const Long *const *tadOffsets, Long numTadsHint) {
    if (N <= 0) return;
    const int gy = N < 64 ? N : 64;
    ND4J_LAUNCH((shuffleKernel<T>), dim3(gridFor(numTadsHint > 0 ? numTadsHint : 4096, 1, kGridCap), gy), dim3(kBlock), 0, s,
                       xs, xInfos, zs, N, map, tadInfos, tadOffsets);
}
template <typename T>
void launchConcat(hipStream_t s, const T *const *data, const Long *const *infos, T *z, const ConcatView &v, int n, Long maxLength,
                  void *scratch) {
    if (n <= 0) return;
    ConcatDesc *desc = reinterpret_cast<ConcatDesc *>(scratch);
    ND4J_LAUNCH(concatPrepareKernel, dim3(1), dim3(kBlock), 0, s, reinterpret_cast<const void *const *>(data), infos, n, v, desc);
    const int gy = n < 65535 ? n : 65535;
    // two 16-byte vectors per thread while that keeps the grid below 2^22 blocks
    int budget = (1 << 22) / gy;
    if (budget < 1) budget = 1;
    const int gx = gridFor(maxLength > 0 ? maxLength : 1, (Long)kBlock * 2 * Pack<T>::N, budget);
    // Short runs (the inputs' slabs alternate in z every few KB): blocks that run together should fill neighbouring
    // runs, so the input index varies fastest.  Long runs: one input after the other.
    const bool inputFastest = v.dim > 0 && n > 1 && gx <= 65535;
    if (inputFastest) ND4J_LAUNCH((concatKernel<T>), dim3(gy, gx), dim3(kBlock), 0, s, infos, z, v, desc, n, 1);
    else ND4J_LAUNCH((concatKernel<T>), dim3(gx, gy), dim3(kBlock), 0, s, infos, z, v, desc, n, 0);
}
size_t concatScratchBytes(int numArrays) { return (size_t)(numArrays > 0 ? numArrays : 1) * sizeof(ConcatDesc); }

// ---- accumulate / average: z[i] = sum_k x[k][i] (/ n), optionally written back to every x[k] ------------------------
// (special_kernels.h:700-822).  x is a device table of n device pointers.  The sum runs in the compute type, in table
// order; one thread owns a 16-byte vector of the result.
template <typename T>
__global__ void __launch_bounds__(kBlock) averageKernel(T *const *xs, T *z, int n, Long length, int average, int propagate) {
    typedef typename Compute<T>::type C;
    constexpr int VEC = Pack<T>::N;
    // the vector part needs every buffer on a 16-byte boundary (whole device allocations are; views may not be)
    bool aligned = z == nullptr || (reinterpret_cast<uintptr_t>(z) & 15) == 0;
    for (int k = 0; k < n; k++) aligned = aligned && (reinterpret_cast<uintptr_t>(xs[k]) & 15) == 0;
    const Long nvec = aligned ? length / VEC : 0;
    for (Long v = (Long)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += (Long)gridDim.x * kBlock) {
        C acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = (C)0;
        for (int k = 0; k < n; k++) {
            const Pack<T> p = loadPack(reinterpret_cast<const Pack<T> *>(xs[k]) + v);
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[e] += toCompute(p.v[e]);
        }
        Pack<T> o;
#pragma unroll
        for (int e = 0; e < VEC; e++) o.v[e] = fromCompute<T>(average ? acc[e] / (C)n : acc[e]);
        if (z != nullptr) storePack(reinterpret_cast<Pack<T> *>(z) + v, o);
        if (propagate)
            for (int k = 0; k < n; k++) storePack(reinterpret_cast<Pack<T> *>(xs[k]) + v, o);
    }
    for (Long i = nvec * VEC + (Long)blockIdx.x * kBlock + threadIdx.x; i < length; i += (Long)gridDim.x * kBlock) {
        C acc = (C)0;
        for (int k = 0; k < n; k++) acc += toCompute(xs[k][i]);
        const T o = fromCompute<T>(average ? acc / (C)n : acc);
        if (z != nullptr) z[i] = o;
        if (propagate)
            for (int k = 0; k < n; k++) xs[k][i] = o;
    }
}
template <typename T> void launchAverage(hipStream_t s, T *const *xs, T *z, int n, Long length, bool average, bool propagate) {
    if (n <= 0 || length <= 0) return;
    const int grid = gridFor(length, (Long)kBlock * Pack<T>::N, kGridCap * 4);
    ND4J_LAUNCH((averageKernel<T>), dim3(grid), dim3(kBlock), 0, s, xs, z, n, length, average ? 1 : 0, propagate ? 1 : 0);
}

// ---- conversions between half, float and double: z[i] = (D)(float)x[i] (type_conversions.h:38-49) -----------------
template <typename S, typename D> __device__ __forceinline__ D convertOne(S v) {
    const float f = (float)toCompute(v);
    return fromCompute<D>((typename Compute<D>::type)f);
}
// Narrowing (or equal width): a thread converts 8 elements per pass, reading two or four 16-byte vectors and writing
// one or two.  Widening: every store instruction should cover one contiguous stretch per wave (stores of 16 bytes
// that alternate between the lanes' halves of 32-byte pieces were a third slower), so a thread converts the
// 16 / sizeof(D) elements of ONE output vector per step and takes two steps a block-width apart.
template <typename S, typename D>
__global__ void __launch_bounds__(kBlock) convertKernel(const S *x, D *z, Long n, int vectors) {
    constexpr bool widening = sizeof(D) > sizeof(S);
    constexpr int E = widening ? 16 / (int)sizeof(D) : 8;
    const Long chunks = vectors ? n / E : 0;
    if (widening) {
        constexpr int STEPS = 2;  // (half -> float over 2^26 elements: 65.6 us; 67.3 with four steps, 68.2 with one)
        typedef typename std::conditional<E * sizeof(S) == 8, unsigned long long, unsigned>::type Word;  // E source elements
        for (Long c0 = (Long)blockIdx.x * (kBlock * STEPS) + threadIdx.x; c0 < chunks; c0 += (Long)gridDim.x * (kBlock * STEPS)) {
            Word w[STEPS];
#pragma unroll
            for (int k = 0; k < STEPS; k++) {
                const Long c = c0 + (Long)k * kBlock;
                if (c < chunks) w[k] = __builtin_nontemporal_load(reinterpret_cast<const Word *>(x) + c);
            }
#pragma unroll
            for (int k = 0; k < STEPS; k++) {
                const Long c = c0 + (Long)k * kBlock;
                if (c >= chunks) break;
                alignas(8) S in[E];
                alignas(16) D out[E];
                *reinterpret_cast<Word *>(in) = w[k];
#pragma unroll
                for (int e = 0; e < E; e++) out[e] = convertOne<S, D>(in[e]);
                __builtin_nontemporal_store(*reinterpret_cast<const U32x4 *>(out), reinterpret_cast<U32x4 *>(z) + c);
            }
        }
    } else {
        for (Long c = (Long)blockIdx.x * kBlock + threadIdx.x; c < chunks; c += (Long)gridDim.x * kBlock) {
            alignas(16) S in[E];
            alignas(16) D out[E];
            constexpr int NS = E * sizeof(S) / 16, ND = E * sizeof(D) / 16;
            const U32x4 *src = reinterpret_cast<const U32x4 *>(x + c * E);
#pragma unroll
            for (int k = 0; k < NS; k++) reinterpret_cast<U32x4 *>(in)[k] = __builtin_nontemporal_load(src + k);
#pragma unroll
            for (int e = 0; e < E; e++) out[e] = convertOne<S, D>(in[e]);
            U32x4 *dst = reinterpret_cast<U32x4 *>(z + c * E);
#pragma unroll
            for (int k = 0; k < ND; k++) __builtin_nontemporal_store(reinterpret_cast<const U32x4 *>(out)[k], dst + k);
        }
    }
    for (Long i = chunks * E + (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += (Long)gridDim.x * kBlock)
        z[i] = convertOne<S, D>(x[i]);
}
template <typename S, typename D> void runConvert(hipStream_t s, const void *x, void *z, Long n) {
    if (n <= 0) return;
    const int vectors = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(z)) & 15) == 0 ? 1 : 0;
    // elements per block and pass: 8 per thread when narrowing, two output vectors per thread when widening
    const Long perBlock = sizeof(D) > sizeof(S) ? (Long)kBlock * 2 * (16 / (Long)sizeof(D)) : (Long)kBlock * 8;
    ND4J_LAUNCH((convertKernel<S, D>), dim3(gridFor(n, perBlock, kMaxGrid)), dim3(kBlock), 0, s,
                       reinterpret_cast<const S *>(x), reinterpret_cast<D *>(z), n, vectors);
}
// type codes of type_conversions.h:11-18: 3 half, 6 float, 7 double
bool launchConvert(hipStream_t s, int srcType, const void *x, Long n, int dstType, void *z) {
    if (srcType == 3 && dstType == 6) runConvert<float16, float>(s, x, z, n);
    else if (srcType == 3 && dstType == 7) runConvert<float16, double>(s, x, z, n);
    else if (srcType == 6 && dstType == 3) runConvert<float, float16>(s, x, z, n);
    else if (srcType == 6 && dstType == 7) runConvert<float, double>(s, x, z, n);
    else if (srcType == 7 && dstType == 3) runConvert<double, float16>(s, x, z, n);
    else if (srcType == 7 && dstType == 6) runConvert<double, float>(s, x, z, n);
    else return false;
    return true;
}

#define INST(T)                                                                                                              \
    template void launchPullRows<T>(hipStream_t, const T *, T *, Long, const Long *, const Long *, const Long *, const Long *, \
                                    const Long *);                                                                           \
    template void launchTear<T>(hipStream_t, const T *, const Long *, T *const *, const Long *, const Long *, const Long *,  \
                                Long);                                                                                       \
    template void launchShuffle<T>(hipStream_t, T *const *, const Long *const *, T *const *, int, const int *,               \
                                   const Long *const *, const Long *const *, Long);                                          \
    template void launchConcat<T>(hipStream_t, const T *const *, const Long *const *, T *, const ConcatView &, int, Long, void *); \
    template void launchTransposeCopy<T>(hipStream_t, const T *, T *, Long, Long, Long, Long);                            \
    template void launchCopyToEws<T>(hipStream_t, const T *, Long, T *, const Long *, Long);                              \
    template void launchAverage<T>(hipStream_t, T *const *, T *, int, Long, bool, bool);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
