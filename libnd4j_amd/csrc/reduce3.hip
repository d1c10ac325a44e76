// Reduce3 family: one number per pair of equally long runs of x and y (distances, dot, cosine ...).
// Reference: include/loops/reduce3.h:838-916 (whole arrays), 998-1081 and 1083-1346 (per TAD), 918-995 (all
// pairs of TADs); functors include/ops/ops.h:2567-2990; opNum table include/loops/legacy_ops.h:183-191.
//
// Every functor is a sum of up to three per-pair terms - the reduction value and the two running values the
// reference keeps in extraParams[0..1] - followed by a closed-form postProcess, so the accumulator is a triple
// and partial triples merge by addition.
//
// One kernel serves all entry points: output r pairs the run of x that starts at xOffsets[r / xDiv] with the
// run of y that starts at yOffsets[r % yMod] (null tables mean offset 0); element f of a run sits at
// map(xm, f) / map(ym, f).  A whole-array call is a single output whose run is cut into slices that a second
// kernel merges.
#include <type_traits>

#include "elementwise.cuh"
#include "launch.h"
#include "reduce_engine.cuh"

namespace nd4j_amd {

template <typename C> struct Acc3 { C r, e0, e1; };

template <typename C, int OP> struct Reduce3Op {
    static __device__ __forceinline__ void accumulate(Acc3<C> &a, C d1, C d2, C eps) {
        switch (OP) {
            case 0: a.r += m::abs_(d1 - d2); break;                                   // ManhattanDistance
            case 1: { C d = d1 - d2; a.r += d * d; break; }                           // EuclideanDistance
            case 2: a.e0 += d1 * d1; a.e1 += d2 * d2; a.r += d1 * d2; break;          // CosineSimilarity
            case 3: a.r += d1 * d2; break;                                            // Dot
            case 4: {                                                                 // EqualsWithEps
                C diff = m::abs_(d1 - d2);
                C v = (C)1;
                if (diff <= eps) v = (C)0;
                else if (diff <= m::max_(m::abs_(d1), m::abs_(d2)) * eps) v = (C)0;
                a.r += v;
                break;
            }
            case 5: a.e0 += m::abs_(d1) * m::abs_(d1); a.e1 += m::abs_(d2) * m::abs_(d2); a.r += d1 * d2; break;  // CosineDistance
            case 6: a.e0 += m::min_(d1, d2); a.e1 += m::max_(d1, d2); break;          // JaccardDistance
            default: a.r += (d1 == d2) ? (C)0 : (C)1; break;                          // SimpleHammingDistance
        }
    }
    static __device__ __forceinline__ C finalize(const Acc3<C> &a, Long n) {
        switch (OP) {
            case 1: return m::sqrt_(a.r);
            case 2: return a.r / (m::sqrt_(a.e0) * m::sqrt_(a.e1));
            case 5: return (C)1 - (a.r / (m::sqrt_(a.e0) * m::sqrt_(a.e1)));
            case 6: return (C)1 - (a.e0 / a.e1);
            case 7: return a.r / (C)n;
            default: return a.r;
        }
    }
};

template <typename C> __device__ __forceinline__ Acc3<C> add3(Acc3<C> a, Acc3<C> b) {
    a.r += b.r; a.e0 += b.e0; a.e1 += b.e1;
    return a;
}
// shape of the merge helpers in reduce_engine.cuh
template <typename C> struct Acc3Merge {
    typedef Acc3<C> Acc;
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return add3(a, b); }
};

struct Reduce3Plan {
    Long runLength;        // pairs per output
    Long numOut;
    Long xDiv, yMod;       // output r -> x run r / xDiv, y run r % yMod
    const Long *xOffsets;  // device; null: 0
    const Long *yOffsets;  // device; null: 0
    DimMap xm, ym;         // pair index inside a run -> element offset
    bool contiguous;       // both maps are unit-stride
    bool allPairs;         // every run of x against every run of y: xDiv == yMod == number of runs of y
};

// GROUP lanes per output (16, 64 or the whole block).  `slices` > 1 (whole-array calls): blockIdx.x is the slice
// of the single run and the block's triple goes to partials[blockIdx.x].
template <typename T, int OP, int GROUP>
__global__ void __launch_bounds__(kBlock) reduce3Kernel(const T *x, const T *y, T *z, const T *extra, Reduce3Plan pl,
                                                        Acc3<typename Compute<T>::type> *partials, Long sliceLength, Long slices,
                                                        unsigned long long *signal, unsigned ticket, unsigned long long *slots,
                                                        unsigned *counter, unsigned slotTicket) {
    typedef typename Compute<T>::type C;
    typedef Acc3<C> Acc;
    constexpr int GROUPS = kBlock / GROUP;
    constexpr int VEC = Pack<T>::N;
    __shared__ Acc smem[kBlock / kWave];
    const C eps = extra != nullptr ? toCompute(extra[0]) : (C)0;
    const int g = threadIdx.x / GROUP, lane = threadIdx.x % GROUP;
    const bool sliced = partials != nullptr;
    const Long units = sliced ? pl.numOut * slices : pl.numOut;
    for (Long u0 = (Long)blockIdx.x * GROUPS; u0 < units; u0 += (Long)gridDim.x * GROUPS) {
        const Long u = u0 + g;
        const bool live = u < units;
        Acc acc;
        acc.r = acc.e0 = acc.e1 = (C)0;
        if (live) {
            const Long r = sliced ? u / slices : u;
            const Long f0 = sliced ? (u - r * slices) * sliceLength : 0;
            Long f1 = sliced ? f0 + sliceLength : pl.runLength;
            if (f1 > pl.runLength) f1 = pl.runLength;
            // (the usual pairing - run r of x with run r of y - needs neither the division nor the remainder)
            const Long xi = pl.xDiv == 1 ? r : r / pl.xDiv, yi = r < pl.yMod ? r : r % pl.yMod;
            const T *xr = x + (pl.xOffsets != nullptr ? pl.xOffsets[xi] : 0);
            const T *yr = y + (pl.yOffsets != nullptr ? pl.yOffsets[yi] : 0);
            // vectors wherever the two runs are misaligned alike (rows of odd length: every row starts elsewhere, but at
            // the same place in x and in y): the elements before the first and after the last aligned vector go singly
            const uintptr_t xa = reinterpret_cast<uintptr_t>(xr + f0), ya = reinterpret_cast<uintptr_t>(yr + f0);
            const bool vec = pl.contiguous && ((xa ^ ya) & 15) == 0 && xa % sizeof(T) == 0;
            if (vec) {
                Long head = (Long)(((16 - (xa & 15)) & 15) / sizeof(T));
                if (head > f1 - f0) head = f1 - f0;
                const Long nvec = (f1 - f0 - head) / VEC;
                const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(xr + f0 + head);
                const Pack<T> *yv = reinterpret_cast<const Pack<T> *>(yr + f0 + head);
                for (Long f = f0 + lane; f < f0 + head; f += GROUP)
                    Reduce3Op<C, OP>::accumulate(acc, toCompute(xr[f]), toCompute(yr[f]), eps);
                Long v = lane;
                // four vectors of each operand requested before the first is used
                for (; v + 3 * GROUP < nvec; v += 4 * GROUP) {
                    Pack<T> a[4], b[4];
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        a[k] = loadPack(xv + v + k * GROUP);
                        b[k] = loadPack(yv + v + k * GROUP);
                    }
#pragma unroll
                    for (int k = 0; k < 4; k++) {
#pragma unroll
                        for (int e = 0; e < VEC; e++) Reduce3Op<C, OP>::accumulate(acc, toCompute(a[k].v[e]), toCompute(b[k].v[e]), eps);
                    }
                }
                for (; v < nvec; v += GROUP) {
                    Pack<T> a0 = loadPack(xv + v), b0 = loadPack(yv + v);
#pragma unroll
                    for (int e = 0; e < VEC; e++) Reduce3Op<C, OP>::accumulate(acc, toCompute(a0.v[e]), toCompute(b0.v[e]), eps);
                }
                for (Long f = f0 + head + nvec * VEC + lane; f < f1; f += GROUP)
                    Reduce3Op<C, OP>::accumulate(acc, toCompute(xr[f]), toCompute(yr[f]), eps);
            } else if (pl.contiguous) {
                for (Long f = f0 + lane; f < f1; f += GROUP)
                    Reduce3Op<C, OP>::accumulate(acc, toCompute(xr[f]), toCompute(yr[f]), eps);
            } else {
                for (Long f = f0 + lane; f < f1; f += GROUP)
                    Reduce3Op<C, OP>::accumulate(acc, toCompute(xr[mapOffset64(pl.xm, (unsigned long long)f)]),
                                                 toCompute(yr[mapOffset64(pl.ym, (unsigned long long)f)]), eps);
            }
        }
        Acc3Merge<C> mg;
        if (GROUP == kBlock) {
            acc = blockMerge<Acc3Merge<C>>(mg, acc, smem);
        } else {
            if (live) acc = waveMerge<Acc3Merge<C>, GROUP>(mg, acc);
        }
        if (live && lane == 0) {
            if (sliced) {
                if (slots != nullptr) publishSlots(slots + (size_t)u * (sizeof(Acc) / 4), acc, slotTicket);
                else partials[u] = acc;
            } else {
                const T r = fromCompute<T>(Reduce3Op<C, OP>::finalize(acc, pl.runLength));
                z[u] = r;
                signalResult(signal, ticket, r);  // set only for a launch with a single result
            }
        }
    }
    if (GROUP == kBlock && slots != nullptr) {
        // A single result cut into one slice per block (`slots` is only given then): the block that counts itself in last
        // merges the slices, as the whole-array reductions do, instead of a second launch.
        __shared__ int mergeHere;
        if (threadIdx.x == 0) mergeHere = countedInLast(counter);
        __syncthreads();
        if (!mergeHere) return;
        Acc3Merge<C> mg;
        Acc acc;
        acc.r = acc.e0 = acc.e1 = (C)0;
        // (the stream's fault word lies 64 bytes behind the tagged words of its pinned block)
        unsigned *fault = signal != nullptr ? reinterpret_cast<unsigned *>(signal + 8) : nullptr;
        const bool missing = slotsWereMissing(mergeSlots<Acc3Merge<C>>(mg, acc, slots, threadIdx.x, kBlock, (int)gridDim.x, slotTicket), fault);
        acc = blockMerge<Acc3Merge<C>>(mg, acc, smem);
        if (threadIdx.x == 0) {
            const T r = missing ? notANumber<T>() : fromCompute<T>(Reduce3Op<C, OP>::finalize(acc, pl.runLength));
            z[0] = r;
            signalResult(signal, ticket, r);
        }
    }
}

template <typename T, int OP>
__global__ void __launch_bounds__(kBlock) reduce3Finish(T *z, const Acc3<typename Compute<T>::type> *partials, int count,
                                                        Long runLength, unsigned long long *signal, unsigned ticket) {
    typedef typename Compute<T>::type C;
    typedef Acc3<C> Acc;
    __shared__ Acc smem[kBlock / kWave];
    // blockIdx.x is the result; its `count` slices lie next to each other
    partials += (Long)blockIdx.x * count;
    Acc acc;
    acc.r = acc.e0 = acc.e1 = (C)0;
    for (int i = threadIdx.x; i < count; i += kBlock) acc = add3(acc, partials[i]);
    Acc3Merge<C> mg;
    acc = blockMerge<Acc3Merge<C>>(mg, acc, smem);
    if (threadIdx.x == 0) {
        const T r = fromCompute<T>(Reduce3Op<C, OP>::finalize(acc, runLength));
        z[blockIdx.x] = r;
        signalResult(signal, ticket, r);  // set only for a launch with a single result
    }
}

// Every run of x against every run of y (execReduce3All), contiguous runs: a block computes a 64 x 64 tile of
// results.  The naive pairing reads both runs from the caches for every result (nx * ny * 2 * length elements: it
// ran at the L2's 9-15 TB/s and no faster); here a block stages 32 elements of its 64 + 64 runs in LDS per step and
// every staged element serves 64 results, a thread keeping a 4 x 4 patch of accumulator triples in registers.
// Each result still sums its pairs in run order, one after the other, as the reference's loop does.
static constexpr int kTileK = 32;    // elements of each run staged per step
static constexpr int kTilePad = 4;   // keeps the LDS rows 16-byte aligned and spreads them over the banks

// PER elements of one run, staged by one thread per step
template <typename T, int PER> struct TileStage {
    typedef typename Compute<T>::type C;
    C v[PER];
    // elements k .. k + PER - 1 of the run at `run` (null: a row beyond the last run), those beyond `length` as zero
    __device__ __forceinline__ void load(const T *run, Long k, Long length) {
        constexpr int N = Pack<T>::N, NP = PER / N > 0 ? PER / N : 1;
        if (run == nullptr || k >= length) {
#pragma unroll
            for (int e = 0; e < PER; e++) v[e] = (C)0;
            return;
        }
        if (PER % N == 0 && k + PER <= length && (reinterpret_cast<uintptr_t>(run + k) & 15) == 0) {
            const Pack<T> *pv = reinterpret_cast<const Pack<T> *>(run + k);
#pragma unroll
            for (int q = 0; q < NP; q++) {
                const Pack<T> pk = pv[q];
#pragma unroll
                for (int e = 0; e < N; e++) v[q * N + e] = toCompute(pk.v[e]);
            }
            return;
        }
#pragma unroll
        for (int e = 0; e < PER; e++) v[e] = k + e < length ? toCompute(run[k + e]) : (C)0;
    }
};

// TR runs of x and of y per block (64, or 32 when 64 would leave most of the chip without a tile); a thread owns a
// TR/16 x TR/16 patch of results.
template <typename T, int OP, int TR>
__global__ void __launch_bounds__(kBlock) reduce3AllTileKernel(const T *x, const T *y, T *z, const T *extra, const Long *xOffsets,
                                                               const Long *yOffsets, Long nx, Long ny, Long length) {
    typedef typename Compute<T>::type C;
    typedef Acc3<C> Acc;
    constexpr int ROW = kTileK + kTilePad;
    constexpr int P = TR / 16;                   // patch edge
    constexpr int PER = TR * kTileK / kBlock;    // staged elements per thread, run and step
    constexpr int LANES_K = kTileK / PER;        // threads along a staged row
    __shared__ __attribute__((aligned(16))) C xs[TR][ROW];
    __shared__ __attribute__((aligned(16))) C ys[TR][ROW];
    const C eps = extra != nullptr ? toCompute(extra[0]) : (C)0;
    const Long tilesY = (ny + TR - 1) / TR;
    const Long tileX = blockIdx.x / tilesY, tileY = blockIdx.x - tileX * tilesY;
    const Long row0 = tileX * TR, col0 = tileY * TR;
    // staging role: one run of x and one of y, PER elements of each per step
    const int sRun = threadIdx.x / LANES_K, sK = (threadIdx.x % LANES_K) * PER;
    const T *xRun = row0 + sRun < nx ? x + xOffsets[row0 + sRun] : nullptr;
    const T *yRun = col0 + sRun < ny ? y + yOffsets[col0 + sRun] : nullptr;
    // computing role: results (row0 + P ti + a, col0 + P tj + b)
    const int ti = threadIdx.x / 16, tj = threadIdx.x % 16;
    Acc acc[P][P];
#pragma unroll
    for (int a = 0; a < P; a++)
#pragma unroll
        for (int b = 0; b < P; b++) acc[a][b].r = acc[a][b].e0 = acc[a][b].e1 = (C)0;

    TileStage<T, PER> sx, sy;
    sx.load(xRun, sK, length);
    sy.load(yRun, sK, length);
    for (Long k0 = 0; k0 < length; k0 += kTileK) {
#pragma unroll
        for (int e = 0; e < PER; e++) {
            xs[sRun][sK + e] = sx.v[e];
            ys[sRun][sK + e] = sy.v[e];
        }
        __syncthreads();
        if (k0 + kTileK < length) {  // the next step's elements travel while this step is computed
            sx.load(xRun, k0 + kTileK + sK, length);
            sy.load(yRun, k0 + kTileK + sK, length);
        }
        const int kmax = length - k0 < kTileK ? (int)(length - k0) : kTileK;
        int kk = 0;
        for (; kk + 4 <= kmax; kk += 4) {
            C xa[P][4], yb[P][4];
#pragma unroll
            for (int a = 0; a < P; a++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    xa[a][q] = xs[P * ti + a][kk + q];
                    yb[a][q] = ys[P * tj + a][kk + q];
                }
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int a = 0; a < P; a++)
#pragma unroll
                    for (int b = 0; b < P; b++) Reduce3Op<C, OP>::accumulate(acc[a][b], xa[a][q], yb[b][q], eps);
        }
        for (; kk < kmax; kk++) {
#pragma unroll
            for (int a = 0; a < P; a++)
#pragma unroll
                for (int b = 0; b < P; b++) Reduce3Op<C, OP>::accumulate(acc[a][b], xs[P * ti + a][kk], ys[P * tj + b][kk], eps);
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < P; a++) {
        const Long r = row0 + P * ti + a;
        if (r >= nx) continue;
#pragma unroll
        for (int b = 0; b < P; b++) {
            const Long g = col0 + P * tj + b;
            if (g < ny) z[r * ny + g] = fromCompute<T>(Reduce3Op<C, OP>::finalize(acc[a][b], length));
        }
    }
}

// The dot product of every pair of runs is a matrix product, and so is the cross term of the two cosine ops: for float
// arithmetic a block's four waves each keep a 32 x 32 quadrant of the 64 x 64 tile in the accumulator of the matrix
// unit (v_mfma_f32_32x32x2_f32: lane l supplies x[row l % 32][k + l / 32] and y[col l % 32][k + l / 32], and holds the
// results of column l % 32 in rows 8 * (v / 4) + 4 * (l / 32) + v % 4, v = 0 .. 15).  LDS holds the staged step with the
// 64 runs' values of one k side by side, so that a wave's operand loads fall in consecutive banks; a staged element is
// read from LDS once per quadrant instead of once per 4 x 4 patch, which is what bounded the vector-ALU tile kernel.
// The operands of a step's 16 matrix instructions are fetched from LDS first, then the instructions follow each other.
// The cosines' norms are sums per run, not per pair: every lane squares the operands it feeds, and the two lanes that
// hold a run's even and odd k add up at the end.  A result sums its pairs in the matrix unit's order (pairs of k),
// not one after the other as the reference's loop does: within the reductions' tolerance, not bit for bit.
typedef float MfmaAcc __attribute__((ext_vector_type(16)));
template <typename T, int OP>
__global__ void __launch_bounds__(kBlock) reduce3AllMfmaKernel(const T *x, const T *y, T *z, const Long *xOffsets,
                                                               const Long *yOffsets, Long nx, Long ny, Long length) {
    static_assert(OP == 2 || OP == 3 || OP == 5, "dot and the cosines");
    static_assert(kTileK == 32, "a step feeds 16 matrix instructions of two k each");
    constexpr int TR = 64, S = TR + 2;             // 66 words per k: the four k groups of a staging wave fall on two bank halves
    constexpr int PER = TR * kTileK / kBlock;      // staged elements per thread, run and step
    constexpr int LANES_K = kTileK / PER;          // threads along a staged run
    constexpr int N = Pack<T>::N, NP = PER / N;    // 16-byte vectors per thread, run and step
    constexpr bool NORMS = OP != 3;
    __shared__ float xs[kTileK][S];
    __shared__ float ys[kTileK][S];
    const Long tilesY = (ny + TR - 1) / TR;
    const Long tileX = blockIdx.x / tilesY, tileY = blockIdx.x - tileX * tilesY;
    const Long row0 = tileX * TR, col0 = tileY * TR;
    const int sRun = threadIdx.x / LANES_K, sK = (threadIdx.x % LANES_K) * PER;
    const T *xRun = row0 + sRun < nx ? x + xOffsets[row0 + sRun] : nullptr;
    const T *yRun = col0 + sRun < ny ? y + yOffsets[col0 + sRun] : nullptr;
    // A tile whose 128 runs all exist, start on 16-byte boundaries and hold whole steps is staged with plain vector
    // loads.  The general staging decides per thread and step between zeros, a vector and single elements, and those
    // decisions run on the compute unit's one scalar unit, which its sixteen waves share.
    const bool plainRun = xRun != nullptr && yRun != nullptr && (reinterpret_cast<uintptr_t>(xRun) & 15) == 0 &&
                          (reinterpret_cast<uintptr_t>(yRun) & 15) == 0;
    const bool plain = __builtin_amdgcn_readfirstlane(__syncthreads_and(plainRun && length % kTileK == 0 ? 1 : 0)) != 0;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int wi = wave / 2, wj = wave % 2, half = lane / 32, col = lane % 32;
    MfmaAcc acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;
    float e0 = 0.0f, e1 = 0.0f;

    TileStage<T, PER> sx, sy;
    auto fetch = [&](Long k) {
        if (plain) {
            const Pack<T> *px = reinterpret_cast<const Pack<T> *>(xRun + k + sK), *py = reinterpret_cast<const Pack<T> *>(yRun + k + sK);
#pragma unroll
            for (int q = 0; q < NP; q++) {
                const Pack<T> vx = px[q], vy = py[q];
#pragma unroll
                for (int e = 0; e < N; e++) {
                    sx.v[q * N + e] = toCompute(vx.v[e]);
                    sy.v[q * N + e] = toCompute(vy.v[e]);
                }
            }
        } else {
            // (elements beyond the end of a run, and runs beyond the last, come as zeros: they add nothing)
            sx.load(xRun, k + sK, length);
            sy.load(yRun, k + sK, length);
        }
    };
    fetch(0);
    for (Long k0 = 0; k0 < length; k0 += kTileK) {
#pragma unroll
        for (int e = 0; e < PER; e++) {
            xs[sK + e][sRun] = sx.v[e];
            ys[sK + e][sRun] = sy.v[e];
        }
        __syncthreads();
        if (k0 + kTileK < length) fetch(k0 + kTileK);  // the next step's elements travel while this step is computed
        float a[16], b[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            a[i] = xs[2 * i + half][wi * 32 + col];
            b[i] = ys[2 * i + half][wj * 32 + col];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[i], acc, 0, 0, 0);
            if (NORMS) {
                e0 = __builtin_fmaf(a[i], a[i], e0);
                e1 = __builtin_fmaf(b[i], b[i], e1);
            }
        }
        __syncthreads();
    }
    if (NORMS) {
        e0 += __shfl_xor(e0, 32, kWave);  // row wi * 32 + lane % 32 of x
        e1 += __shfl_xor(e1, 32, kWave);  // column wj * 32 + lane % 32 of y
    }
    const Long g = col0 + wj * 32 + col;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int m = 8 * (v / 4) + 4 * half + v % 4;
        Acc3<float> a3;
        a3.r = acc[v];
        a3.e0 = NORMS ? __shfl(e0, m, kWave) : 0.0f;
        a3.e1 = e1;
        const Long r = row0 + wi * 32 + m;
        if (r < nx && g < ny) z[r * ny + g] = fromCompute<T>(Reduce3Op<float, OP>::finalize(a3, length));
    }
}

template <typename T> struct Reduce3Body {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const T *x, const T *y, T *z, const T *extra, const Reduce3Plan &pl, Workspace ws) {
            typedef Acc3<typename Compute<T>::type> Acc;
            if (pl.numOut <= 0) return true;
            // all pairs of contiguous runs, enough of them to fill tiles
            if (pl.allPairs && pl.contiguous && pl.xOffsets != nullptr && pl.yOffsets != nullptr && pl.yMod >= 16 &&
                pl.numOut / pl.yMod >= 16 && pl.runLength >= 8) {
                const Long nx = pl.numOut / pl.yMod, ny = pl.yMod;
                const Long tiles64 = ((nx + 63) / 64) * ((ny + 63) / 64), tiles32 = ((nx + 31) / 32) * ((ny + 31) / 32);
                if constexpr ((OP == 2 || OP == 3 || OP == 5) && std::is_same<typename Compute<T>::type, float>::value) {
                    if (tiles64 >= 512 && tiles64 <= kMaxGrid) {
                        ND4J_LAUNCH((reduce3AllMfmaKernel<T, OP>), dim3((unsigned)tiles64), dim3(kBlock), 0, s, x, y, z, pl.xOffsets,
                                           pl.yOffsets, nx, ny, pl.runLength);
                        return true;
                    }
                }
                if (tiles64 >= 512 && tiles64 <= kMaxGrid) {
                    ND4J_LAUNCH((reduce3AllTileKernel<T, OP, 64>), dim3((unsigned)tiles64), dim3(kBlock), 0, s, x, y, z, extra,
                                       pl.xOffsets, pl.yOffsets, nx, ny, pl.runLength);
                    return true;
                }
                if (tiles32 <= kMaxGrid) {
                    ND4J_LAUNCH((reduce3AllTileKernel<T, OP, 32>), dim3((unsigned)tiles32), dim3(kBlock), 0, s, x, y, z, extra,
                                       pl.xOffsets, pl.yOffsets, nx, ny, pl.runLength);
                    return true;
                }
            }
            // one long run, or a few: cut into slices that a second kernel merges (a block per run would leave most of
            // the chip idle)
            if ((pl.numOut == 1 && pl.runLength >= 4 * kBlock) || (pl.numOut <= 1024 && pl.runLength >= 16384)) {
                Long perBlock = (Long)kBlock * 8 * Pack<T>::N;
                Long slices = (pl.runLength + perBlock - 1) / perBlock;
                // A single result: one block per compute unit (256 on this chip) and no more.  Measured over 2^26 pairs,
                // whole call: 128 slices 112 us, 192 95, 256 92, 320 108 (a second, thin round of blocks), 512 94, 1024 97,
                // 2048 102 (the last block merges as many triples as there are slices).
                const Long cap = pl.numOut == 1 ? 256 : 2048 / pl.numOut;
                if (slices > cap) slices = cap;
                if ((size_t)(slices * pl.numOut) * sizeof(Acc) > ws.bytes) slices = (Long)(ws.bytes / sizeof(Acc)) / pl.numOut;
                if (slices < 1) slices = 1;
                // slices start on 16-byte boundaries whenever the run does
                Long sliceLength = (pl.runLength + slices - 1) / slices;
                sliceLength = (sliceLength + 63) / 64 * 64;
                slices = (pl.runLength + sliceLength - 1) / sliceLength;
                if (slices >= 2) {  // a single slice needs no second launch: the per-result kernels below do it in one
                    Acc *partials = reinterpret_cast<Acc *>(ws.ptr);
                    if (pl.numOut == 1 && ws.slots != nullptr && ws.counter != nullptr && ws.slotTicketSource != nullptr &&
                        slices <= (Long)kFlatMaxBlocks && (size_t)slices * sizeof(Acc) * 2 <= ws.slotBytes) {
                        // one result: one launch, the last block merging the slices
                        ND4J_LAUNCH((reduce3Kernel<T, OP, kBlock>), dim3((unsigned)slices), dim3(kBlock), 0, s, x, y, z, extra, pl,
                                    partials, sliceLength, slices, ws.signal, ws.ticket, ws.slots, ws.counter, ws.nextSlotTicket());
                        return true;
                    }
                    ND4J_LAUNCH((reduce3Kernel<T, OP, kBlock>), dim3((unsigned)(slices * pl.numOut)), dim3(kBlock), 0, s, x, y, z,
                                       extra, pl, partials, sliceLength, slices, (unsigned long long *)nullptr, 0u,
                                       (unsigned long long *)nullptr, (unsigned *)nullptr, 0u);
                    ND4J_LAUNCH((reduce3Finish<T, OP>), dim3((unsigned)pl.numOut), dim3(kBlock), 0, s, z, partials, (int)slices,
                                       pl.runLength, pl.numOut == 1 ? ws.signal : nullptr, ws.ticket);
                    return true;
                }
            }
            Acc *none = nullptr;
            unsigned long long *signal = pl.numOut == 1 ? ws.signal : nullptr;
            const unsigned ticket = ws.ticket;
            if (pl.runLength >= 4096) {
                int grid = gridFor(pl.numOut, 1, kGridCap);
                ND4J_LAUNCH((reduce3Kernel<T, OP, kBlock>), dim3(grid), dim3(kBlock), 0, s, x, y, z, extra, pl, none, (Long)0, (Long)1, signal, ticket, (unsigned long long *)nullptr, (unsigned *)nullptr, 0u);
            } else if (pl.runLength >= 128) {
                int grid = gridFor(pl.numOut, kBlock / 64, kGridCap);
                ND4J_LAUNCH((reduce3Kernel<T, OP, 64>), dim3(grid), dim3(kBlock), 0, s, x, y, z, extra, pl, none, (Long)0, (Long)1, signal, ticket, (unsigned long long *)nullptr, (unsigned *)nullptr, 0u);
            } else {
                int grid = gridFor(pl.numOut, kBlock / 16, kGridCap);
                ND4J_LAUNCH((reduce3Kernel<T, OP, 16>), dim3(grid), dim3(kBlock), 0, s, x, y, z, extra, pl, none, (Long)0, (Long)1, signal, ticket, (unsigned long long *)nullptr, (unsigned *)nullptr, 0u);
            }
            return true;
        }
    };
};

template <typename T>
bool launchReduce3(hipStream_t s, int opNum, const T *x, const T *y, T *z, const T *extra, const Reduce3Launch &in,
                   Workspace ws) {
    Reduce3Plan pl;
    pl.runLength = in.runLength;
    pl.numOut = in.numOut;
    pl.xDiv = in.xDiv < 1 ? 1 : in.xDiv;
    pl.yMod = in.yMod < 1 ? 1 : in.yMod;
    pl.xOffsets = in.xOffsets;
    pl.yOffsets = in.yOffsets;
    pl.xm = in.xm;
    pl.ym = in.ym;
    pl.allPairs = in.allPairs;
    pl.contiguous = in.xm.rank <= 1 && in.ym.rank <= 1 && (in.xm.rank == 0 || in.xm.stride[0] == 1) &&
                    (in.ym.rank == 0 || in.ym.stride[0] == 1);
    return dispatchSeq<Reduce3Body<T>::template Run>(opNum, std::make_integer_sequence<int, 8>{}, s, x, y, z, extra, pl, ws);
}

#define INST(T)                                                                                                  \
    template bool launchReduce3<T>(hipStream_t, int, const T *, const T *, T *, const T *, const Reduce3Launch &, \
                                   Workspace);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
