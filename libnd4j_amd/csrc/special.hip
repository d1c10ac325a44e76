// Whole-array special transforms that travel through execTransform: SoftMax (38), SoftMaxDerivative (39),
// LogSoftMax (40) over the rows of a matrix or over a vector, and IsMax (41).
// Reference: include/ops/special_ops.h:1422-1573 (SoftMax), 1575-1730 (LogSoftMax), 1734-1943 (SoftMaxDerivative),
// 1945-2260 (IsMax); the CUDA back end runs the first three as five separate launches
// (blas/cuda/NativeOps.cu:3138-3252: max-reduce, subtract-broadcast, exp, sum-reduce, divide-broadcast).
//
// Here one launch does a row: maximum, sum of exp(x - max), then the result - exp is evaluated twice instead of
// being stored and read back, so a row costs one read of x from HBM (the second and third pass hit the caches
// for rows of ordinary length) and one write of z: 8 bytes per element instead of the chain's 32.
#include <atomic>

#include "elementwise.cuh"
#include <stdexcept>

#include "launch.h"
#include "reduce_engine.cuh"

namespace nd4j_amd {

template <typename C> struct MaxMerge {
    typedef C Acc;
    __device__ __forceinline__ C combine(C a, C b) const { return m::max_(a, b); }
};
template <typename C> struct SumMerge {
    typedef C Acc;
    __device__ __forceinline__ C combine(C a, C b) const { return a + b; }
};

template <typename C> __device__ __forceinline__ C laneBroadcast(C v, int srcLane, int width) {
    static_assert(sizeof(C) % 4 == 0, "compute type is a multiple of 4 bytes");
    constexpr int W = sizeof(C) / 4;
    struct Words { int w[W]; };
    Words in = __builtin_bit_cast(Words, v), out;
#pragma unroll
    for (int i = 0; i < W; i++) out.w[i] = __shfl(in.w[i], srcLane, width);
    return __builtin_bit_cast(C, out);
}

// MODE 0: softmax, 1: softmax * (1 - softmax), 2: log(softmax)
// `inv` is 1 / sum, taken once per row: multiplying by it is within 1 ULP of dividing every element by the sum (what
// the reference's loops say; its build allows the compiler the same substitution), far inside the tolerance that the
// re-associated row sum already needs.
template <int MODE, typename C> __device__ __forceinline__ C softmaxFinish(C e, C inv) {
    C v = e * inv;
    if (MODE == 1) return v * ((C)1 - v);
    if (MODE == 2) return m::logSoft_(v);
    return v;
}
// log(sum) where the logarithm needs it
template <int MODE, typename C> __device__ __forceinline__ C rowLog(C sum) { return MODE == 2 ? m::logSoft_(sum) : (C)0; }
// The result for an element d = x - max below its row's maximum.  The logarithm of exp(d) / sum is d - log(sum): one
// logarithm a row (`logSum`) instead of one an element, and no exp.  Where exp(d) has left the normal range (d < -87)
// the reference's quotient is a denormal or zero, and its logarithm is taken as the reference takes it.
template <int MODE, typename C> __device__ __forceinline__ C softmaxAt(C d, C inv, C logSum) {
    if (MODE == 2) {
        const bool far = d < (C)-87;
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(far) != 0ull, 0)) {  // a branch on the whole wave, so that it stays a branch
            const C viaExp = m::logSoft_(m::expSoft_(d) * inv);
            return far ? viaExp : d - logSum;
        }
        return d - logSum;
    }
    return softmaxFinish<MODE, C>(m::expSoft_(d), inv);
}
// what the register-resident kernels keep of an element between the pass that sums and the pass that writes: e = exp(d),
// or d itself for the logarithm (which needs e only for the sum)
template <int MODE, typename C> __device__ __forceinline__ C softmaxKeep(C e, C d) { return MODE == 2 ? d : e; }
template <int MODE, typename C> __device__ __forceinline__ C softmaxFromKept(C kept, C inv, C logSum) {
    if (MODE == 2) return softmaxAt<2, C>(kept, inv, logSum);
    return softmaxFinish<MODE, C>(kept, inv);
}
// A whole vector of kept values into results; inv and logSum per element (PER true: arrays) or one for all.  The
// logarithm's rare detour (an element more than 87 below its maximum) is looked for once per vector, not per element.
template <typename T, int MODE, bool PER, typename C>
__device__ __forceinline__ Pack<T> softmaxPackFromKept(const Pack<T> &kept, const C *inv, const C *logSum) {
    constexpr int N = Pack<T>::N;
    Pack<T> o;
    if (MODE != 2) {
#pragma unroll
        for (int e = 0; e < N; e++) o.v[e] = fromCompute<T>(softmaxFinish<MODE, C>(toCompute(kept.v[e]), inv[PER ? e : 0]));
        return o;
    }
    bool far = false;
#pragma unroll
    for (int e = 0; e < N; e++) {
        const C d = toCompute(kept.v[e]);
        far = far || d < (C)-87;
        o.v[e] = fromCompute<T>(d - logSum[PER ? e : 0]);
    }
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(far) != 0ull, 0)) {
#pragma unroll
        for (int e = 0; e < N; e++) {
            const C d = toCompute(kept.v[e]);
            if (d < (C)-87) o.v[e] = fromCompute<T>(m::logSoft_(m::expSoft_(d) * inv[PER ? e : 0]));
        }
    }
    return o;
}

// Rows whose elements are `xEl` / `zEl` apart, row r starting at r * xRow / r * zRow; GROUP lanes per row.
template <typename T, int MODE, int GROUP>
__global__ void __launch_bounds__(kBlock) softmaxRowKernel(const T *x, T *z, Long numRows, Long length, Long xRow, Long xEl,
                                                           Long zRow, Long zEl) {
    typedef typename Compute<T>::type C;
    constexpr int GROUPS = kBlock / GROUP;
    __shared__ C smem[kBlock / kWave];
    __shared__ C bcast;
    const int g = threadIdx.x / GROUP, lane = threadIdx.x % GROUP;
    for (Long r0 = (Long)blockIdx.x * GROUPS; r0 < numRows; r0 += (Long)gridDim.x * GROUPS) {
        const Long r = r0 + g;
        const bool live = r < numRows;
        const T *xr = x + (live ? r * xRow : 0);
        T *zr = z + (live ? r * zRow : 0);
        // FLOAT_MAX_VALUE of the reference's vector branch; rows of a matrix start from their first element there,
        // which gives the same maximum
        C mx = (C)-3.4028235e38;
        if (live)
            for (Long c = lane; c < length; c += GROUP) mx = m::max_(mx, toCompute(xr[c * xEl]));
        if (GROUP == kBlock) {
            MaxMerge<C> mg;
            mx = blockMerge<MaxMerge<C>>(mg, mx, smem);
            if (threadIdx.x == 0) bcast = mx;
            __syncthreads();
            mx = bcast;
        } else {
            MaxMerge<C> mg;
            mx = waveMerge<MaxMerge<C>, GROUP>(mg, mx);
            mx = laneBroadcast(mx, 0, GROUP);
        }
        C sum = (C)0;
        if (live)
            for (Long c = lane; c < length; c += GROUP) sum += m::expSoft_(toCompute(xr[c * xEl]) - mx);
        if (GROUP == kBlock) {
            SumMerge<C> mg;
            sum = blockMerge<SumMerge<C>>(mg, sum, smem);
            __syncthreads();
            if (threadIdx.x == 0) bcast = sum;
            __syncthreads();
            sum = bcast;
        } else {
            SumMerge<C> mg;
            sum = waveMerge<SumMerge<C>, GROUP>(mg, sum);
            sum = laneBroadcast(sum, 0, GROUP);
        }
        const C logSum = rowLog<MODE, C>(sum);
        sum = (C)1 / sum;
        if (live)
            for (Long c = lane; c < length; c += GROUP)
                zr[c * zEl] = fromCompute<T>(softmaxAt<MODE, C>(toCompute(xr[c * xEl]) - mx, sum, logSum));
        if (GROUP == kBlock) __syncthreads();
    }
}

// Rows that are adjacent in memory (an f-order matrix): lane <-> row, so a wave reads 64 neighbouring rows of one
// column at a time; the block's four waves split the columns and merge maximum and sum through LDS.
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock) softmaxColKernel(const T *x, T *z, Long numRows, Long length, Long xRow, Long xEl,
                                                           Long zRow, Long zEl) {
    typedef typename Compute<T>::type C;
    constexpr int WAVES = kBlock / kWave;
    __shared__ C smem[WAVES][kWave];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const Long r = (Long)blockIdx.x * kWave + lane;
    const bool live = r < numRows;
    const T *xr = x + (live ? r * xRow : 0);
    T *zr = z + (live ? r * zRow : 0);
    C mx = (C)-3.4028235e38;
    if (live) {
        Long c = wave;
        for (; c + 3 * WAVES < length; c += 4 * WAVES) {
            C v0 = toCompute(xr[c * xEl]), v1 = toCompute(xr[(c + WAVES) * xEl]), v2 = toCompute(xr[(c + 2 * WAVES) * xEl]),
              v3 = toCompute(xr[(c + 3 * WAVES) * xEl]);
            mx = m::max_(m::max_(mx, v0), m::max_(m::max_(v1, v2), v3));
        }
        for (; c < length; c += WAVES) mx = m::max_(mx, toCompute(xr[c * xEl]));
    }
    smem[wave][lane] = mx;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < WAVES; w++) mx = m::max_(mx, smem[w][lane]);
    __syncthreads();
    C sum = (C)0;
    if (live) {
        Long c = wave;
        for (; c + 3 * WAVES < length; c += 4 * WAVES) {
            C v0 = toCompute(xr[c * xEl]), v1 = toCompute(xr[(c + WAVES) * xEl]), v2 = toCompute(xr[(c + 2 * WAVES) * xEl]),
              v3 = toCompute(xr[(c + 3 * WAVES) * xEl]);
            sum += (m::expSoft_(v0 - mx) + m::expSoft_(v1 - mx)) + (m::expSoft_(v2 - mx) + m::expSoft_(v3 - mx));
        }
        for (; c < length; c += WAVES) sum += m::expSoft_(toCompute(xr[c * xEl]) - mx);
    }
    smem[wave][lane] = sum;
    __syncthreads();
    sum = (C)0;
#pragma unroll
    for (int w = 0; w < WAVES; w++) sum += smem[w][lane];
    const C logSum = rowLog<MODE, C>(sum);
    sum = (C)1 / sum;
    if (live) {
        Long c = wave;
        for (; c + 3 * WAVES < length; c += 4 * WAVES) {
            C v0 = toCompute(xr[c * xEl]), v1 = toCompute(xr[(c + WAVES) * xEl]), v2 = toCompute(xr[(c + 2 * WAVES) * xEl]),
              v3 = toCompute(xr[(c + 3 * WAVES) * xEl]);
            zr[c * zEl] = fromCompute<T>(softmaxAt<MODE, C>(v0 - mx, sum, logSum));
            zr[(c + WAVES) * zEl] = fromCompute<T>(softmaxAt<MODE, C>(v1 - mx, sum, logSum));
            zr[(c + 2 * WAVES) * zEl] = fromCompute<T>(softmaxAt<MODE, C>(v2 - mx, sum, logSum));
            zr[(c + 3 * WAVES) * zEl] = fromCompute<T>(softmaxAt<MODE, C>(v3 - mx, sum, logSum));
        }
        for (; c < length; c += WAVES) zr[c * zEl] = fromCompute<T>(softmaxAt<MODE, C>(toCompute(xr[c * xEl]) - mx, sum, logSum));
    }
}

template <typename C> __device__ __forceinline__ C laneXor(C v, int mask) {
    static_assert(sizeof(C) % 4 == 0, "compute type is a multiple of 4 bytes");
    constexpr int W = sizeof(C) / 4;
    struct Words { int w[W]; };
    Words in = __builtin_bit_cast(Words, v), out;
#pragma unroll
    for (int i = 0; i < W; i++) out.w[i] = __shfl_xor(in.w[i], mask);
    return __builtin_bit_cast(C, out);
}

// Every lane of a GROUP-lane team (a part of a wave, a wave, or the whole block) gets the merged value.
template <class Merge, int GROUP, typename C> __device__ __forceinline__ C teamAll(C v, C *smem) {
    Merge mg;
    constexpr int W = GROUP < kWave ? GROUP : kWave;
#pragma unroll
    for (int d = W / 2; d >= 1; d >>= 1) v = mg.combine(v, laneXor(v, d));
    if (GROUP > kWave) {
        const int wave = threadIdx.x / kWave;
        __syncthreads();  // smem may still be read from the previous merge
        if (threadIdx.x % kWave == 0) smem[wave] = v;
        __syncthreads();
        v = smem[0];
#pragma unroll
        for (int w = 1; w < GROUP / kWave; w++) v = mg.combine(v, smem[w]);
    }
    return v;
}

// Contiguous rows short enough to stay in registers: GROUP lanes own a row and keep PACKS 16-byte vectors of it
// each (vector j of a lane is vector lane + j * GROUP of the row's aligned part), so x is read once and z written once.
// exp(x - max) replaces x in the registers (rounded to T, which only matters for half).
// A row need not start on a 16-byte boundary, nor hold a whole number of vectors: the elements before its first and
// after its last aligned vector (fewer than 2 N, the "edge") are kept one per lane by the team's first lanes.  x and z
// must be misaligned alike in every row (the host checks it).
// (EDGES false: the host has seen that every row starts aligned and holds whole vectors, and the edge code folds away.)
// (BLOCK: threads of a block, a multiple of GROUP; the 1024-thread blocks serve the longest rows, one team a block.)
template <typename T, int MODE, int GROUP, int PACKS, bool EDGES, int BLOCK = kBlock>
__global__ void __launch_bounds__(BLOCK) softmaxRowRegKernel(const T *x, T *z, Long numRows, Long length, Long xRow, Long zRow) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N;
    constexpr int GROUPS = BLOCK / GROUP;
    __shared__ C smem[BLOCK / kWave];
    const int g = threadIdx.x / GROUP, lane = threadIdx.x % GROUP;
    // GROUP == BLOCK: every thread of the block runs the same trip count, so teamAll may synchronise
    for (Long r0 = (Long)blockIdx.x * GROUPS; r0 < numRows; r0 += (Long)gridDim.x * GROUPS) {
        const Long r = r0 + g;
        const bool live = r < numRows;
        const T *xrow = x + (live ? r * xRow : 0);
        T *zrow = z + (live ? r * zRow : 0);
        Long head = EDGES ? (Long)(((16 - (reinterpret_cast<uintptr_t>(xrow) & 15)) & 15) / sizeof(T)) : 0;
        if (head > length) head = length;
        const Long npack = (length - head) / N;
        const Long tail0 = head + npack * N;           // first element after the last whole vector
        const int edges = (int)(head + (length - tail0));  // < 2 N <= 16 <= GROUP
        const Long edgeAt = lane < head ? lane : tail0 + (lane - head);
        const bool hasEdge = EDGES && live && lane < edges;
        const Pack<T> *xr = reinterpret_cast<const Pack<T> *>(xrow + head);
        Pack<T> *zr = reinterpret_cast<Pack<T> *>(zrow + head);
        Pack<T> cache[PACKS];
        // (one branch round all the loads, none round each: a load inside a branch of its own makes the compiler wait for
        // the loads before it, and a lane's vectors then arrive one round trip after the other instead of together; a
        // vector beyond the row re-reads the row's last one and is not used - a dead row reads the first row)
        if (npack > 0) {
#pragma unroll
            for (int j = 0; j < PACKS; j++) {
                const Long at = lane + j * GROUP;
                cache[j] = loadPack(xr + (at < npack ? at : npack - 1));
            }
        }
        C edge = hasEdge ? toCompute(xrow[edgeAt]) : (C)0;
        C mx = hasEdge ? edge : (C)-3.4028235e38;
#pragma unroll
        for (int j = 0; j < PACKS; j++)
            if (live && lane + j * GROUP < npack) {
#pragma unroll
                for (int e = 0; e < N; e++) mx = m::max_(mx, toCompute(cache[j].v[e]));
            }
        mx = teamAll<MaxMerge<C>, GROUP>(mx, smem);
        C sum = (C)0;
        if (hasEdge) {
            const C d = edge - mx, ex = m::expSoft_(d);
            sum = toCompute(fromCompute<T>(ex));  // rounded to T like the cached ones
            edge = toCompute(fromCompute<T>(softmaxKeep<MODE, C>(ex, d)));
        }
#pragma unroll
        for (int j = 0; j < PACKS; j++)
            if (live && lane + j * GROUP < npack) {
#pragma unroll
                for (int e = 0; e < N; e++) {
                    const C d = toCompute(cache[j].v[e]) - mx, ex = m::expSoft_(d);
                    sum += ex;
                    cache[j].v[e] = fromCompute<T>(softmaxKeep<MODE, C>(ex, d));
                }
            }
        sum = teamAll<SumMerge<C>, GROUP>(sum, smem);
        const C logSum = rowLog<MODE, C>(sum);
        sum = (C)1 / sum;
#pragma unroll
        for (int j = 0; j < PACKS; j++)
            if (live && lane + j * GROUP < npack) {
                storePack(zr + lane + j * GROUP, softmaxPackFromKept<T, MODE, false, C>(cache[j], &sum, &logSum));
            }
        if (hasEdge) zrow[edgeAt] = fromCompute<T>(softmaxFromKept<MODE, C>(edge, sum, logSum));
    }
}

// Rows adjacent in memory (an f-order matrix) and at most kColCols * PACKS columns: a 1024-thread block owns
// 8 * Pack::N neighbouring rows at a time - eight row lanes, each loading Pack::N rows of one column as one 16-byte
// vector (a whole 128-byte line between them), times 128 column groups - and keeps all of it in registers (PACKS vectors
// a thread).  Row maxima and sums are merged over the column groups with three butterfly steps inside a wave and
// through LDS across the 16 waves.
//
// Such a block fills a compute unit, and it loads, then computes, then stores, all 16 waves in step: the unit's memory
// pipes idle while it computes.  Two smaller blocks per unit would overlap, but the registers of a unit hold 32 rows of
// 2048 floats only once; 512-thread blocks of 16 rows (half a 128-byte line per request) were slower by a third even
// with neighbouring groups of rows placed on one die, and persistent blocks that issue the next group's loads behind
// the current group's stores were slower by a tenth.  What is left to this layout is to keep the arithmetic short.
static constexpr int kColBlock = 1024, kColRowLanes = 8, kColCols = kColBlock / kColRowLanes;
template <typename T, int MODE, int PACKS>
__global__ void __launch_bounds__(kColBlock) softmaxColRegKernel(const T *x, T *z, Long numRows, Long length, Long xEl, Long zEl,
                                                                 Long groups) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N;
    constexpr int WAVES = kColBlock / kWave;
    __shared__ C smax[WAVES][kColRowLanes][N], ssum[WAVES][kColRowLanes][N];
    const int rl = threadIdx.x % kColRowLanes, cg = threadIdx.x / kColRowLanes;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    // (the LDS arrays need no barrier between two rounds: who writes smax again has passed the second barrier of the
    // round before, behind which nobody reads it; who writes ssum again has passed the first barrier of this round)
    const int cg0 = cg;
    for (Long g = blockIdx.x; g < groups; g += gridDim.x) {
    // (opaque to the optimiser, which would otherwise carry the sixteen column offsets through the loop in registers
    // that the row data needs)
    int cg = cg0;
    asm volatile("" : "+v"(cg));
    const Long row0 = (g * kColRowLanes + rl) * N;  // numRows is a multiple of N: a vector is all live or all dead
    const bool live = row0 < numRows;
    Pack<T> cache[PACKS];
    // (unconditional loads, see softmaxRowRegKernel: a column beyond the matrix re-reads the lane's first one, a dead lane
    // the matrix's first rows; neither is used.  cg < kColCols <= length wherever this kernel is chosen)
    {
        const Long liveRow = live ? row0 : 0;
#pragma unroll
        for (int j = 0; j < PACKS; j++) {
            const int col = cg + j * kColCols < length ? cg + j * kColCols : (cg < length ? cg : 0);
            cache[j] = loadPack(reinterpret_cast<const Pack<T> *>(x + liveRow + (Long)col * xEl));
        }
    }
    C mx[N], sum[N];
#pragma unroll
    for (int e = 0; e < N; e++) mx[e] = (C)-3.4028235e38;
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (live && cg + j * kColCols < length) {
#pragma unroll
            for (int e = 0; e < N; e++) mx[e] = m::max_(mx[e], toCompute(cache[j].v[e]));
        }
#pragma unroll
    for (int d = kColRowLanes; d < kWave; d <<= 1) {
#pragma unroll
        for (int e = 0; e < N; e++) mx[e] = m::max_(mx[e], laneXor(mx[e], d));
    }
    if (lane < kColRowLanes) {
#pragma unroll
        for (int e = 0; e < N; e++) smax[wave][lane][e] = mx[e];
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
#pragma unroll
        for (int e = 0; e < N; e++) mx[e] = m::max_(mx[e], smax[w][rl][e]);
    }
#pragma unroll
    for (int e = 0; e < N; e++) sum[e] = (C)0;
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (live && cg + j * kColCols < length) {
#pragma unroll
            for (int e = 0; e < N; e++) {
                const C d = toCompute(cache[j].v[e]) - mx[e], ex = m::expSoft_(d);
                sum[e] += ex;
                cache[j].v[e] = fromCompute<T>(softmaxKeep<MODE, C>(ex, d));
            }
        }
#pragma unroll
    for (int d = kColRowLanes; d < kWave; d <<= 1) {
#pragma unroll
        for (int e = 0; e < N; e++) sum[e] += laneXor(sum[e], d);
    }
    if (lane < kColRowLanes) {
#pragma unroll
        for (int e = 0; e < N; e++) ssum[wave][lane][e] = sum[e];
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < N; e++) sum[e] = ssum[0][rl][e];
#pragma unroll
    for (int w = 1; w < WAVES; w++) {
#pragma unroll
        for (int e = 0; e < N; e++) sum[e] += ssum[w][rl][e];
    }
    C logSum[N];
#pragma unroll
    for (int e = 0; e < N; e++) { logSum[e] = rowLog<MODE, C>(sum[e]); sum[e] = (C)1 / sum[e]; }
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (live && cg + j * kColCols < length) {
            storePack(reinterpret_cast<Pack<T> *>(z + row0 + (Long)(cg + j * kColCols) * zEl),
                      softmaxPackFromKept<T, MODE, true, C>(cache[j], sum, logSum));
        }
    }
}

// ---- rows too long for one block's registers, in one pass: the blocks of a row cooperate ------------------------------
// A row is cut into slices of kCoopPacks * 256 vectors; a block keeps one slice in registers, takes the slice's maximum
// m and its sum s of exp(x - m), and publishes (m, s) in the row's slot group (8-byte words tagged with the launch's
// ticket, one relaxed device-scope store each: complete or absent, no fence).  Then it waits until every slice of its
// row has published, merges the pairs (M = max m_i, S = sum s_i exp(m_i - M)) and finishes its slice from the
// registers: exp(x - m) exp(m - M) / S.  x is read once and z written once, where maxima and sums from a reduction
// pass followed by an elementwise pass read x twice.
//
// Waiting for other blocks needs them to be running.  The blocks of a row have consecutive numbers, and workgroups are
// handed out in order (per die as well), so when a block waits, the blocks before it are running or done, and the
// first row that is not finished has all its blocks on the chip: it completes and makes room.  That order is how the
// chip behaves, not a promise of the programming model, and two such launches on two streams could block each other.
// So every wait is bounded, and what a row does is decided once, by a compare-and-swap on the row's state word (the
// words lie 128 bytes apart: device-scope atomics on one 128-byte line are served one after the other, and with the
// rows' words side by side the kernel took twice as long): the
// first block that has seen all the row's slices commits the row; a block whose wait ran out first aborts it.  After a
// commit every slice is known to be there, so late blocks just read them; after an abort no block of the row writes
// anything, and the repair kernel behind the launch computes such rows the slow way, from x, which nobody has touched
// (z may be x).
static constexpr int kCoopPacks = 8;
static constexpr unsigned kCoopCommit = 1u, kCoopAbort = 2u;
static constexpr int kCoopStateStride = 32;  // the rows' state words are 128 bytes apart
static constexpr int kCoopLateTries = 5000;   // polls (a microsecond or two each) for a slice that is known to have been published
// polls a block spends on a slice that may not have been published yet before it votes to abort its row; a test may
// set it to zero, so that whatever is not there at the first look counts as missing
static std::atomic<int> gCoopWaitTries{5000};
void setCooperativeWaitLimit(int tries) { gCoopWaitTries.store(tries < 0 ? 0 : tries); }

template <typename C> struct CoopPair { C m, s; };

// one word of a slot group, waiting at most `tries` polls for the ticket; false when it did not come
__device__ __forceinline__ bool tryAwaitSlot(const unsigned long long *slot, unsigned ticket, int tries, unsigned &payload) {
    unsigned long long v = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int t = 0; (unsigned)(v >> 32) != ticket && t < tries; t++) {
        __builtin_amdgcn_s_sleep(8);
        v = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    payload = (unsigned)v;
    return (unsigned)(v >> 32) == ticket;
}
template <typename C> __device__ __forceinline__ bool tryAwaitPair(const unsigned long long *slot, unsigned ticket, int tries, CoopPair<C> &out) {
    constexpr int W = sizeof(CoopPair<C>) / 4;
    struct Words { unsigned w[W]; };
    Words in;
    bool ok = true;
#pragma unroll
    for (int i = 0; i < W; i++) ok = tryAwaitSlot(slot + i, ticket, tries, in.w[i]) && ok;
    out = __builtin_bit_cast(CoopPair<C>, in);
    return ok;
}

template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock) softmaxRowCoopKernel(const T *x, T *z, Long row0, Long numRows, Long length, Long xRow, Long zRow,
                                                               int slices, unsigned long long *slots, unsigned *rowState, unsigned ticket, int waitTries) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N, PACKS = kCoopPacks;
    constexpr int W = sizeof(CoopPair<C>) / 4;
    __shared__ C smem[kBlock / kWave];
    __shared__ unsigned decision;
    __shared__ int allThere;
    const Long local = (Long)blockIdx.x / slices;   // row within this launch
    const int sl = (int)((Long)blockIdx.x - local * slices);
    const Long r = row0 + local;
    if (r >= numRows) return;
    const T *xrow = x + r * xRow;
    T *zrow = z + r * zRow;
    // A row need not start on a 16-byte boundary nor hold whole vectors: the elements before its first aligned vector
    // are kept, one per lane, by the first lanes of its first slice, those behind its last whole vector by the first
    // lanes of its last slice (x and z are misaligned alike in every row: the host checks it).
    Long head = (Long)(((16 - (reinterpret_cast<uintptr_t>(xrow) & 15)) & 15) / sizeof(T));
    if (head > length) head = length;
    const Long nvecRow = (length - head) / N;
    const Long tail0 = head + nvecRow * N;
    const Long v0 = (Long)sl * PACKS * kBlock;       // first vector of the slice
    const bool holdsHead = sl == 0 && (Long)threadIdx.x < head;
    const bool holdsTail = sl == slices - 1 && (Long)threadIdx.x < length - tail0;
    const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(xrow + head);
    Pack<T> cache[PACKS];
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (v0 + j * kBlock + threadIdx.x < nvecRow) cache[j] = loadPack(xv + v0 + j * kBlock + threadIdx.x);
    C edge = holdsTail ? toCompute(xrow[tail0 + threadIdx.x]) : (C)0;
    C front = holdsHead ? toCompute(xrow[threadIdx.x]) : (C)0;
    C mx = holdsTail ? edge : (C)-3.4028235e38;
    if (holdsHead) mx = m::max_(mx, front);
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (v0 + j * kBlock + threadIdx.x < nvecRow) {
#pragma unroll
            for (int e = 0; e < N; e++) mx = m::max_(mx, toCompute(cache[j].v[e]));
        }
    mx = teamAll<MaxMerge<C>, kBlock>(mx, smem);
    C sum = (C)0;
    if (holdsTail) {
        const C d = edge - mx, ex = m::expSoft_(d);
        sum = toCompute(fromCompute<T>(ex));
        edge = toCompute(fromCompute<T>(softmaxKeep<MODE, C>(ex, d)));
    }
    if (holdsHead) {
        const C d = front - mx, ex = m::expSoft_(d);
        sum += toCompute(fromCompute<T>(ex));
        front = toCompute(fromCompute<T>(softmaxKeep<MODE, C>(ex, d)));
    }
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (v0 + j * kBlock + threadIdx.x < nvecRow) {
#pragma unroll
            for (int e = 0; e < N; e++) {
                const C d = toCompute(cache[j].v[e]) - mx, ex = m::expSoft_(d);
                sum += ex;
                cache[j].v[e] = fromCompute<T>(softmaxKeep<MODE, C>(ex, d));
            }
        }
    sum = teamAll<SumMerge<C>, kBlock>(sum, smem);
    unsigned long long *group = slots + (size_t)local * slices * W;
    if (threadIdx.x == 0) {
        CoopPair<C> mine;
        mine.m = mx;
        mine.s = sum;
        publishSlots(group + (size_t)sl * W, mine, ticket);
        allThere = 1;
    }
    __syncthreads();
    // thread t collects slice t of the row (a row has at most 256 slices)
    CoopPair<C> theirs;
    theirs.m = (C)-3.4028235e38;
    theirs.s = (C)0;
    bool have = true;
    if ((int)threadIdx.x < slices) {
        have = tryAwaitPair<C>(group + (size_t)threadIdx.x * W, ticket, waitTries, theirs);
        if (!have) allThere = 0;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        // the row's decision: the first block to get here makes it for all
        const unsigned want = (ticket << 2) | (allThere ? kCoopCommit : kCoopAbort);
        unsigned seen = __hip_atomic_load(rowState + local * kCoopStateStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        while ((seen >> 2) != ticket) {
            if (__hip_atomic_compare_exchange_strong(rowState + local * kCoopStateStride, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                seen = want;
                break;
            }
        }
        decision = seen & 3u;
    }
    __syncthreads();
    if (decision != kCoopCommit) return;  // aborted: the repair kernel computes this row
    // committed: every slice of the row has been published (a thread that gave up waiting finds its slice now)
    if (!have) tryAwaitPair<C>(group + (size_t)threadIdx.x * W, ticket, kCoopLateTries, theirs);
    const C rowMax = teamAll<MaxMerge<C>, kBlock>(theirs.m, smem);
    const C rowSum = teamAll<SumMerge<C>, kBlock>((int)threadIdx.x < slices ? theirs.s * m::expSoft_(theirs.m - rowMax) : (C)0, smem);
    // this slice's exp(x - mx) -> exp(x - rowMax) / rowSum; for the logarithm (x - mx) + (mx - rowMax) - log(rowSum)
    const C shift = mx - rowMax;
    const C scale = m::expSoft_(shift) / rowSum;
    const C logSum = rowLog<MODE, C>(rowSum) - shift;
    Pack<T> *zv = reinterpret_cast<Pack<T> *>(zrow + head);
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (v0 + j * kBlock + threadIdx.x < nvecRow)
            storePack(zv + v0 + j * kBlock + threadIdx.x, softmaxPackFromKept<T, MODE, false, C>(cache[j], &scale, &logSum));
    if (holdsTail) zrow[tail0 + threadIdx.x] = fromCompute<T>(softmaxFromKept<MODE, C>(edge, scale, logSum));
    if (holdsHead) zrow[threadIdx.x] = fromCompute<T>(softmaxFromKept<MODE, C>(front, scale, logSum));
}

// Rows that softmaxRowCoopKernel aborted (none, unless the chip handed out workgroups in an unexpected order or two such
// launches got in each other's way): a block per aborted row, three passes over the row, which nobody has written.
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock) softmaxRowRepairKernel(const T *x, T *z, Long row0, Long rowsHere, Long length, Long xRow, Long zRow,
                                                                 const unsigned *rowState, unsigned ticket) {
    typedef typename Compute<T>::type C;
    __shared__ C smem[kBlock / kWave];
    for (Long local = blockIdx.x; local < rowsHere; local += gridDim.x) {
        const unsigned st = __hip_atomic_load(rowState + local * kCoopStateStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (st == ((ticket << 2) | kCoopCommit)) continue;  // (a block-uniform decision)
        const T *xr = x + (row0 + local) * xRow;
        T *zr = z + (row0 + local) * zRow;
        C mx = (C)-3.4028235e38;
        for (Long c = threadIdx.x; c < length; c += kBlock) mx = m::max_(mx, toCompute(xr[c]));
        mx = teamAll<MaxMerge<C>, kBlock>(mx, smem);
        C sum = (C)0;
        for (Long c = threadIdx.x; c < length; c += kBlock) sum += m::expSoft_(toCompute(xr[c]) - mx);
        sum = teamAll<SumMerge<C>, kBlock>(sum, smem);
        const C logSum = rowLog<MODE, C>(sum), inv = (C)1 / sum;
        __syncthreads();  // in place: every thread has read its part of the row in both passes before any writes
        for (Long c = threadIdx.x; c < length; c += kBlock) zr[c] = fromCompute<T>(softmaxAt<MODE, C>(toCompute(xr[c]) - mx, inv, logSum));
        __syncthreads();
    }
}

// true when the call was taken: contiguous rows, misaligned alike in x and z, too long for the register-resident kernels
template <typename T> bool launchSoftmaxCooperative(hipStream_t s, int opNum, const T *x, T *z, const SoftmaxPlan &pl, Workspace ws) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N;
    constexpr int W = sizeof(CoopPair<C>) / 4;
    if (opNum < 38 || opNum > 40) return false;
    if (pl.xEl != 1 || pl.zEl != 1 || pl.numRows <= 0 || pl.length < (Long)kCoopPacks * kBlock * N) return false;
    // x and z misaligned alike in every row: equal distance of the bases and of the row pitches from a 16-byte boundary
    const uintptr_t xa = reinterpret_cast<uintptr_t>(x), za = reinterpret_cast<uintptr_t>(z);
    if (xa % sizeof(T) != 0 || (xa & 15) != (za & 15)) return false;
    if (pl.numRows > 1 && ((pl.xRow - pl.zRow) * (Long)sizeof(T)) % 16 != 0) return false;
    if (ws.slots == nullptr || ws.rowStates == nullptr || ws.slotTicketSource == nullptr) return false;
    const Long perSlice = (Long)kCoopPacks * kBlock * N;
    // (a row that starts off a boundary has up to N - 1 elements before its first vector; they travel with slice 0)
    const Long slices = (pl.length + perSlice - 1) / perSlice;
    if (slices > kBlock) return false;  // a thread per slice collects the row's pairs
    // rows per launch: what the slot groups and the state words hold (and a grid may number)
    Long rowsPer = (Long)(ws.slotBytes / sizeof(unsigned long long)) / (slices * W);
    if (rowsPer > (Long)ws.rowStateCount / kCoopStateStride) rowsPer = (Long)ws.rowStateCount / kCoopStateStride;
    if (rowsPer * slices > (Long)kMaxGrid) rowsPer = (Long)kMaxGrid / slices;
    if (rowsPer < 1) return false;
    for (Long row0 = 0; row0 < pl.numRows; row0 += rowsPer) {
        const Long rowsHere = pl.numRows - row0 < rowsPer ? pl.numRows - row0 : rowsPer;
        const unsigned ticket = ws.nextSlotTicket() & 0x3fffffffu;
        const dim3 grid((unsigned)(rowsHere * slices));
        const dim3 repair((unsigned)(rowsHere < 1024 ? rowsHere : 1024));
#define ND4J_COOP(MODE)                                                                                                         \
    do {                                                                                                                        \
        ND4J_LAUNCH((softmaxRowCoopKernel<T, MODE>), grid, dim3(kBlock), 0, s, x, z, row0, pl.numRows, pl.length, pl.xRow, pl.zRow, \
                    (int)slices, ws.slots, ws.rowStates, ticket, gCoopWaitTries.load());                                          \
        ND4J_LAUNCH((softmaxRowRepairKernel<T, MODE>), repair, dim3(kBlock), 0, s, x, z, row0, rowsHere, pl.length, pl.xRow,   \
                    pl.zRow, ws.rowStates, ticket);                                                                             \
    } while (0)
        if (opNum == 38) ND4J_COOP(0);
        else if (opNum == 39) ND4J_COOP(1);
        else ND4J_COOP(2);
#undef ND4J_COOP
    }
    return true;
}

template <typename T> static bool aligned16(const T *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ---- rows adjacent in memory (f-order) whose columns are shared out over cooperating blocks ---------------------------
// softmaxColRegKernel keeps 8 * Pack::N whole rows in the registers of a 1024-thread block: a 128-byte piece of every
// column, and no row longer than 2048 floats.  Here the columns of a group of rows are cut into slices of
// (block / RL) * PACKS; a 512-thread block keeps one slice of RL * Pack::N rows, two blocks to a compute unit.  With
// RL = 16 a block asks for 256 contiguous bytes of each of its columns, which the memory serves better than 128, and
// rows may be as long as the threads of a block can collect pairs for.  The blocks of a group exchange the rows' maxima
// and sums the way the blocks of a long row do (softmaxRowCoopKernel): pairs in ticket-tagged slots, bounded waits, the
// group's fate decided once by a compare-and-swap on its state word, a repair kernel behind the launch.
//
// Measured on 32768 x 2048 floats (the one-block kernel: 125 us): 8 row lanes and 2 slices 132 us, 16 and 4 117 us,
// 32 and 8 138 us, 16 and 8 with 256-thread blocks 137 us - wider pieces help, more slices to exchange cost more than
// they help.  Letting every lane start its exponentials from the maximum of its own columns, before the block has
// agreed on the rows' maxima, gained nothing (122 us), nor did late starts for the first blocks (151 us); handing
// neighbouring groups to blocks that do not run at the same time cost a third (152 us): what the memory likes here is
// that the blocks running together sweep the same columns of adjacent rows.
static constexpr int kCCCollect = 1;  // pairs each thread of a block collects
template <typename T, int MODE, int PACKS, int RL, int kCCBlock>
__global__ void __launch_bounds__(kCCBlock) __attribute__((amdgpu_waves_per_eu(4)))  // two blocks to a compute unit: 128 registers a lane
softmaxColCoopKernel(const T *x, T *z, Long group0, Long numRows, Long length, Long xEl, Long zEl,
                                                                 int slices, unsigned long long *slots, unsigned *groupState, unsigned ticket,
                                                                 int waitTries) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N, WAVES = kCCBlock / kWave, R = RL * N;  // RL row lanes, R rows to a group
    constexpr int kCCCols = kCCBlock / RL;
    constexpr int W = sizeof(CoopPair<C>) / 4;
    __shared__ C smax[WAVES][RL][N], ssum[WAVES][RL][N];
    __shared__ C allM[kCCBlock * kCCCollect], allS[kCCBlock * kCCCollect];  // the pairs of all slices: slice i, row r at [i * R + r]
    __shared__ unsigned decision;
    __shared__ int allThere;
    const int rl = threadIdx.x % RL, cg = threadIdx.x / RL;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const Long local = (Long)blockIdx.x / slices;  // group within this launch
    const int sl = (int)((Long)blockIdx.x - local * slices);
    const Long row0 = ((group0 + local) * RL + rl) * N;  // numRows is a multiple of N: a vector is all live or all dead
    const bool live = row0 < numRows;
    // this lane's columns are colFirst + j * kCCCols for j < mine (none when its rows are beyond the matrix)
    const int colFirst = sl * PACKS * kCCCols + cg;
    int mine = live && colFirst < length ? (int)((length - colFirst + kCCCols - 1) / kCCCols) : 0;
    if (mine > PACKS) mine = PACKS;
    Pack<T> cache[PACKS];
    {
        const T *px = x + row0 + (Long)colFirst * xEl;
#pragma unroll
        for (int j = 0; j < PACKS; j++)
            if (j < mine) cache[j] = loadPack(reinterpret_cast<const Pack<T> *>(px + (Long)j * kCCCols * xEl));
    }
    C mx[N], sum[N];
#pragma unroll
    for (int e = 0; e < N; e++) mx[e] = (C)-3.4028235e38;
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (j < mine) {
#pragma unroll
            for (int e = 0; e < N; e++) mx[e] = m::max_(mx[e], toCompute(cache[j].v[e]));
        }
#pragma unroll
    for (int d = RL; d < kWave; d <<= 1) {
#pragma unroll
        for (int e = 0; e < N; e++) mx[e] = m::max_(mx[e], laneXor(mx[e], d));
    }
    if (lane < RL) {
#pragma unroll
        for (int e = 0; e < N; e++) smax[wave][lane][e] = mx[e];
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
#pragma unroll
        for (int e = 0; e < N; e++) mx[e] = m::max_(mx[e], smax[w][rl][e]);
    }
#pragma unroll
    for (int e = 0; e < N; e++) sum[e] = (C)0;
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (j < mine) {
#pragma unroll
            for (int e = 0; e < N; e++) {
                const C d = toCompute(cache[j].v[e]) - mx[e], ex = m::expSoft_(d);
                sum[e] += ex;
                cache[j].v[e] = fromCompute<T>(softmaxKeep<MODE, C>(ex, d));
            }
        }
#pragma unroll
    for (int d = RL; d < kWave; d <<= 1) {
#pragma unroll
        for (int e = 0; e < N; e++) sum[e] += laneXor(sum[e], d);
    }
    if (lane < RL) {
#pragma unroll
        for (int e = 0; e < N; e++) ssum[wave][lane][e] = sum[e];
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < N; e++) sum[e] = ssum[0][rl][e];
#pragma unroll
    for (int w = 1; w < WAVES; w++) {
#pragma unroll
        for (int e = 0; e < N; e++) sum[e] += ssum[w][rl][e];
    }
    // the slice's pairs, one per row, go out from the first eight lanes; thread t then collects pair t of the group
    unsigned long long *group = slots + (size_t)local * slices * R * W;
    if (threadIdx.x < RL) {
#pragma unroll
        for (int e = 0; e < N; e++) {
            CoopPair<C> mine;
            mine.m = mx[e];
            mine.s = sum[e];
            publishSlots(group + ((size_t)sl * R + rl * N + e) * W, mine, ticket);
        }
    }
    if (threadIdx.x == 0) allThere = 1;
    __syncthreads();
    // thread t collects pair t (t + the block size, .. when kCCCollect is more than one) of the group's slices * R
    CoopPair<C> theirs[kCCCollect];
    bool have[kCCCollect];
    const int pairs = slices * R;
#pragma unroll
    for (int k = 0; k < kCCCollect; k++) {
        theirs[k].m = (C)-3.4028235e38;
        theirs[k].s = (C)0;
        have[k] = true;
        const int at = threadIdx.x + k * kCCBlock;
        if (at < pairs) {
            have[k] = tryAwaitPair<C>(group + (size_t)at * W, ticket, waitTries, theirs[k]);
            if (!have[k]) allThere = 0;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned want = (ticket << 2) | (allThere ? kCoopCommit : kCoopAbort);
        unsigned seen = __hip_atomic_load(groupState + local * kCoopStateStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        while ((seen >> 2) != ticket) {
            if (__hip_atomic_compare_exchange_strong(groupState + local * kCoopStateStride, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                seen = want;
                break;
            }
        }
        decision = seen & 3u;
    }
    __syncthreads();
    if (decision != kCoopCommit) return;  // aborted: the repair kernel computes this group, which nobody has written
#pragma unroll
    for (int k = 0; k < kCCCollect; k++) {
        const int at = threadIdx.x + k * kCCBlock;
        if (!have[k]) tryAwaitPair<C>(group + (size_t)at * W, ticket, kCoopLateTries, theirs[k]);
        allM[at] = theirs[k].m;
        allS[at] = theirs[k].s;
    }
    __syncthreads();
    C scale[N], logSum[N];
#pragma unroll
    for (int e = 0; e < N; e++) {
        const int r = rl * N + e;
        C rowMax = allM[r];
        for (int i = 1; i < slices; i++) rowMax = m::max_(rowMax, allM[i * R + r]);
        C rowSum = (C)0;
        for (int i = 0; i < slices; i++) rowSum += allS[i * R + r] * m::expSoft_(allM[i * R + r] - rowMax);
        // this slice's exp(x - mx) -> exp(x - rowMax) / rowSum; for the logarithm (x - mx) + (mx - rowMax) - log(rowSum)
        const C shift = mx[e] - rowMax;
        scale[e] = m::expSoft_(shift) / rowSum;
        logSum[e] = rowLog<MODE, C>(rowSum) - shift;
    }
    // (opaque to the optimiser, which would otherwise work out the sixteen addresses early and hold them in registers
    // that the row data needs)
    int colAgain = colFirst;
    asm volatile("" : "+v"(colAgain));
    T *pz = z + row0 + (Long)colAgain * zEl;
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (j < mine) storePack(reinterpret_cast<Pack<T> *>(pz + (Long)j * kCCCols * zEl), softmaxPackFromKept<T, MODE, true, C>(cache[j], scale, logSum));
}

// Groups of rows that softmaxColCoopKernel aborted: a block per such group, a lane per row and some columns, three passes.
template <typename T, int MODE, int RL>
__global__ void __launch_bounds__(kBlock) softmaxColRepairKernel(const T *x, T *z, Long group0, Long groupsHere, Long numRows, Long length,
                                                                 Long xEl, Long zEl, const unsigned *groupState, unsigned ticket) {
    typedef typename Compute<T>::type C;
    constexpr int R = RL * Pack<T>::N, CL = kBlock / R;
    __shared__ C part[CL][R];
    const int r = threadIdx.x % R, cl = threadIdx.x / R;
    for (Long local = blockIdx.x; local < groupsHere; local += gridDim.x) {
        const unsigned st = __hip_atomic_load(groupState + local * kCoopStateStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (st == ((ticket << 2) | kCoopCommit)) continue;  // (a block-uniform decision)
        const Long row = (group0 + local) * R + r;
        const bool live = row < numRows;
        C mx = (C)-3.4028235e38;
        if (live) for (Long c = cl; c < length; c += CL) mx = m::max_(mx, toCompute(x[row + c * xEl]));
        part[cl][r] = mx;
        __syncthreads();
        for (int k = 0; k < CL; k++) mx = m::max_(mx, part[k][r]);
        __syncthreads();
        C sum = (C)0;
        if (live) for (Long c = cl; c < length; c += CL) sum += m::expSoft_(toCompute(x[row + c * xEl]) - mx);
        part[cl][r] = sum;
        __syncthreads();  // (in place: every lane has read its share of the rows in both passes before any writes)
        sum = (C)0;
        for (int k = 0; k < CL; k++) sum += part[k][r];
        const C logSum = rowLog<MODE, C>(sum), inv = (C)1 / sum;
        if (live) for (Long c = cl; c < length; c += CL) z[row + c * zEl] = fromCompute<T>(softmaxAt<MODE, C>(toCompute(x[row + c * xEl]) - mx, inv, logSum));
        __syncthreads();
    }
}

// true when the call was taken: an f-order matrix whose column pitch keeps the row vectors aligned, with more columns than
// one block's slice and no more than the threads of a block can collect pairs for
template <typename T, int MODE, int RL, int kCCBlock> static bool runColCooperative(hipStream_t s, const T *x, T *z, const SoftmaxPlan &pl, Workspace ws) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N, R = RL * N, kCCCols = kCCBlock / RL;
    // vectors a lane keeps: a half vector unpacks to eight float maxima and sums (and eight shifts for the logarithm), so
    // fewer of them fit beside
    constexpr int PACKS = sizeof(T) == 2 ? (MODE == 2 ? 4 : 8) : 16;
    constexpr int W = sizeof(CoopPair<C>) / 4;
    const Long perSlice = (Long)PACKS * kCCCols;
    const Long slices = (pl.length + perSlice - 1) / perSlice;
    if (slices < 2 || slices * R > kCCBlock * kCCCollect) return false;
    const Long groups = (pl.numRows + R - 1) / R;
    Long groupsPer = (Long)(ws.slotBytes / sizeof(unsigned long long)) / (slices * R * W);
    if (groupsPer > (Long)ws.rowStateCount / kCoopStateStride) groupsPer = (Long)ws.rowStateCount / kCoopStateStride;
    if (groupsPer * slices > (Long)kMaxGrid) groupsPer = (Long)kMaxGrid / slices;
    if (groupsPer < 1) return false;
    for (Long group0 = 0; group0 < groups; group0 += groupsPer) {
        const Long groupsHere = groups - group0 < groupsPer ? groups - group0 : groupsPer;
        const unsigned ticket = ws.nextSlotTicket() & 0x3fffffffu;
        const dim3 grid((unsigned)(groupsHere * slices));
        const dim3 repair((unsigned)(groupsHere < 1024 ? groupsHere : 1024));
        ND4J_LAUNCH((softmaxColCoopKernel<T, MODE, PACKS, RL, kCCBlock>), grid, dim3(kCCBlock), 0, s, x, z, group0, pl.numRows, pl.length, pl.xEl,
                    pl.zEl, (int)slices, ws.slots, ws.rowStates, ticket, gCoopWaitTries.load());
        ND4J_LAUNCH((softmaxColRepairKernel<T, MODE, RL>), repair, dim3(kBlock), 0, s, x, z, group0, groupsHere, pl.numRows, pl.length,
                    pl.xEl, pl.zEl, ws.rowStates, ticket);
    }
    return true;
}
// Measurement aid: a copy of an f-order float matrix (rows adjacent in memory, columns `rows` elements apart) that moves
// exactly the tiles softmaxColCoopKernel moves, in its block order - a 512-thread block takes 64 rows x 512 columns as
// 16 row lanes x 32 column lanes, 16 vectors a lane, asking for 256 contiguous bytes of each column - with no arithmetic
// and no exchange between blocks: what that access pattern costs on its own.
__global__ void __launch_bounds__(512) forderTileCopyKernel(const float *x, float *z, Long numRows, Long length, int slices) {
    constexpr int N = 4, RL = 16, PACKS = 16, kCols = 512 / RL;
    const int rl = threadIdx.x % RL, cg = threadIdx.x / RL;
    const Long group = (Long)blockIdx.x / slices;
    const int sl = (int)((Long)blockIdx.x - group * slices);
    const Long row0 = (group * RL + rl) * N;
    if (row0 >= numRows) return;
    const int colFirst = sl * PACKS * kCols + cg;
    int mine = colFirst < length ? (int)((length - colFirst + kCols - 1) / kCols) : 0;
    if (mine > PACKS) mine = PACKS;
    Pack<float> cache[PACKS];
    const float *px = x + row0 + (Long)colFirst * numRows;
    float *pz = z + row0 + (Long)colFirst * numRows;
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (j < mine) cache[j] = loadPack(reinterpret_cast<const Pack<float> *>(px + (Long)j * kCols * numRows));
#pragma unroll
    for (int j = 0; j < PACKS; j++)
        if (j < mine) storePack(reinterpret_cast<Pack<float> *>(pz + (Long)j * kCols * numRows), cache[j]);
}
void launchForderTileCopy(hipStream_t s, const float *x, float *z, Long numRows, Long length) {
    if (numRows <= 0 || length <= 0 || numRows % 4 != 0 || !aligned16(x) || !aligned16(z))
        throw std::invalid_argument("forderTileCopy: needs 16-byte aligned operands and a row count that is a multiple of 4");
    const Long groups = (numRows + 63) / 64, slices = (length + 511) / 512;
    if (groups * slices > kMaxGrid) throw std::invalid_argument("forderTileCopy: matrix too large for one launch");
    ND4J_LAUNCH(forderTileCopyKernel, dim3((unsigned)(groups * slices)), dim3(512), 0, s, x, z, numRows, length, (int)slices);
}

template <typename T> bool launchSoftmaxColCooperative(hipStream_t s, int opNum, const T *x, T *z, const SoftmaxPlan &pl, Workspace ws) {
    constexpr int N = Pack<T>::N;
    if (opNum < 38 || opNum > 40) return false;
    if (pl.xRow != 1 || pl.zRow != 1 || pl.numRows < 256 || pl.numRows % N != 0 || pl.xEl % N != 0 || pl.zEl % N != 0) return false;
    if (!aligned16(x) || !aligned16(z)) return false;
    if (ws.slots == nullptr || ws.rowStates == nullptr || ws.slotTicketSource == nullptr) return false;
    // Sixteen row lanes (256 bytes of each column to a block, half as many columns) where the row count and the pairs to
    // collect allow it, else eight (a 128-byte line)
    constexpr int kWideLanes = sizeof(T) == 2 ? 8 : 16;
    constexpr int kWideBlock = 512;  // (64 rows of halves to a group are the most a repair block seats)
    if (opNum == 38) return runColCooperative<T, 0, kWideLanes, kWideBlock>(s, x, z, pl, ws) || runColCooperative<T, 0, 8, 512>(s, x, z, pl, ws);
    if (opNum == 39) return runColCooperative<T, 1, kWideLanes, kWideBlock>(s, x, z, pl, ws) || runColCooperative<T, 1, 8, 512>(s, x, z, pl, ws);
    return runColCooperative<T, 2, kWideLanes, kWideBlock>(s, x, z, pl, ws) || runColCooperative<T, 2, 8, 512>(s, x, z, pl, ws);
}

template <typename T, int MODE, int GROUP, int PACKS, int BLOCK = kBlock> void runRowReg(hipStream_t s, const T *x, T *z, const SoftmaxPlan &pl) {
    int grid = gridFor(pl.numRows, BLOCK / GROUP, kMaxGrid / (BLOCK / kBlock));
    constexpr int N = Pack<T>::N;
    const bool whole = aligned16(x) && aligned16(z) && pl.length % N == 0 && (pl.numRows == 1 || (pl.xRow % N == 0 && pl.zRow % N == 0));
    if (whole)
        ND4J_LAUNCH((softmaxRowRegKernel<T, MODE, GROUP, PACKS, false, BLOCK>), dim3(grid), dim3(BLOCK), 0, s, x, z, pl.numRows,
                           pl.length, pl.xRow, pl.zRow);
    else
        ND4J_LAUNCH((softmaxRowRegKernel<T, MODE, GROUP, PACKS, true, BLOCK>), dim3(grid), dim3(BLOCK), 0, s, x, z, pl.numRows,
                           pl.length, pl.xRow, pl.zRow);
}
template <typename T, int MODE, int PACKS> void runColReg(hipStream_t s, const T *x, T *z, const SoftmaxPlan &pl) {
    const Long rowsPerBlock = (Long)kColRowLanes * Pack<T>::N;
    const Long groups = (pl.numRows + rowsPerBlock - 1) / rowsPerBlock;
    const int grid = (int)(groups < (Long)kMaxGrid / 4 ? groups : (Long)kMaxGrid / 4);  // blocks of 1024 threads walk the rest
    ND4J_LAUNCH((softmaxColRegKernel<T, MODE, PACKS>), dim3(grid), dim3(kColBlock), 0, s, x, z, pl.numRows, pl.length, pl.xEl,
                       pl.zEl, groups);
}

// The widest team of the rows-in-registers kernel, and the vectors each of its lanes keeps: a 1024-thread block leaves
// a lane 128 registers, which hold 16 vectors of floats or 8 of doubles.  Halves (widened to float while they are
// worked on) would spill there, so their longest rows stay with 256 lanes of 16 vectors.
// One such block works on a row alone, so the wide team is for matrices with enough rows to occupy a good part of
// the chip; fewer, longer rows are spread over many blocks by the kernels that pass over the data more than once.
static constexpr int kRowRegLanes = 1024, kWideRowsFrom = 128;
template <typename T> struct WideRow {
    static constexpr int PACKS = sizeof(T) == 4 ? 16 : sizeof(T) == 8 ? 8 : 0;
    static constexpr Long kMostPacks = PACKS ? (Long)kRowRegLanes * PACKS : 256 * 16;  // vectors of the longest row kept in registers
};
// Which kind of kernel a softmax call gets: rows in registers, neighbouring rows in registers, or three passes.
enum SoftmaxRoute { SM_ROW_REGISTERS, SM_COL_REGISTERS, SM_PASSES };
template <typename T> SoftmaxRoute softmaxRoute(const T *x, const T *z, const SoftmaxPlan &pl) {
    constexpr int N = Pack<T>::N;
    // vectors a thread of the neighbouring-rows kernel may hold: a half vector unpacks to eight float maxima and
    // sums, which leaves room for fewer of them
    constexpr int kColPacks = sizeof(T) == 2 ? 8 : 16;
    // contiguous rows of up to WideRow::kMostPacks vectors; x and z misaligned alike in every row (equal distance
    // of the bases and of the row pitches from a 16-byte boundary), so that one row's aligned vectors are the other's
    const uintptr_t xa = reinterpret_cast<uintptr_t>(x), za = reinterpret_cast<uintptr_t>(z);
    if (pl.xEl == 1 && pl.zEl == 1 && pl.length >= 16 * N && xa % sizeof(T) == 0 && (xa & 15) == (za & 15) &&
        (pl.numRows == 1 || ((pl.xRow - pl.zRow) * (Long)sizeof(T)) % 16 == 0) && pl.length / N <= (pl.numRows >= kWideRowsFrom ? WideRow<T>::kMostPacks : 256 * 16))
        return SM_ROW_REGISTERS;
    if (!(aligned16(x) && aligned16(z))) return SM_PASSES;
    // an f-order matrix whose column stride keeps the row vectors aligned
    if (pl.xRow == 1 && pl.zRow == 1 && pl.numRows % N == 0 && pl.xEl % N == 0 && pl.zEl % N == 0 && pl.numRows >= kWave &&
        pl.length <= (Long)kColCols * kColPacks && true)
        return SM_COL_REGISTERS;
    return SM_PASSES;
}

template <typename T, int MODE> void runSoftmax(hipStream_t s, const T *x, T *z, const SoftmaxPlan &pl) {
    if (pl.numRows <= 0 || pl.length <= 0) return;
    constexpr int N = Pack<T>::N;
    constexpr int kColPacks = sizeof(T) == 2 ? 8 : 16;
    const SoftmaxRoute route = softmaxRoute<T>(x, z, pl);
    if (route == SM_ROW_REGISTERS) {
        const Long npack = pl.length / N;  // at most this many aligned vectors in a row (fewer when it starts off a boundary)
        if (npack <= 16 * 2) runRowReg<T, MODE, 16, 2>(s, x, z, pl);
        else if (npack <= 64 * 2) runRowReg<T, MODE, 64, 2>(s, x, z, pl);
        // (a wave per row up to 256 vectors, a block per row beyond: rows of 2048 floats 88 -> 86 us, log-softmax 90 -> 86)
        else if (npack <= 64 * 4) runRowReg<T, MODE, 64, 8>(s, x, z, pl);
        else if (npack <= 256 * 4) runRowReg<T, MODE, kBlock, 4>(s, x, z, pl);
        else if (npack <= 256 * 8) runRowReg<T, MODE, kBlock, 8>(s, x, z, pl);
        else if (npack <= 256 * 16) runRowReg<T, MODE, kBlock, 16>(s, x, z, pl);
        else if constexpr (WideRow<T>::PACKS > 0) runRowReg<T, MODE, kRowRegLanes, WideRow<T>::PACKS, kRowRegLanes>(s, x, z, pl);
        return;
    }
    if (route == SM_COL_REGISTERS) {
        if (pl.length <= (Long)kColCols * 2) runColReg<T, MODE, 2>(s, x, z, pl);
        else if (pl.length <= (Long)kColCols * kColPacks / 2) runColReg<T, MODE, kColPacks / 2>(s, x, z, pl);
        else runColReg<T, MODE, kColPacks>(s, x, z, pl);
        return;
    }
    if (pl.xRow == 1 && pl.zRow == 1 && pl.numRows >= kWave) {
        int grid = (int)((pl.numRows + kWave - 1) / kWave);
        ND4J_LAUNCH((softmaxColKernel<T, MODE>), dim3(grid), dim3(kBlock), 0, s, x, z, pl.numRows, pl.length, pl.xRow, pl.xEl,
                           pl.zRow, pl.zEl);
        return;
    }
    if (pl.length >= 2048 || pl.numRows < 4) {
        int grid = gridFor(pl.numRows, 1, kGridCap);
        ND4J_LAUNCH((softmaxRowKernel<T, MODE, kBlock>), dim3(grid), dim3(kBlock), 0, s, x, z, pl.numRows, pl.length, pl.xRow,
                           pl.xEl, pl.zRow, pl.zEl);
    } else if (pl.length >= 128) {
        int grid = gridFor(pl.numRows, kBlock / 64, kGridCap);
        ND4J_LAUNCH((softmaxRowKernel<T, MODE, 64>), dim3(grid), dim3(kBlock), 0, s, x, z, pl.numRows, pl.length, pl.xRow,
                           pl.xEl, pl.zRow, pl.zEl);
    } else {
        int grid = gridFor(pl.numRows, kBlock / 16, kGridCap);
        ND4J_LAUNCH((softmaxRowKernel<T, MODE, 16>), dim3(grid), dim3(kBlock), 0, s, x, z, pl.numRows, pl.length, pl.xRow,
                           pl.xEl, pl.zRow, pl.zEl);
    }
}

// true when runSoftmax would take one of the kernels that keep their rows in registers
template <typename T> bool softmaxFitsRegisters(const T *x, const T *z, const SoftmaxPlan &pl) {
    return softmaxRoute<T>(x, z, pl) != SM_PASSES;
}

// Last step of the softmax family when the row maxima and the row sums of exp(x - max) came from the reduction
// kernels (rows too long for registers): p = exp(x - max[r]) / sum[r], as the register-resident kernels compute it.
// Threads run along the direction in which x is contiguous (alongRows: down the rows of an f-order matrix),
// blockIdx.y walks the other one.
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock) softmaxFinishKernel(const T *x, T *z, const T *maxima,
                                                              const typename Compute<T>::type *sums, Long numRows,
                                                              Long length, Long xRow, Long xEl, Long zRow, Long zEl, int alongRows) {
    typedef typename Compute<T>::type C;
    const Long fastLen = alongRows ? numRows : length, slowLen = alongRows ? length : numRows;
    for (Long sl = blockIdx.y; sl < slowLen; sl += gridDim.y) {
        for (Long f = (Long)blockIdx.x * kBlock + threadIdx.x; f < fastLen; f += (Long)gridDim.x * kBlock) {
            const Long r = alongRows ? f : sl, c = alongRows ? sl : f;
            const C d = toCompute(x[r * xRow + c * xEl]) - toCompute(maxima[r]);
            z[r * zRow + c * zEl] = fromCompute<T>(softmaxAt<MODE, C>(d, (C)1 / sums[r], rowLog<MODE, C>(sums[r])));
        }
    }
}
// The same with 16-byte accesses over the matrix as one list of vectors.  ALONG 0: rows are contiguous, a vector lies
// within one row.  ALONG 1: rows are adjacent in memory (f-order), a vector holds neighbouring rows of one column, with
// their maxima and sums as vectors too.  A capped grid walks the list (the lookup tables are staged once per block), and
// each thread asks for its next vector before it works on the current one; the first is requested before the tables.
template <typename T, int MODE, int ALONG> struct SoftmaxFinishItem {
    typedef typename Compute<T>::type C;
    Pack<T> a, pm;
    C ps[Pack<T>::N];
    C mx, sum;
    Long sl, v;
    __device__ __forceinline__ void load(Long id, bool small, const T *x, const T *maxima, const C *sums, Long fastVecs, Long xSlow) {
        sl = small ? (Long)((unsigned)id / (unsigned)fastVecs) : id / fastVecs;
        v = id - sl * fastVecs;
        a = loadPack(reinterpret_cast<const Pack<T> *>(x + sl * xSlow) + v);
        if (ALONG == 1) {
            pm = reinterpret_cast<const Pack<T> *>(maxima)[v];
#pragma unroll
            for (int e = 0; e < Pack<T>::N; e++) ps[e] = sums[v * Pack<T>::N + e];
        } else {
            mx = toCompute(maxima[sl]);
            sum = sums[sl];
        }
    }
    __device__ __forceinline__ void finish(T *z, Long zSlow) const {
        constexpr int N = Pack<T>::N;
        Pack<T> o;
        const C inv = ALONG == 1 ? (C)0 : (C)1 / sum, logInv = ALONG == 1 ? (C)0 : rowLog<MODE, C>(sum);
#pragma unroll
        for (int e = 0; e < N; e++) {
            const C m1 = ALONG == 1 ? toCompute(pm.v[e]) : mx;
            const C i1 = ALONG == 1 ? (C)1 / ps[e] : inv;
            const C logSum = ALONG == 1 ? rowLog<MODE, C>(ps[e]) : logInv;
            o.v[e] = fromCompute<T>(softmaxAt<MODE, C>(toCompute(a.v[e]) - m1, i1, logSum));
        }
        storePack(reinterpret_cast<Pack<T> *>(z + sl * zSlow) + v, o);
    }
};
template <typename T, int MODE, int ALONG>
__global__ void __launch_bounds__(kBlock) softmaxFinishVecKernel(const T *x, T *z, const T *maxima,
                                                                 const typename Compute<T>::type *sums, Long fastVecs,
                                                                 Long slowLen, Long xSlow, Long zSlow) {
    const Long total = fastVecs * slowLen, stride = (Long)gridDim.x * kBlock;
    const bool small = total <= 0xffffffffLL;
    Long id = (Long)blockIdx.x * kBlock + threadIdx.x;
    SoftmaxFinishItem<T, MODE, ALONG> cur, next;
    bool have = id < total;
    if (have) cur.load(id, small, x, maxima, sums, fastVecs, xSlow);
    while (have) {
        id += stride;
        const bool more = id < total;
        if (more) next.load(id, small, x, maxima, sums, fastVecs, xSlow);
        cur.finish(z, zSlow);
        cur = next;
        have = more;
    }
}

// Contiguous rows whose starts are not all 16-byte aligned (an odd row length, e.g. a 50257-word vocabulary): each row
// is finished with 16-byte accesses between its own aligned head and tail, which works whenever x and z are misaligned
// alike in every row (same row stride, bases equally aligned).  blockIdx.y walks the rows, blockIdx.x the row's vectors.
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock) softmaxFinishRowsKernel(const T *x, T *z, const T *maxima,
                                                                  const typename Compute<T>::type *sums, Long numRows, Long length,
                                                                  Long xRow, Long zRow) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N;
    for (Long r = blockIdx.y; r < numRows; r += gridDim.y) {
        const T *xr = x + r * xRow;
        T *zr = z + r * zRow;
        const C mx = toCompute(maxima[r]), inv = (C)1 / sums[r], logSum = rowLog<MODE, C>(sums[r]);
        Long head = (Long)(((16 - (reinterpret_cast<uintptr_t>(xr) & 15)) & 15) / sizeof(T));
        if (head > length) head = length;
        const Long nvec = (length - head) / N;
        const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(xr + head);
        Pack<T> *zv = reinterpret_cast<Pack<T> *>(zr + head);
        for (Long v = (Long)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += (Long)gridDim.x * kBlock) {
            const Pack<T> a = loadPack(xv + v);
            Pack<T> o;
#pragma unroll
            for (int e = 0; e < N; e++) o.v[e] = fromCompute<T>(softmaxAt<MODE, C>(toCompute(a.v[e]) - mx, inv, logSum));
            storePack(zv + v, o);
        }
        if (blockIdx.x == 0) {
            // the elements before the first and after the last whole vector: fewer than 2 N of them
            const Long tail0 = head + nvec * N;
            for (Long f = threadIdx.x; f < head + (length - tail0); f += kBlock) {
                const Long c = f < head ? f : tail0 + (f - head);
                zr[c] = fromCompute<T>(softmaxAt<MODE, C>(toCompute(xr[c]) - mx, inv, logSum));
            }
        }
    }
}

template <typename T>
bool launchSoftmaxFinish(hipStream_t s, int opNum, const T *x, T *z, const T *maxima, const typename Compute<T>::type *sums,
                         const SoftmaxPlan &pl) {
    if (pl.numRows <= 0 || pl.length <= 0) return true;
    const int alongRows = (pl.xRow == 1 && pl.xEl != 1) ? 1 : 0;
    const Long fastLen = alongRows ? pl.numRows : pl.length, slowLen = alongRows ? pl.length : pl.numRows;
    constexpr int N = Pack<T>::N;
    const Long xSlow = alongRows ? pl.xEl : pl.xRow, zSlow = alongRows ? pl.zEl : pl.zRow;
    const bool contiguous = alongRows ? (pl.xRow == 1 && pl.zRow == 1) : (pl.xEl == 1 && pl.zEl == 1);
    if (contiguous && fastLen % N == 0 && (slowLen == 1 || (xSlow % N == 0 && zSlow % N == 0)) && aligned16(x) && aligned16(z) &&
        aligned16(maxima) && aligned16(sums)) {
        const Long vecs = fastLen / N;
        const dim3 vgrid((unsigned)gridFor(vecs * slowLen, kBlock, kGridCap));
#define ND4J_FINISH_VEC(MODE)                                                                                              \
    do {                                                                                                                   \
        if (alongRows)                                                                                                     \
            ND4J_LAUNCH((softmaxFinishVecKernel<T, MODE, 1>), vgrid, dim3(kBlock), 0, s, x, z, maxima, sums, vecs,   \
                               slowLen, xSlow, zSlow);                                                                     \
        else                                                                                                               \
            ND4J_LAUNCH((softmaxFinishVecKernel<T, MODE, 0>), vgrid, dim3(kBlock), 0, s, x, z, maxima, sums, vecs,   \
                               slowLen, xSlow, zSlow);                                                                     \
    } while (0)
        switch (opNum) {
            case 38: ND4J_FINISH_VEC(0); return true;
            case 39: ND4J_FINISH_VEC(1); return true;
            case 40: ND4J_FINISH_VEC(2); return true;
            default: return false;
        }
#undef ND4J_FINISH_VEC
    }
    if (!alongRows && pl.xEl == 1 && pl.zEl == 1 && pl.length >= 8 * N &&
        (reinterpret_cast<uintptr_t>(x) & 15) == (reinterpret_cast<uintptr_t>(z) & 15) &&
        (reinterpret_cast<uintptr_t>(x) & (sizeof(T) - 1)) == 0 && (pl.numRows == 1 || pl.xRow == pl.zRow)) {
        const Long gy = pl.numRows < 65535 ? pl.numRows : 65535;
        Long gx = (pl.length / N + kBlock - 1) / kBlock;
        const Long budget = kGridCap * 2 / gy > 0 ? kGridCap * 2 / gy : 1;  // about 16384 blocks in all
        if (gx > budget) gx = budget;
        const dim3 rgrid((unsigned)gx, (unsigned)gy);
#define ND4J_FINISH_ROWS(MODE)                                                                                                \
    ND4J_LAUNCH((softmaxFinishRowsKernel<T, MODE>), rgrid, dim3(kBlock), 0, s, x, z, maxima, sums, pl.numRows, pl.length, \
                       pl.xRow, pl.zRow)
        switch (opNum) {
            case 38: ND4J_FINISH_ROWS(0); return true;
            case 39: ND4J_FINISH_ROWS(1); return true;
            case 40: ND4J_FINISH_ROWS(2); return true;
            default: return false;
        }
#undef ND4J_FINISH_ROWS
    }
    const dim3 grid((unsigned)gridFor(fastLen, kBlock, 4096), (unsigned)(slowLen < 65535 ? slowLen : 65535));
#define ND4J_FINISH(MODE)                                                                                                 \
    ND4J_LAUNCH((softmaxFinishKernel<T, MODE>), grid, dim3(kBlock), 0, s, x, z, maxima, sums, pl.numRows, pl.length, \
                       pl.xRow, pl.xEl, pl.zRow, pl.zEl, alongRows)
    switch (opNum) {
        case 38: ND4J_FINISH(0); return true;
        case 39: ND4J_FINISH(1); return true;
        case 40: ND4J_FINISH(2); return true;
        default: return false;
    }
#undef ND4J_FINISH
}

template <typename T> bool launchSoftmax(hipStream_t s, int opNum, const T *x, T *z, const SoftmaxPlan &pl) {
    switch (opNum) {
        case 38: runSoftmax<T, 0>(s, x, z, pl); return true;
        case 39: runSoftmax<T, 1>(s, x, z, pl); return true;
        case 40: runSoftmax<T, 2>(s, x, z, pl); return true;
        default: return false;
    }
}

// IsMax: z = 1 where the (first) maximum sits, 0 elsewhere.  `index` holds the winning position as the index
// reductions store it (in the data type): one value for the whole array, or one per TAD.
template <typename T>
__global__ void __launch_bounds__(kBlock) isMaxFillKernel(T *z, const T *index, Long n, int strided, Long ews, DimMap zm) {
    typedef typename Compute<T>::type C;
    const Long hit = (Long)toCompute(index[0]);
    if (strided && ews == 1) {
        // a dense result: 16-byte stores between a head and a tail of single elements
        constexpr int N = Pack<T>::N;
        const uintptr_t addr = reinterpret_cast<uintptr_t>(z);
        Long head = ((addr & (sizeof(T) - 1)) == 0) ? (Long)(((16 - (addr & 15)) & 15) / sizeof(T)) : n;
        if (head > n) head = n;
        const Long nvec = (n - head) / N, gtid = (Long)blockIdx.x * kBlock + threadIdx.x;
        const T one = fromCompute<T>((C)1), zero = fromCompute<T>((C)0);
        if (gtid < head) z[gtid] = gtid == hit ? one : zero;
        Pack<T> *zv = reinterpret_cast<Pack<T> *>(z + head);
        for (Long v = gtid; v < nvec; v += (Long)gridDim.x * kBlock) {
            const Long i0 = head + v * N;
            Pack<T> o;
#pragma unroll
            for (int e = 0; e < N; e++) o.v[e] = (i0 + e == hit) ? one : zero;
            storePack(zv + v, o);
        }
        const Long tail = head + nvec * N;
        if (gtid < n - tail) z[tail + gtid] = (tail + gtid == hit) ? one : zero;
        return;
    }
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += (Long)gridDim.x * kBlock) {
        const Long o = strided ? i * ews : mapOffset64(zm, (unsigned long long)i);
        z[o] = fromCompute<T>(i == hit ? (C)1 : (C)0);
    }
}
template <typename T>
__global__ void __launch_bounds__(kBlock) isMaxTadFillKernel(T *z, const T *index, const Long *offsets, Long tadLength, Long numTads,
                                                             int strided, Long tadEws, DimMap tm) {
    typedef typename Compute<T>::type C;
    const Long total = tadLength * numTads;
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < total; i += (Long)gridDim.x * kBlock) {
        const Long r = i / tadLength, f = i - r * tadLength;
        const Long o = offsets[r] + (strided ? f * tadEws : mapOffset64(tm, (unsigned long long)f));
        z[o] = fromCompute<T>(f == (Long)toCompute(index[r]) ? (C)1 : (C)0);
    }
}

// TADs with contiguous elements: GROUP lanes write one TAD, with 16-byte stores where the TAD allows them
template <typename T, int GROUP>
__global__ void __launch_bounds__(kBlock) isMaxRowFillKernel(T *z, const T *index, const Long *offsets, Long tadLength, Long numTads) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N;
    constexpr int GROUPS = kBlock / GROUP;
    const int g = threadIdx.x / GROUP, lane = threadIdx.x % GROUP;
    const T one = fromCompute<T>((C)1), zero = fromCompute<T>((C)0);
    if (GROUP == kBlock) {
        // long TADs are written in pieces of four vectors per lane, so that a few of them still fill the chip
        const Long piece = (Long)kBlock * 4 * N, pieces = (tadLength + piece - 1) / piece;
        for (Long u = blockIdx.x; u < numTads * pieces; u += gridDim.x) {
            const Long r = u / pieces, f0 = (u - r * pieces) * piece;
            const Long f1 = f0 + piece < tadLength ? f0 + piece : tadLength;
            T *zr = z + offsets[r];
            const Long hit = (Long)toCompute(index[r]);
            if ((reinterpret_cast<uintptr_t>(zr) & 15) == 0 && tadLength % N == 0) {
                Pack<T> *zv = reinterpret_cast<Pack<T> *>(zr);
                for (Long p = f0 / N + lane; p < f1 / N; p += GROUP) {
                    Pack<T> o;
#pragma unroll
                    for (int e = 0; e < N; e++) o.v[e] = (p * N + e == hit) ? one : zero;
                    storePack(zv + p, o);
                }
            } else {
                for (Long f = f0 + lane; f < f1; f += GROUP) zr[f] = (f == hit) ? one : zero;
            }
        }
        return;
    }
    for (Long r = (Long)blockIdx.x * GROUPS + g; r < numTads; r += (Long)gridDim.x * GROUPS) {
        T *zr = z + offsets[r];
        const Long hit = (Long)toCompute(index[r]);
        if ((reinterpret_cast<uintptr_t>(zr) & 15) == 0 && tadLength % N == 0) {
            Pack<T> *zv = reinterpret_cast<Pack<T> *>(zr);
            for (Long p = lane; p < tadLength / N; p += GROUP) {
                Pack<T> o;
#pragma unroll
                for (int e = 0; e < N; e++) o.v[e] = (p * N + e == hit) ? one : zero;
                storePack(zv + p, o);
            }
        } else {
            for (Long f = lane; f < tadLength; f += GROUP) zr[f] = (f == hit) ? one : zero;
        }
    }
}
// TADs whose elements are tadEws apart: thread <-> TAD (neighbouring TADs are neighbours in memory for the usual
// layouts), blockIdx.y splits the TAD's elements
template <typename T>
__global__ void __launch_bounds__(kBlock) isMaxColFillKernel(T *z, const T *index, const Long *offsets, Long tadLength, Long numTads,
                                                             Long tadEws, Long perSplit) {
    typedef typename Compute<T>::type C;
    const Long t = (Long)blockIdx.x * kBlock + threadIdx.x;
    if (t >= numTads) return;
    const T one = fromCompute<T>((C)1), zero = fromCompute<T>((C)0);
    T *zt = z + offsets[t];
    const Long hit = (Long)toCompute(index[t]);
    const Long f0 = (Long)blockIdx.y * perSplit;
    Long f1 = f0 + perSplit;
    if (f1 > tadLength) f1 = tadLength;
    for (Long f = f0; f < f1; f++) zt[f * tadEws] = (f == hit) ? one : zero;
}

template <typename T> void launchIsMaxFill(hipStream_t s, T *z, const T *index, const FlatPlan &zp) {
    if (zp.n <= 0) return;
    // (the head and the tail of a dense result are written by the first threads of the grid: it never has fewer than 16)
    // a dense result: one 16-byte store per thread (2^26 floats in 39 us; 55 us with eight stores per thread on a capped grid)
    int grid = zp.strided && zp.ews == 1 ? gridFor(zp.n, kBlock * Pack<T>::N, kMaxGrid) : gridFor(zp.n, kBlock * 4, kGridCap);
    ND4J_LAUNCH((isMaxFillKernel<T>), dim3(grid), dim3(kBlock), 0, s, z, index, zp.n, zp.strided ? 1 : 0, zp.ews, zp.xm);
}
template <typename T> void launchIsMaxTadFill(hipStream_t s, T *z, const T *index, const TadPlan &zt) {
    if (zt.numTads <= 0 || zt.tadLength <= 0) return;
    if (zt.kind == TadPlan::ROW) {
        if (zt.tadLength >= 2048) {
            const Long pieces = (zt.tadLength + (Long)kBlock * 4 * Pack<T>::N - 1) / ((Long)kBlock * 4 * Pack<T>::N);
            ND4J_LAUNCH((isMaxRowFillKernel<T, kBlock>), dim3(gridFor(zt.numTads * pieces, 1, kMaxGrid)), dim3(kBlock), 0, s, z,
                               index, zt.offsets, zt.tadLength, zt.numTads);
        } else if (zt.tadLength >= 256) {
            ND4J_LAUNCH((isMaxRowFillKernel<T, 64>), dim3(gridFor(zt.numTads, kBlock / 64, kMaxGrid)), dim3(kBlock), 0, s, z,
                               index, zt.offsets, zt.tadLength, zt.numTads);
        } else {
            ND4J_LAUNCH((isMaxRowFillKernel<T, 16>), dim3(gridFor(zt.numTads, kBlock / 16, kMaxGrid)), dim3(kBlock), 0, s, z,
                               index, zt.offsets, zt.tadLength, zt.numTads);
        }
        return;
    }
    if (zt.kind == TadPlan::COL && zt.numTads >= kBlock) {
        const Long gx = (zt.numTads + kBlock - 1) / kBlock;
        Long splits = (4096 + gx - 1) / gx;  // enough blocks to fill the chip
        if (splits > zt.tadLength) splits = zt.tadLength;
        if (splits > 65535) splits = 65535;
        const Long per = (zt.tadLength + splits - 1) / splits;
        splits = (zt.tadLength + per - 1) / per;
        if (gx <= kMaxGrid) {
            ND4J_LAUNCH((isMaxColFillKernel<T>), dim3((unsigned)gx, (unsigned)splits), dim3(kBlock), 0, s, z, index, zt.offsets,
                               zt.tadLength, zt.numTads, zt.tadEws, per);
            return;
        }
    }
    int grid = gridFor(zt.numTads * zt.tadLength, kBlock * 4, kGridCap);
    ND4J_LAUNCH((isMaxTadFillKernel<T>), dim3(grid), dim3(kBlock), 0, s, z, index, zt.offsets, zt.tadLength, zt.numTads,
                       zt.kind == TadPlan::GENERAL ? 0 : 1, zt.tadEws, zt.tm);
}

#define INST(T)                                                                                           \
    template bool launchSoftmax<T>(hipStream_t, int, const T *, T *, const SoftmaxPlan &);                \
    template bool launchSoftmaxCooperative<T>(hipStream_t, int, const T *, T *, const SoftmaxPlan &, Workspace);  \
    template bool launchSoftmaxColCooperative<T>(hipStream_t, int, const T *, T *, const SoftmaxPlan &, Workspace);  \
    template bool softmaxFitsRegisters<T>(const T *, const T *, const SoftmaxPlan &);                     \
    template bool launchSoftmaxFinish<T>(hipStream_t, int, const T *, T *, const T *, const Compute<T>::type *, const SoftmaxPlan &); \
    template void launchIsMaxFill<T>(hipStream_t, T *, const T *, const FlatPlan &);                      \
    template void launchIsMaxTadFill<T>(hipStream_t, T *, const T *, const TadPlan &);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
