// Whole-array transforms that travel through execTransform* with a routine of their own instead of a per-element
// functor: Col2Im 36, Im2col 37, Histogram 48, Reverse 70, Pooling2D 71.
// Reference: include/ops/special_ops.h - Pooling2D::execSpecial 227-359, Im2col::execSpecial 530-663,
// Histogram::execSpecial 811-882, Col2Im::execSpecial 997-1129, Reverse::execSpecial 1317-1414.
//
// Shapes and strides come from the host copies of the shapeInfos (the launchers' arguments); extraParams is a device
// pointer in the caller's storage type and is read by the kernels.  All five are data movement with little arithmetic:
// one thread per result element, neighbouring threads on neighbouring result elements, index decomposition through
// host-prepared multipliers instead of divisions.
#include "elementwise.cuh"
#include "launch.h"

namespace nd4j_amd {

namespace {

constexpr int kWholeGrid = 1 << 20;

inline int gridFor(Long items, int perBlock = kBlock) {
    Long blocks = (items + perBlock - 1) / perBlock;
    if (blocks < 1) blocks = 1;
    return (int)(blocks > kWholeGrid ? kWholeGrid : blocks);
}

template <typename T> __device__ __forceinline__ int paramInt(const T *extra, int i) { return (int)toCompute(extra[i]); }

// what storing into T and reading back leaves of a value of the compute type (half rounds; float and double keep it):
// the reference's loops accumulate in T
template <typename T> __device__ __forceinline__ typename Compute<T>::type stored(typename Compute<T>::type v) {
    return toCompute(fromCompute<T>(v));
}

__device__ __forceinline__ bool inRange(int a, int b) { return (unsigned)a < (unsigned)b; }

}  // namespace

// ---- Reverse ---------------------------------------------------------------------------------------------------
// Contiguous, out of place: a thread stores one aligned 16-byte vector of z and loads the mirrored stretch of x, which
// is aligned only when the length and the two pointers happen to agree (the hardware serves misaligned global loads).
template <typename T>  // (goes by blockDim.x)
__global__ void __launch_bounds__(kBlock) reverseVecKernel(const T *x, T *z, Long n, int head) {
    constexpr int N = Pack<T>::N;
    // z[0 .. head) one by one, so that the vectors of z start on a 16-byte boundary
    const Long gtid = (Long)blockIdx.x * (int)blockDim.x + threadIdx.x;
    const Long lead = head < n ? head : n;
    if (gtid < lead) z[gtid] = x[n - 1 - gtid];
    const Long nvec = (n - lead) / N;
    for (Long v = gtid; v < nvec; v += (Long)gridDim.x * (int)blockDim.x) {
        const Long j = lead + v * N;  // z[j .. j + N) <- x[n - N - j .. n - j) back to front
        const Pack<T> a = loadPackAnywhere(x + (n - N - j));
        Pack<T> r;
#pragma unroll
        for (int k = 0; k < N; k++) r.v[k] = a.v[N - 1 - k];
        storePack(reinterpret_cast<Pack<T> *>(z + j), r);
    }
    const Long tail = lead + nvec * N;
    if (gtid < n - tail) z[tail + gtid] = x[n - 1 - tail - gtid];
}

// Contiguous, in place: element e swaps with element n - 1 - e for e < n / 2.  A thread takes an aligned vector of
// the front half and the mirrored (possibly misaligned) one of the back half; the pairs left over go one by one.
template <typename T>
__global__ void __launch_bounds__(kBlock) reverseSwapVecKernel(T *x, Long n, int head) {
    constexpr int N = Pack<T>::N;
    const Long pairs = n / 2;
    const Long gtid = (Long)blockIdx.x * kBlock + threadIdx.x;
    if (gtid < head && gtid < pairs) {
        const T t = x[gtid];
        x[gtid] = x[n - 1 - gtid];
        x[n - 1 - gtid] = t;
    }
    const Long nvec = pairs > head ? (pairs - head) / N : 0;
    for (Long v = gtid; v < nvec; v += (Long)gridDim.x * kBlock) {
        const Long j = head + v * N;
        Pack<T> *front = reinterpret_cast<Pack<T> *>(x + j);
        T *back = x + (n - N - j);
        const Pack<T> a = *front, b = loadPackAnywhere(back);
        Pack<T> ra, rb;
#pragma unroll
        for (int k = 0; k < N; k++) { ra.v[k] = b.v[N - 1 - k]; rb.v[k] = a.v[N - 1 - k]; }
        *front = ra;
        storePackAnywhere(back, rb);
    }
    const Long tail = head + nvec * N;
    if (pairs > tail && gtid < pairs - tail) {
        const Long e = tail + gtid;
        const T t = x[e];
        x[e] = x[n - 1 - e];
        x[n - 1 - e] = t;
    }
}

// Strided or mapped: z[zmap(n - 1 - e)] = x[xmap(e)] for e < count; SWAP exchanges the two elements of x instead.
template <typename T, bool SWAP>
__global__ void __launch_bounds__(kBlock) reverseMapKernel(const T *x, DimMap xm, T *z, DimMap zm, Long n, Long count) {
    for (Long e = (Long)blockIdx.x * kBlock + threadIdx.x; e < count; e += (Long)gridDim.x * kBlock) {
        const Long ox = mapOffsetAny(xm, e), oz = mapOffsetAny(zm, n - 1 - e);
        if (SWAP) {
            const T a = z[ox], b = z[oz];
            z[ox] = b;
            z[oz] = a;
        } else {
            z[oz] = x[ox];
        }
    }
}

template <typename T> void launchReverse(hipStream_t s, const T *x, T *z, const ReversePlan &p) {
    if (p.n <= 0) return;
    constexpr int N = Pack<T>::N;
    if (p.contiguous) {
        const int head = (int)(((16 - (reinterpret_cast<uintptr_t>(z) & 15)) & 15) / sizeof(T));
        if (p.swap) {
            ND4J_LAUNCH(reverseSwapVecKernel<T>, dim3(gridFor(p.n / 2 / N + 1)), dim3(kBlock), 0, s, z, p.n, head);
        } else {
            // (blocks of one wave: 2^26 floats in 83.4 us against 86.5 with blocks of 128 or 256 threads)
            ND4J_LAUNCH(reverseVecKernel<T>, dim3(gridFor(p.n / N + 1, 64)), dim3(64), 0, s, x, z, p.n, head);
        }
        return;
    }
    if (p.swap) {
        ND4J_LAUNCH((reverseMapKernel<T, true>), dim3(gridFor(p.count)), dim3(kBlock), 0, s, x, p.xm, z, p.zm, p.n, p.count);
    } else {
        ND4J_LAUNCH((reverseMapKernel<T, false>), dim3(gridFor(p.count)), dim3(kBlock), 0, s, x, p.xm, z, p.zm, p.n, p.count);
    }
}

// ---- Histogram -------------------------------------------------------------------------------------------------
// extra = [numBins, min, max].  The reference's compiled loop multiplies (x - min) by 1 / binSize (its release flags
// turn the loop-invariant division into a reciprocal) and truncates the way x86 does; half rounds the difference and
// the product to half, while the reciprocal stays in float (float16's operators compute in float and round the result).
template <typename T> struct HistogramBins {
    typedef typename Compute<T>::type C;
    int numBins;
    C lo, perBin;
    __device__ __forceinline__ HistogramBins(const T *extra, int capacity) {
        numBins = paramInt(extra, 0);
        lo = toCompute(extra[1]);
        const C hi = toCompute(extra[2]);
        const C binSize = stored<T>(stored<T>(hi - lo) / stored<T>((C)numBins));
        perBin = (C)1 / binSize;
        if (numBins > capacity) numBins = capacity;
    }
    __device__ __forceinline__ int operator()(T v) const {
        int idx = m::toIntX86(stored<T>(stored<T>(toCompute(v) - lo) * perBin));
        if (idx < 0) idx = 0;
        else if (idx >= numBins) idx = numBins - 1;
        return idx;
    }
};

__global__ void __launch_bounds__(kBlock) clearCountsKernel(unsigned *counts, int n) {
    for (int i = blockIdx.x * kBlock + threadIdx.x; i < n; i += gridDim.x * kBlock) counts[i] = 0u;
}

// Counts per block in LDS (when the bins fit); otherwise atomics on the global counters directly.  LDS atomics of one
// wave that meet in one bank are served one after the other, whether they name the same word or not, so the bank should
// follow from the lane and not from the bin: the block keeps `copies` (a power of two, as many as fit, up to 32)
// counters per bin side by side, lane l counting in word bin * copies + l % copies.  With 32 copies the word's bank is
// the lane's number modulo 32, which no two lanes of a half wave share.
// A block hands its counts over in one of two ways.  ROWS: it stores them, zeros included, as row blockIdx of a
// [blocks, capacity] table that the adding kernel sums; nothing needs clearing, and no two blocks touch the same word.
// Otherwise it adds them to one shared row, cleared first, with an atomic per non-empty bin: atomics of many blocks on
// the same few hundred words are served one after the other, so this way is kept for bin counts whose table would be too
// large.  Either way a block costs its share of clearing and adding up 32 KiB of LDS and of the hand-over, whatever it
// counts: two blocks per compute unit are the measured optimum (2^26 floats, 256 bins, whole call: 256 blocks 72 us,
// 384 58, 512 49, 768 51, 1024 56, 2048 64; of the 49, the counting kernel is 44 and the adding kernel 5).
constexpr int kLdsBins = 8192;
constexpr Long kHistogramTableWords = 1 << 20;
constexpr int kHistogramBlocks = 512;
constexpr int kHistogramInFlight = 4;  // vectors a lane loads before it counts them (8 measured slower)
template <typename T, bool LDS, bool ROWS>
__global__ void __launch_bounds__(kBlock) histogramCountKernel(const T *x, Long n, const T *extra, unsigned *counts, int capacity) {
    static_assert(LDS || !ROWS, "a table of rows is filled from the block's counts in LDS");
    __shared__ unsigned local[LDS ? kLdsBins : 1];
    const HistogramBins<T> bins(extra, capacity);
    if (bins.numBins <= 0) return;
    int copies = 1;
    if (LDS) {
        const int fit = kLdsBins / bins.numBins;
        while (copies < 32 && copies * 2 <= fit) copies *= 2;
        for (int b = threadIdx.x; b < bins.numBins * copies; b += kBlock) local[b] = 0u;
        __syncthreads();
    }
    const int shift = __builtin_ctz(copies);
    unsigned *myBins = local + (LDS ? (threadIdx.x & (copies - 1)) : 0);
    constexpr int N = Pack<T>::N;
    const int head = (int)(((16 - (reinterpret_cast<uintptr_t>(x) & 15)) & 15) / sizeof(T));
    const Long gtid = (Long)blockIdx.x * kBlock + threadIdx.x;
    auto count = [&](T v) {
        const int idx = bins(v);
        if (LDS) atomicAdd(&myBins[idx << shift], 1u);
        else atomicAdd(&counts[idx], 1u);
    };
    const Long lead = head < n ? head : n;
    if (gtid < lead) count(x[gtid]);
    const Long nvec = (n - lead) / N;
    const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x + lead);
    // four vectors in flight per lane: the counting of one batch then overlaps the memory latency of the next lanes'
    const Long step = (Long)gridDim.x * kBlock;
    Long v = gtid;
    for (; v + (kHistogramInFlight - 1) * step < nvec; v += kHistogramInFlight * step) {
        Pack<T> a[kHistogramInFlight];
#pragma unroll
        for (int u = 0; u < kHistogramInFlight; u++) a[u] = loadPack(xv + v + u * step);
#pragma unroll
        for (int u = 0; u < kHistogramInFlight; u++) {
#pragma unroll
            for (int k = 0; k < N; k++) count(a[u].v[k]);
        }
    }
    for (; v < nvec; v += step) {
        const Pack<T> a = loadPack(xv + v);
#pragma unroll
        for (int k = 0; k < N; k++) count(a.v[k]);
    }
    const Long tail = lead + nvec * N;
    if (gtid < n - tail) count(x[tail + gtid]);
    if (LDS) {
        __syncthreads();
        for (int b = threadIdx.x; b < bins.numBins; b += kBlock) {
            unsigned c = 0u;
            // thread b starts at copy b % copies, so that the lanes of a wave read different banks
            for (int k = 0; k < copies; k++) c += local[(b << shift) + ((k + b) & (copies - 1))];
            if (ROWS) counts[(Long)blockIdx.x * capacity + b] = c;
            else if (c != 0u) atomicAdd(&counts[b], c);
        }
    }
}

// z[b] += the counts of bin b over the table's rows, as the reference adds its counts onto what the result holds; one
// wave per bin
template <typename T>
__global__ void __launch_bounds__(kBlock) histogramAddKernel(T *z, const T *extra, const unsigned *counts, int capacity, int rows) {
    int numBins = paramInt(extra, 0);
    if (numBins > capacity) numBins = capacity;
    const int lane = threadIdx.x & 63, wavesPerBlock = kBlock / 64;
    for (int b = blockIdx.x * wavesPerBlock + (threadIdx.x >> 6); b < numBins; b += gridDim.x * wavesPerBlock) {
        unsigned c = 0u;
        for (int r = lane; r < rows; r += 64) c += counts[(Long)r * capacity + b];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
        typedef typename Compute<T>::type C;
        if (lane == 0) z[b] = fromCompute<T>(toCompute(z[b]) + (C)(int)c);
    }
}

// blocks of the counting launch, and rows of the table it fills (0: one shared row, cleared first and added to with atomics)
inline void histogramLaunchShape(Long vectors, int capacity, int &grid, int &rows) {
    grid = gridFor(vectors + 1) > kHistogramBlocks ? kHistogramBlocks : gridFor(vectors + 1);
    rows = (capacity <= kLdsBins && (Long)grid * capacity <= kHistogramTableWords) ? grid : 0;
}
size_t histogramScratchBytes(Long n, int elementBytes, int capacity) {
    int grid, rows;
    histogramLaunchShape(n / (16 / elementBytes), capacity, grid, rows);
    return (size_t)(rows > 0 ? rows : 1) * (size_t)capacity * sizeof(unsigned);
}

template <typename T>
void launchHistogram(hipStream_t s, const T *x, Long n, T *z, int capacity, const T *extra, unsigned *counts) {
    if (capacity <= 0) return;
    int grid, rows;
    histogramLaunchShape(n / Pack<T>::N, capacity, grid, rows);
    if (n <= 0) rows = 0;
    if (rows == 0) ND4J_LAUNCH(clearCountsKernel, dim3(gridFor(capacity)), dim3(kBlock), 0, s, counts, capacity);
    if (n > 0) {
        if (rows > 0)
            ND4J_LAUNCH((histogramCountKernel<T, true, true>), dim3(grid), dim3(kBlock), 0, s, x, n, extra, counts, capacity);
        else if (capacity <= kLdsBins)
            ND4J_LAUNCH((histogramCountKernel<T, true, false>), dim3(grid), dim3(kBlock), 0, s, x, n, extra, counts, capacity);
        else
            ND4J_LAUNCH((histogramCountKernel<T, false, false>), dim3(grid), dim3(kBlock), 0, s, x, n, extra, counts, capacity);
    }
    const int addGrid = (capacity + kBlock / 64 - 1) / (kBlock / 64);
    ND4J_LAUNCH(histogramAddKernel<T>, dim3(addGrid > 2048 ? 2048 : addGrid), dim3(kBlock), 0, s, z, extra, counts, capacity,
                rows > 0 ? rows : 1);
}

// ---- Im2col ----------------------------------------------------------------------------------------------------
// z[b, c, kr, kc, orow, ocol] = x[b, c, kr * dH + orow * sH - pH, kc * dW + ocol * sW - pW], zero outside the image.
// extra = [kH, kW, sH, sW, pH, pW, dH, dW]; the kernel extents are taken from z's shape.
template <typename T>
__global__ void __launch_bounds__(kBlock) im2colKernel(const T *x, T *z, const T *extra, ConvGeometry g, unsigned total) {
    const int sH = paramInt(extra, 2), sW = paramInt(extra, 3), pH = paramInt(extra, 4), pW = paramInt(extra, 5);
    const int dH = paramInt(extra, 6), dW = paramInt(extra, 7);
    for (unsigned i = blockIdx.x * kBlock + threadIdx.x; i < total; i += gridDim.x * kBlock) {
        unsigned t = i, ocol, orow, kc, kr, c;
        t = g.dOW.divmod(t, ocol);
        t = g.dOH.divmod(t, orow);
        t = g.dKW.divmod(t, kc);
        t = g.dKH.divmod(t, kr);
        const unsigned b = g.dIC.divmod(t, c);
        const int r = (int)kr * dH + (int)orow * sH - pH, q = (int)kc * dW + (int)ocol * sW - pW;
        T v = fromCompute<T>(0);
        if (inRange(r, g.iH) && inRange(q, g.iW)) v = x[b * g.imS[0] + c * g.imS[1] + r * g.imS[2] + q * g.imS[3]];
        z[b * g.colS[0] + c * g.colS[1] + kr * g.colS[2] + kc * g.colS[3] + orow * g.colS[4] + ocol * g.colS[5]] = v;
    }
}

// The same for a dense c-order result whose rows hold whole 16-byte vectors: a block owns one (b, c, kr, kc) plane of
// oH x oW results at a time, so the five-fold index decomposition happens once per plane, and a thread fills one aligned
// vector of the plane (N neighbouring columns of one row) from N image elements a stride sW apart.
template <typename T>
__global__ void __launch_bounds__(kBlock) im2colPlaneKernel(const T *x, T *z, const T *extra, ConvGeometry g, unsigned planes,
                                                            unsigned launched, int byDie) {
    constexpr int N = Pack<T>::N;
    const int sH = paramInt(extra, 2), sW = paramInt(extra, 3), pH = paramInt(extra, 4), pW = paramInt(extra, 5);
    const int dH = paramInt(extra, 6), dW = paramInt(extra, 7);
    const unsigned vecsPerRow = (unsigned)g.oW / N, vecs = vecsPerRow * (unsigned)g.oH;
    const FastDiv dRow = g.dAux;
    // The kH * kW planes of one image channel all read that channel.  Workgroups go to the chip's eight dies in turn, each
    // die with a cache of its own, so in plain order the planes of a channel land on different dies and each die fetches
    // the channel again.  `byDie`: workgroup w serves die w % 8, and the w / 8 -th plane of that die's channels (the
    // channels die, die + 8, ...), so that a channel is fetched by one die only.
    const unsigned perChannel = (unsigned)(g.kH * g.kW);
    for (unsigned w = blockIdx.x; w < launched; w += gridDim.x) {
        unsigned plane = w;
        if (byDie) {
            const unsigned die = w & 7u, local = w >> 3;
            unsigned k;
            const unsigned channel = g.dAux2.divmod(local, k) * 8u + die;
            plane = channel * perChannel + k;
        }
        if (plane >= planes) continue;
        unsigned t = plane, kc, kr, c;
        t = g.dKW.divmod(t, kc);
        t = g.dKH.divmod(t, kr);
        const unsigned b = g.dIC.divmod(t, c);
        const T *image = x + (b * g.imS[0] + c * g.imS[1]);
        Pack<T> *out = reinterpret_cast<Pack<T> *>(z + (Long)plane * g.oH * g.oW);
        const int r0 = (int)kr * dH - pH, q0 = (int)kc * dW - pW;
        for (unsigned v = threadIdx.x; v < vecs; v += kBlock) {
            unsigned vc;
            const unsigned orow = dRow.divmod(v, vc);
            const int r = r0 + (int)orow * sH;
            Pack<T> o;
#pragma unroll
            for (int k = 0; k < N; k++) {
                const int q = q0 + ((int)vc * N + k) * sW;
                o.v[k] = (inRange(r, g.iH) && inRange(q, g.iW)) ? image[r * g.imS[2] + q * g.imS[3]] : fromCompute<T>(0);
            }
            storePack(out + v, o);
        }
    }
}

// With many (batch, channel) pairs a block (or up to four: blockIdx.y) takes a whole channel: its kH * kW result planes as one list of vectors (a
// plane alone is rarely a whole number of rounds of the block: 784 vectors of a 56 x 56 plane leave the fourth round of
// 256 threads nearly empty), all of them reading the one image plane, which stays in the unit's cache.  Offsets are
// 32-bit (the host has checked the spans).  dAux: vectors per result row, dAux2: vectors per plane.
template <typename T>
__global__ void __launch_bounds__(kBlock) im2colChannelKernel(const T *x, T *z, const T *extra, ConvGeometry g, unsigned channels) {
    constexpr int N = Pack<T>::N;
    const int sH = paramInt(extra, 2), sW = paramInt(extra, 3), pH = paramInt(extra, 4), pW = paramInt(extra, 5);
    const int dH = paramInt(extra, 6), dW = paramInt(extra, 7);
    const unsigned vecsPerRow = (unsigned)g.oW / N, vecs = vecsPerRow * (unsigned)g.oH;
    const unsigned all = vecs * (unsigned)(g.kH * g.kW);
    const int is2 = (int)g.imS[2], is3 = (int)g.imS[3];
    for (unsigned ch = blockIdx.x; ch < channels; ch += gridDim.x) {
        unsigned c;
        const unsigned b = g.dIC.divmod(ch, c);
        const T *image = x + (int)(b * (unsigned)g.imS[0] + c * (unsigned)g.imS[1]);
        Pack<T> *out = reinterpret_cast<Pack<T> *>(z + (Long)ch * all * N);
        // four vectors per thread and round, all their loads before the first store (the compiler must assume that a store
        // to z changes the image, so it does not start the next vector's loads by itself: one vector per trip waits out a
        // memory latency per trip)
        for (unsigned v0 = blockIdx.y * (4 * kBlock) + threadIdx.x; v0 < all; v0 += gridDim.y * (4 * kBlock)) {
            Pack<T> o[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const unsigned v = v0 + u * kBlock;
                if (v < all) {
                    unsigned within, kc, vc;
                    const unsigned cell = g.dAux2.divmod(v, within);
                    const unsigned kr = g.dKW.divmod(cell, kc);
                    const unsigned orow = g.dAux.divmod(within, vc);
                    const int r = (int)kr * dH - pH + (int)orow * sH;
                    const int q0 = (int)kc * dW - pW + (int)(vc * N) * sW;
                    const bool rowIn = inRange(r, g.iH);
                    const T *line = image + r * is2;
                    if (sW == 1 && is3 == 1 && rowIn && q0 >= 0 && q0 + N <= g.iW) {
                        // the vector's N image elements lie side by side: one 16-byte load at whatever alignment they have
                        // (element by element the vector cache serves four requests a vector, and sets the pace)
                        o[u] = loadPackAnywhere(line + q0);
                    } else {
#pragma unroll
                        for (int k = 0; k < N; k++) {
                            const int q = q0 + k * sW;
                            o[u].v[k] = (rowIn && inRange(q, g.iW)) ? line[q * is3] : fromCompute<T>(0);
                        }
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (v0 + u * kBlock < all) storePack(out + v0 + u * kBlock, o[u]);
        }
    }
}

template <typename T> void launchIm2col(hipStream_t s, const T *x, T *z, const T *extra, const ConvGeometry &g) {
    const Long total = (Long)g.bS * g.iC * g.kH * g.kW * g.oH * g.oW;
    if (total <= 0) return;
    constexpr int N = Pack<T>::N;
    const Long plane = (Long)g.oH * g.oW;
    const bool dense = g.colS[5] == 1 && g.colS[4] == g.oW && g.colS[3] == plane && g.colS[2] == plane * g.kW &&
                       g.colS[1] == plane * g.kW * g.kH && g.colS[0] == plane * g.kW * g.kH * g.iC;
    if (dense && g.oW % N == 0 && (reinterpret_cast<uintptr_t>(z) & 15) == 0) {
        const Long planes = total / plane;
        ConvGeometry gv = g;
        gv.dAux = FastDiv((unsigned)(g.oW / N));
        const Long perChannel = (Long)g.kH * g.kW, channels = planes / perChannel;
        if (channels >= 1024 && plane / N * perChannel < (1LL << 31)) {
            gv.dAux2 = FastDiv((unsigned)(plane / N));
            // (a channel's rounds of four vectors per thread go to up to four blocks: a 3 x 3 window over [32, 64, 56, 56]
            // takes 44.6 us with one block per channel, 42.8 with two, 42.5 with four, 43.2 with seven)
            const Long rounds = (plane / N * perChannel + 4 * kBlock - 1) / (4 * kBlock);
            const unsigned parts = (unsigned)(rounds >= 8 ? 4 : (rounds >= 2 ? rounds / 2 : 1));
            ND4J_LAUNCH(im2colChannelKernel<T>, dim3(gridFor(channels, 1), parts), dim3(kBlock), 0, s, x, z, extra, gv, (unsigned)channels);
            return;
        }
        gv.dAux2 = FastDiv((unsigned)perChannel);
        // workgroups for whole rounds of eight channels; in one launch when that fits, else in plain order
        const Long byDie = (channels + 7) / 8 * 8 * perChannel;
        if (byDie <= kWholeGrid)
            ND4J_LAUNCH(im2colPlaneKernel<T>, dim3((unsigned)byDie), dim3(kBlock), 0, s, x, z, extra, gv, (unsigned)planes,
                               (unsigned)byDie, 1);
        else
            ND4J_LAUNCH(im2colPlaneKernel<T>, dim3(gridFor(planes, 1)), dim3(kBlock), 0, s, x, z, extra, gv, (unsigned)planes,
                               (unsigned)planes, 0);
        return;
    }
    ND4J_LAUNCH(im2colKernel<T>, dim3(gridFor(total)), dim3(kBlock), 0, s, x, z, extra, g, (unsigned)total);
}

// ---- Col2Im ----------------------------------------------------------------------------------------------------
// z[b, c, h, w] = sum of the column entries that im2col would have read from (h, w), added one after the other in the
// order (kr, kc) the reference's scatter loop reaches them (for one (kr, kc) at most one output position maps to a
// pixel).  extra = [sH, sW, pH, pW, iH, iW, dH, dW].  ACCUMULATE: start from what z holds instead of from zero.
// The output position that reads a pixel through kernel cell (kr, kc) is (pixel + padding - cell * dilation) / stride when
// that divides.  The strides sit in device memory, so the compiler sees divisions by unknowns, a dozen per pixel, which
// cost more than the memory traffic: strides that are powers of two (1 included) go by shifts instead - the kernel picks
// its loop once, the same for every lane.
// The cells of the kernel window are taken kCellBatch at a time: first the loads of a batch, all of them in flight
// together, then the additions in the reference's order.  (One load per trip of a loop whose bounds the compiler does not
// know waits for each value before it asks for the next: a pixel then costs nine memory latencies in a row.)
// Offsets are 32-bit: the host has checked that both arrays span fewer than 2^31 elements, and 64-bit products of a
// lane's index and a stride are what this kernel would otherwise spend its time on.
// A compute unit has one scalar unit, and with window extents that are only known at run time the bookkeeping of the
// window (cell counters, their comparisons and branches, all the same for every lane, so all scalar) came to 48 scalar
// instructions per element and set the pace.  The usual windows (1x1, 2x2, 3x3, 5x5) are therefore compiled in (KH, KW > 0):
// their cells are constants and the batch is the whole window.
static constexpr int kCellBatch = 16;
template <typename T, bool SHIFTS, int KH, int KW>
__device__ __forceinline__ typename Compute<T>::type col2imPixel(typename Compute<T>::type acc, const T *col, const ConvGeometry &g, int h, int w,
                                                                 int sH, int sW, int pH, int pW, int dH, int dW, int shH, int shW) {
    typedef typename Compute<T>::type C;
    const int cs2 = (int)g.colS[2], cs3 = (int)g.colS[3], cs4 = (int)g.colS[4], cs5 = (int)g.colS[5];
    if constexpr (KH > 0) {
        constexpr int CELLS = KH * KW;
        C v[CELLS];
        bool ok[CELLS];
#pragma unroll
        for (int u = 0; u < CELLS; u++) {
            const int kr = u / KW, kc = u % KW;
            const int hh = h + pH - kr * dH, ww = w + pW - kc * dW;
            const int orow = SHIFTS ? hh >> shH : (hh >= 0 ? hh / sH : 0), ocol = SHIFTS ? ww >> shW : (ww >= 0 ? ww / sW : 0);
            ok[u] = hh >= 0 && ww >= 0 && orow * sH == hh && ocol * sW == ww && orow < g.oH && ocol < g.oW;
            v[u] = ok[u] ? toCompute(col[kr * cs2 + kc * cs3 + orow * cs4 + ocol * cs5]) : (C)0;
        }
#pragma unroll
        for (int u = 0; u < CELLS; u++)
            if (ok[u]) acc = stored<T>(acc + v[u]);
        return acc;
    } else {
        const int cells = g.kH * g.kW;
        int kr = 0, kc = 0;  // the cell's row and column in the window (the same for every lane)
        for (int cell0 = 0; cell0 < cells; cell0 += kCellBatch) {
            C v[kCellBatch];
            bool ok[kCellBatch];
#pragma unroll
            for (int u = 0; u < kCellBatch; u++) {
                ok[u] = false;
                v[u] = (C)0;
                if (cell0 + u < cells) {  // (a branch of the whole wave)
                    const int hh = h + pH - kr * dH, ww = w + pW - kc * dW;
                    const int orow = SHIFTS ? hh >> shH : (hh >= 0 ? hh / sH : 0), ocol = SHIFTS ? ww >> shW : (ww >= 0 ? ww / sW : 0);
                    ok[u] = hh >= 0 && ww >= 0 && orow * sH == hh && ocol * sW == ww && orow < g.oH && ocol < g.oW;
                    if (ok[u]) v[u] = toCompute(col[kr * cs2 + kc * cs3 + orow * cs4 + ocol * cs5]);
                    if (++kc == g.kW) { kc = 0; kr++; }
                }
            }
#pragma unroll
            for (int u = 0; u < kCellBatch; u++)
                if (ok[u]) acc = stored<T>(acc + v[u]);
        }
        return acc;
    }
}
template <typename T, bool ACCUMULATE, int KH, int KW>
__global__ void __launch_bounds__(kBlock) col2imKernel(const T *x, T *z, const T *extra, ConvGeometry g, unsigned total) {
    typedef typename Compute<T>::type C;
    const int sH = paramInt(extra, 0), sW = paramInt(extra, 1), pH = paramInt(extra, 2), pW = paramInt(extra, 3);
    const int iH = paramInt(extra, 4), iW = paramInt(extra, 5), dH = paramInt(extra, 6), dW = paramInt(extra, 7);
    const bool shifts = sH > 0 && sW > 0 && (sH & (sH - 1)) == 0 && (sW & (sW - 1)) == 0;
    const int shH = shifts ? __builtin_ctz((unsigned)sH) : 0, shW = shifts ? __builtin_ctz((unsigned)sW) : 0;
    for (unsigned i = blockIdx.x * kBlock + threadIdx.x; i < total; i += gridDim.x * kBlock) {
        unsigned t = i, w, h, c;
        t = g.dIW.divmod(t, w);
        t = g.dIH.divmod(t, h);
        const unsigned b = g.dIC.divmod(t, c);
        T *out = z + (int)(b * (unsigned)g.imS[0] + c * (unsigned)g.imS[1] + h * (unsigned)g.imS[2] + w * (unsigned)g.imS[3]);
        C acc = ACCUMULATE ? toCompute(*out) : (C)0;
        if ((int)h < iH && (int)w < iW) {
            const T *col = x + (int)(b * (unsigned)g.colS[0] + c * (unsigned)g.colS[1]);
            if (shifts) acc = col2imPixel<T, true, KH, KW>(acc, col, g, (int)h, (int)w, sH, sW, pH, pW, dH, dW, shH, shW);
            else acc = col2imPixel<T, false, KH, KW>(acc, col, g, (int)h, (int)w, sH, sW, pH, pW, dH, dW, shH, shW);
        }
        *out = fromCompute<T>(acc);
    }
}

__global__ void __launch_bounds__(kBlock) clearBytesKernel(U32x4 *p, Long vectors, unsigned char *tail, int tailBytes) {
    const U32x4 zero = {0u, 0u, 0u, 0u};
    const Long gtid = (Long)blockIdx.x * kBlock + threadIdx.x;
    for (Long v = gtid; v < vectors; v += (Long)gridDim.x * kBlock) p[v] = zero;
    if (gtid < tailBytes) tail[gtid] = 0;
}

template <typename T> void launchCol2im(hipStream_t s, const T *x, T *z, const T *extra, const ConvGeometry &g, Long clearFirst) {
    const Long total = (Long)g.bS * g.iC * g.iH * g.iW;
    if (total <= 0) return;
    if (clearFirst > 0) {
        // the reference clears the first length(z) elements of z's buffer whatever z's strides are, and adds onto the rest
        unsigned char *base = reinterpret_cast<unsigned char *>(z);
        Long bytes = clearFirst * (Long)sizeof(T);
        Long lead = (Long)((16 - (reinterpret_cast<uintptr_t>(base) & 15)) & 15);
        if (lead > bytes) lead = bytes;
        if (lead > 0) ND4J_LAUNCH(clearBytesKernel, dim3(1), dim3(kBlock), 0, s, nullptr, 0, base, (int)lead);
        const Long vectors = (bytes - lead) / 16;
        const int tailBytes = (int)(bytes - lead - vectors * 16);
        ND4J_LAUNCH(clearBytesKernel, dim3(gridFor(vectors + 1)), dim3(kBlock), 0, s, reinterpret_cast<U32x4 *>(base + lead), vectors,
                           base + lead + vectors * 16, tailBytes);
    }
    const dim3 grid(gridFor(total, kBlock * 2));  // two pixels to a thread, one after the other
#define ND4J_COL2IM(KH, KW)                                                                                                   \
    do {                                                                                                                      \
        if (clearFirst > 0) ND4J_LAUNCH((col2imKernel<T, true, KH, KW>), grid, dim3(kBlock), 0, s, x, z, extra, g, (unsigned)total);  \
        else ND4J_LAUNCH((col2imKernel<T, false, KH, KW>), grid, dim3(kBlock), 0, s, x, z, extra, g, (unsigned)total);                \
    } while (0)
    if (g.kH == 3 && g.kW == 3) ND4J_COL2IM(3, 3);
    else if (g.kH == 1 && g.kW == 1) ND4J_COL2IM(1, 1);
    else if (g.kH == 2 && g.kW == 2) ND4J_COL2IM(2, 2);
    else if (g.kH == 5 && g.kW == 5) ND4J_COL2IM(5, 5);
    else ND4J_COL2IM(0, 0);
#undef ND4J_COL2IM
}

// ---- Pooling2D -------------------------------------------------------------------------------------------------
// extra = [kH, kW, sH, sW, pH, pW, dH, dW, -, mode, p]: mode 0 maximum (from -1e37, the reference's MAX_FLOAT), 1 average
// (p == 0: over the cells inside the image, p == 1: over kH * kW), 2 p-norm.  One thread per result element; the window
// is clipped to the image in steps of the dilation, as the reference clips it.
// The window's cells for the usual 2x2 and 3x3 windows without dilation, compiled in (see col2imPixel: loops whose bounds
// differ from lane to lane cost a round of exec-mask bookkeeping on the one scalar unit per trip): all loads first, a
// cell counting when it lies inside the image, which is what the clipped bounds select; then the reference's order.
template <typename T, int KH, int KW>
__device__ __forceinline__ typename Compute<T>::type poolCells(typename Compute<T>::type acc, const T *in, int hs0, int ws0, int iH, int iW,
                                                               int is2, int is3, int mode, typename Compute<T>::type p0) {
    typedef typename Compute<T>::type C;
    C v[KH * KW];
    bool ok[KH * KW];
    if (KW == 2 && is3 == 1 && ws0 >= 0 && ws0 + 2 <= iW) {
        // both cells of a window row lie side by side inside the image: one load of two elements (element by element a
        // wave asks the vector cache for every line twice, and its request rate sets the pace)
        struct __attribute__((packed, aligned(sizeof(T)))) Two { T a, b; };
#pragma unroll
        for (int r = 0; r < KH; r++) {
            const int ky = hs0 + r;
            ok[2 * r] = ok[2 * r + 1] = inRange(ky, iH);
            Two t = {fromCompute<T>(0), fromCompute<T>(0)};
            if (ok[2 * r]) t = *reinterpret_cast<const Two *>(in + ky * is2 + ws0);
            v[2 * r] = toCompute(t.a);
            v[2 * r + 1] = toCompute(t.b);
        }
    } else {
#pragma unroll
        for (int u = 0; u < KH * KW; u++) {
            const int ky = hs0 + u / KW, kx = ws0 + u % KW;
            ok[u] = inRange(ky, iH) && inRange(kx, iW);
            v[u] = ok[u] ? toCompute(in[ky * is2 + kx * is3]) : (C)0;
        }
    }
#pragma unroll
    for (int u = 0; u < KH * KW; u++)
        if (ok[u]) {
            if (mode == 0) { if (v[u] > acc) acc = v[u]; }
            else if (mode == 1) acc = stored<T>(acc + v[u]);
            else if (mode == 2) acc = stored<T>(acc + stored<T>(m::pow_(m::abs_(v[u]), p0)));
        }
    return acc;
}

// 2 x 2 windows, stride 2, no padding or dilation, unit innermost strides: OUT neighbouring results per thread from 2 OUT
// input elements of each of two image rows.  Same order of operations per result as the general path: upper row left,
// right, lower row left, right.
template <typename T, int OUT>
__device__ __forceinline__ void pool2x2(const T *x, T *z, const ConvGeometry &g, int mode, typename Compute<T>::type p0, unsigned total) {
    typedef typename Compute<T>::type C;
    constexpr int N = Pack<T>::N, PACKS = 2 * OUT / N;
    static_assert(PACKS >= 1 && 2 * OUT % N == 0, "whole vectors per row");
    const int is2 = (int)g.imS[2];
    const C div = ((int)p0 == 0 || (int)p0 == 1) ? (C)4 : (C)0;
    for (unsigned j = blockIdx.x * kBlock + threadIdx.x; j < total / OUT; j += gridDim.x * kBlock) {
        unsigned t = j * OUT, xx, yy, c;
        t = g.dOW.divmod(t, xx);
        t = g.dOH.divmod(t, yy);
        const unsigned b = g.dIC.divmod(t, c);
        const T *in = x + (int)(b * (unsigned)g.imS[0] + c * (unsigned)g.imS[1]) + (int)(2 * yy) * is2 + (int)(2 * xx);
        Pack<T> up[PACKS], low[PACKS];
#pragma unroll
        for (int q = 0; q < PACKS; q++) {
            up[q] = loadPackAnywhere(in + q * N);
            low[q] = loadPackAnywhere(in + is2 + q * N);
        }
        T *out = z + (int)(b * (unsigned)g.colS[0] + c * (unsigned)g.colS[1] + yy * (unsigned)g.colS[2] + xx);
        T r[OUT];
#pragma unroll
        for (int k = 0; k < OUT; k++) {
            const int h = (2 * k) / N, e = (2 * k) % N;
            const C v0 = toCompute(up[h].v[e]), v1 = toCompute(up[h].v[e + 1]), v2 = toCompute(low[h].v[e]), v3 = toCompute(low[h].v[e + 1]);
            C acc;
            if (mode == 0) {
                acc = (C)-1e37;
                if (v0 > acc) acc = v0;
                if (v1 > acc) acc = v1;
                if (v2 > acc) acc = v2;
                if (v3 > acc) acc = v3;
            } else if (mode == 1) {
                acc = stored<T>(stored<T>(stored<T>(stored<T>((C)0 + v0) + v1) + v2) + v3) / div;
            } else {
                acc = (C)0;  // (what the general path leaves for a mode it does not know)
            }
            r[k] = fromCompute<T>(acc);
        }
        if constexpr (OUT == N) {
            Pack<T> o;
#pragma unroll
            for (int k = 0; k < N; k++) o.v[k] = r[k];
            streamPackAnywhere(out, o);
        } else {
#pragma unroll
            for (int k = 0; k < OUT; k++) out[k] = r[k];
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(kBlock) pooling2dKernel(const T *x, T *z, const T *extra, ConvGeometry g, unsigned total) {
    typedef typename Compute<T>::type C;
    const int kH = paramInt(extra, 0), kW = paramInt(extra, 1), sH = paramInt(extra, 2), sW = paramInt(extra, 3);
    const int pH = paramInt(extra, 4), pW = paramInt(extra, 5), dH = paramInt(extra, 6), dW = paramInt(extra, 7);
    const int mode = paramInt(extra, 9);
    if (mode == 2) lm::loadTables();  // the p-norm's powf (the same decision in every thread of the grid)
    const C p0 = toCompute(extra[10]);
    const int kHEff = kH + (kH - 1) * (dH - 1), kWEff = kW + (kW - 1) * (dW - 1);
    constexpr int N = Pack<T>::N;
    if (mode != 2 && kH == 2 && kW == 2 && sH == 2 && sW == 2 && pH == 0 && pW == 0 && dH == 1 && dW == 1 && g.imS[3] == 1 &&
        g.colS[3] == 1 && 2 * g.oW <= g.iW && 2 * g.oH <= g.iH) {
        // The everyday case, 2 x 2 windows side by side: a thread takes N neighbouring results - one 16-byte store, four
        // 16-byte loads at whatever alignment the rows have - or N / 2 (two loads) when the result's rows do not hold whole
        // groups of N.
        if (g.oW % N == 0) { pool2x2<T, N>(x, z, g, mode, p0, total); return; }
        if (N >= 2 && g.oW % (N / 2) == 0) { pool2x2<T, (N >= 2 ? N / 2 : 1)>(x, z, g, mode, p0, total); return; }
    }
    for (unsigned i = blockIdx.x * kBlock + threadIdx.x; i < total; i += gridDim.x * kBlock) {
        unsigned t = i, xx, yy, c;
        t = g.dOW.divmod(t, xx);
        t = g.dOH.divmod(t, yy);
        const unsigned b = g.dIC.divmod(t, c);
        int hs = (int)yy * sH - pH, ws = (int)xx * sW - pW, he = hs + kHEff, we = ws + kWEff;
        // (without dilation, the usual case and the same for every lane, the clipping needs no division)
        if (dH == 1) { hs = hs < 0 ? 0 : hs; he = he > g.iH ? g.iH : he; }
        else {
            if (hs < 0) hs += ((-hs + dH - 1) / dH) * dH;
            if (he > g.iH) he -= ((he - g.iH + dH - 1) / dH) * dH;
        }
        if (dW == 1) { ws = ws < 0 ? 0 : ws; we = we > g.iW ? g.iW : we; }
        else {
            if (ws < 0) ws += ((-ws + dW - 1) / dW) * dW;
            if (we > g.iW) we -= ((we - g.iW + dW - 1) / dW) * dW;
        }
        const T *in = x + (int)(b * (unsigned)g.imS[0] + c * (unsigned)g.imS[1]);  // (offsets fit 32 bits: the host has checked the spans)
        C acc = mode == 0 ? (C)-1e37 : (C)0;
        const int is2 = (int)g.imS[2], is3 = (int)g.imS[3];
        const int hs0 = (int)yy * sH - pH, ws0 = (int)xx * sW - pW;
        if (dH == 1 && dW == 1 && kH == 2 && kW == 2) acc = poolCells<T, 2, 2>(acc, in, hs0, ws0, g.iH, g.iW, is2, is3, mode, p0);
        else if (dH == 1 && dW == 1 && kH == 3 && kW == 3) acc = poolCells<T, 3, 3>(acc, in, hs0, ws0, g.iH, g.iW, is2, is3, mode, p0);
        else
        for (int ky = hs; ky < he; ky += dH)
            for (int kx = ws; kx < we; kx += dW) {
                const C v = toCompute(in[ky * is2 + kx * is3]);
                if (mode == 0) { if (v > acc) acc = v; }
                else if (mode == 1) acc = stored<T>(acc + v);
                else if (mode == 2) acc = stored<T>(acc + stored<T>(m::pow_(m::abs_(v), p0)));
            }
        if (mode == 1) {
            // ceil((he - hs) / dH) * ceil((we - ws) / dW), also where clipping has turned a window inside out
            int rowsIn = he - hs, colsIn = we - ws;
            if (dH != 1) rowsIn = he >= hs ? (he - hs + dH - 1) / dH : -((hs - he) / dH);
            if (dW != 1) colsIn = we >= ws ? (we - ws + dW - 1) / dW : -((ws - we) / dW);
            int div = 0;
            if ((int)p0 == 0) div = rowsIn * colsIn;
            else if ((int)p0 == 1) div = kH * kW;
            acc = acc / (C)div;
        } else if (mode == 2) {
            acc = m::pow_(acc, stored<T>((C)1 / p0));
        }
        z[(int)(b * (unsigned)g.colS[0] + c * (unsigned)g.colS[1] + yy * (unsigned)g.colS[2] + xx * (unsigned)g.colS[3])] = fromCompute<T>(acc);
    }
}

template <typename T> void launchPooling2d(hipStream_t s, const T *x, T *z, const T *extra, const ConvGeometry &g) {
    const Long total = (Long)g.bS * g.iC * g.oH * g.oW;
    if (total <= 0) return;
    // (a vector's worth of results to a thread: what the 2 x 2 path takes per thread, so that none of its blocks starts for
    // nothing - 47 -> 45 us over a [64, 64, 112, 112] image against two results per thread; the general path walks its
    // share in a loop)
    ND4J_LAUNCH(pooling2dKernel<T>, dim3(gridFor(total, kBlock * Pack<T>::N)), dim3(kBlock), 0, s, x, z, extra, g, (unsigned)total);
}

// ---- DropOut 43 / DropOutInverted 44 as transforms ---------------------------------------------------------------
// z = rnd >= p ? 0 : x (inverted: x / p) with rnd uniform in [0, 1).  The reference draws rnd from the C library's
// unseeded rand() on the CPU and from the clock on CUDA (include/ops/ops.h:3520-3562), so no two of its runs agree;
// here rnd is a hash of the element's index and a per-call seed.
__device__ __forceinline__ float unitHash(unsigned long long v) {
    v += 0x9e3779b97f4a7c15ull;
    v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ull;
    v = (v ^ (v >> 27)) * 0x94d049bb133111ebull;
    v ^= v >> 31;
    return (float)(v >> 40) * (1.0f / 16777216.0f);
}
template <typename T, bool INVERTED>
__global__ void __launch_bounds__(kBlock) dropoutTransformKernel(const T *x, DimMap xm, T *z, DimMap zm, const T *extra, Long n,
                                                                 unsigned long long seed) {
    typedef typename Compute<T>::type C;
    const C prob = toCompute(extra[0]);
    for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += (Long)gridDim.x * kBlock) {
        const C v = toCompute(x[mapOffsetAny(xm, i)]);
        const C rnd = (C)unitHash(seed + (unsigned long long)i);
        z[mapOffsetAny(zm, i)] = fromCompute<T>(rnd >= prob ? (C)0 : (INVERTED ? v / prob : v));
    }
}
template <typename T>
void launchDropoutTransform(hipStream_t s, bool inverted, const T *x, const DimMap &xm, T *z, const DimMap &zm, const T *extra,
                            Long n, unsigned long long seed) {
    if (n <= 0) return;
    if (inverted)
        ND4J_LAUNCH((dropoutTransformKernel<T, true>), dim3(gridFor(n)), dim3(kBlock), 0, s, x, xm, z, zm, extra, n, seed);
    else
        ND4J_LAUNCH((dropoutTransformKernel<T, false>), dim3(gridFor(n)), dim3(kBlock), 0, s, x, xm, z, zm, extra, n, seed);
}

#define INST(T)                                                                                                   \
    template void launchDropoutTransform<T>(hipStream_t, bool, const T *, const DimMap &, T *, const DimMap &, const T *, Long, \
                                            unsigned long long);                                                  \
    template void launchReverse<T>(hipStream_t, const T *, T *, const ReversePlan &);                             \
    template void launchHistogram<T>(hipStream_t, const T *, Long, T *, int, const T *, unsigned *);              \
    template void launchIm2col<T>(hipStream_t, const T *, T *, const T *, const ConvGeometry &);                  \
    template void launchCol2im<T>(hipStream_t, const T *, T *, const T *, const ConvGeometry &, Long);            \
    template void launchPooling2d<T>(hipStream_t, const T *, T *, const T *, const ConvGeometry &);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
