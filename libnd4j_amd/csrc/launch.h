// Interface between the host boundary (native_ops.cpp) and the kernel translation units.
// Every launcher enqueues on `stream` and returns false when opNum has no functor (the caller then
// reports it the way the reference does, op_boilerplate.h:1148: a printed error, output untouched).
#pragma once

#include <hip/hip_runtime.h>

#include "types.h"
#include "view.h"

namespace nd4j_amd {

// Every kernel launch of the library goes through this macro: with debug and verbose mode both on (enableDebugMode,
// enableVerboseMode) it prints the kernel and its launch dimensions first, as the reference's CUDA back end prints its
// launch parameters (blas/cuda/NativeOps.cu:195-196, 257, 282).
bool launchesAreVerbose();
void printLaunch(const char *kernel, dim3 grid, dim3 block, size_t ldsBytes);
#define ND4J_LAUNCH(kernel, grid, block, lds, stream, ...)                                        \
    do {                                                                                          \
        if (::nd4j_amd::launchesAreVerbose()) ::nd4j_amd::printLaunch(#kernel, grid, block, lds); \
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                        \
    } while (0)

// ---- elementwise -----------------------------------------------------------------------------------
template <typename T>
bool launchTransformStrided(hipStream_t stream, int opNum, const T *x, Long xs, T *z, Long zs, const T *extra, Long n);
template <typename T>
bool launchTransformGeneral(hipStream_t stream, int opNum, const T *x, const DimMap &xm, T *z, const DimMap &zm,
                            const T *extra, Long n);
// ys == 0 broadcasts y[0]
template <typename T>
bool launchPairwiseStrided(hipStream_t stream, int opNum, const T *x, Long xs, const T *y, Long ys, T *z, Long zs,
                           const T *extra, Long n);
template <typename T>
bool launchPairwiseGeneral(hipStream_t stream, int opNum, const T *x, const DimMap &xm, const T *y, const DimMap &ym,
                           T *z, const DimMap &zm, const T *extra, Long n);

struct BroadcastPlan {
    enum Kind { ROW, COL, GENERAL } kind;
    Long tadLength, numTads;
    Long tadEws, yEws, zEws;     // ROW / COL
    DimMap xm, ym, zm;           // GENERAL: element index inside the TAD -> offset
    const Long *xOffsets;        // device, numTads entries
    const Long *zOffsets;        // device, numTads entries
    bool consecutive = false;    // ROW only: TAD r starts at r * tadLength in x and in z (rows of a dense c-order array)
    bool denseAlike = false;     // ROW / COL: x and z are dense arrays of one layout, y is contiguous: memory position i of
                                 // either takes y[(i / tadEws) % tadLength]
    unsigned runLength = 0;      // GENERAL only, 0 = not applicable: the three maps end in contiguous runs of this many elements
    bool runMajor = false;       //   ... and the same run of neighbouring TADs is nearer in memory than the next run of one TAD
    // The whole call as one element-wise walk, when the host could state it so (wholeRun > 0): maps over all of x's
    // dimensions - y's with stride 0 along those that are not the TAD's - that end in contiguous runs of wholeRun elements;
    // wholeN elements in all.  Needs no offset tables.
    DimMap wx, wy, wz;
    Long wholeN = 0;
    unsigned wholeRun = 0;
    // GENERAL: x and z are dense arrays [A, slabMid, slabInner] walked as plain vectors, y a dense [A, slabInner]
    unsigned slabInner = 0, slabMid = 0;
    Long flatInner = 0, flatExtent = 0;  // per-TAD scalars over dense x and z of one layout: memory position i takes
                                         // scalars[(i / flatInner) % flatExtent]; 0 = not applicable
};
template <typename T>
bool launchBroadcast(hipStream_t stream, int opNum, const T *x, const T *y, T *z, const BroadcastPlan &plan);

// ---- scalar ----------------------------------------------------------------------------------------
template <typename T>
bool launchScalarStrided(hipStream_t stream, int opNum, const T *x, Long xs, T *z, Long zs,
                         typename Compute<T>::type scalar, const T *extra, Long n);
template <typename T>
bool launchScalarGeneral(hipStream_t stream, int opNum, const T *x, const DimMap &xm, T *z, const DimMap &zm,
                         typename Compute<T>::type scalar, const T *extra, Long n);
// one scalar per TAD: plan.kind ROW (tadEws == 1) or COL (tadEws > 1); yEws is unused
template <typename T>
bool launchScalarTad(hipStream_t stream, int opNum, const T *x, const T *scalars, T *z, const T *extra,
                     const BroadcastPlan &plan);

// ---- reductions ------------------------------------------------------------------------------------
// How the elements of one TAD are addressed and how TADs relate to each other.
struct TadPlan {
    enum Kind {
        ROW,      // tadEws == 1: lanes cooperate along a contiguous TAD
        COL,      // tadEws  > 1: one lane per TAD, rows of adjacent TADs coalesce
        GENERAL   // no element-wise stride: per-element coordinate map
    } kind;
    Long tadLength, numTads, tadEws;
    DimMap tm;               // GENERAL
    unsigned runLength = 0;  // GENERAL: extent of the map's innermost dimension when its stride is 1 (contiguous runs), else 0
    const Long *offsets;     // device, numTads entries
    // When the last dimension of x that the TADs do not take is its contiguous one: that dimension's extent (TADs
    // t .. t + keptInner - 1, t a multiple of keptInner, then start on consecutive elements), and the greatest common
    // divisor of x's other strides (what decides whether rows of such a group start on 16-byte boundaries).  0: not so.
    unsigned keptInner = 0;
    Long otherStrides = 0;
};

// Scratch for multi-block stages.  `bytes` is what the pointer is known to hold.
struct Workspace {
    void *ptr;
    size_t bytes;
    // Optional hand-over of a scalar result to a waiting host: the thread that stores the result also stores it, 32 bits
    // a word, into the 8-byte words at `signal` (host memory the device can write), each word tagged with `ticket` in
    // its upper half, so that the host may wait for the value itself instead of for the stream.  Null for array results.
    unsigned long long *signal = nullptr;
    unsigned ticket = 0;
    // Optional: what the whole-array reductions need to finish in one launch - `slotBytes` bytes of 8-byte slots that no
    // other kernel writes (zero when allocated), 16 KiB of block counters that are zero between calls, and tickets that differ
    // from launch to launch on this stream (never zero).  Without them the reduction takes a second, merging launch.
    unsigned long long *slots = nullptr;
    size_t slotBytes = 0;
    unsigned *counter = nullptr;
    unsigned *rowStates = nullptr;         // rowStateCount 32-bit words beside the slots, for launches that decide per row
    size_t rowStateCount = 0;
    unsigned *slotTicketSource = nullptr;  // host memory: the last ticket handed out for these slots
    // pinned host word the device can write: a merging block that gave up waiting for a slot stores 1 here (and NaN as
    // the result), which the host reports at its next look (null: nobody looks)
    unsigned *fault = nullptr;
    // the next ticket: every launch that uses the slots takes its own
    unsigned nextSlotTicket() const {
        unsigned t = ++*slotTicketSource;
        if (t == 0) t = ++*slotTicketSource;
        return t;
    }
};

// Full-array view for scalar reductions: either 1-D strided (ews >= 1) or a C-order coordinate map.
struct FlatPlan {
    Long n;
    bool strided;
    Long ews;
    DimMap xm;
};

template <typename T>
bool launchReduceTad(hipStream_t stream, int opNum, const T *x, const T *extra, T *z, const TadPlan &plan,
                     Workspace ws);
// writes the post-processed scalar to z[0] (device) and, if hostResult != nullptr, leaves it there for
// the caller to read after synchronising (hostResult must be device-visible pinned memory or null)
template <typename T>
bool launchReduceScalar(hipStream_t stream, int opNum, const T *x, const T *extra, T *z, const FlatPlan &plan,
                        Workspace ws);

// The whole-array reduction with its partial accumulators in a file-scope device array instead of a workspace: no
// device memory is allocated or freed.  Calls that overlap on one GPU share (and race on) that array.
// prepareNoAllocScratch looks the array's address up for the current device (the launch does so on its first call too).
void prepareNoAllocScratch();
bool launchReduceScalarNoAlloc(hipStream_t stream, int opNum, const float *x, const float *extra, float *z, const FlatPlan &plan);

template <typename T>
bool launchIndexReduceTad(hipStream_t stream, int opNum, const T *x, const T *extra, T *z, const TadPlan &plan,
                          Workspace ws);
template <typename T>
bool launchIndexReduceScalar(hipStream_t stream, int opNum, const T *x, const T *extra, T *z, const FlatPlan &plan,
                             Workspace ws);

template <typename T>
bool launchSummaryStatsTad(hipStream_t stream, int opNum, bool biasCorrected, bool phantomZero, const T *x, T *z,
                           const TadPlan &plan, Workspace ws);
template <typename T>
bool launchSummaryStatsScalar(hipStream_t stream, int opNum, bool biasCorrected, const T *x, T *z,
                              const FlatPlan &plan, Workspace ws);

// ---- reduce3 ---------------------------------------------------------------------------------------
// numOut results; result r pairs the run of x at xOffsets[r / xDiv] with the run of y at yOffsets[r % yMod]
// (a null table: offset 0); element f of a run sits at map(xm, f) / map(ym, f) behind the run's offset.
struct Reduce3Launch {
    Long runLength, numOut;
    Long xDiv, yMod;
    const Long *xOffsets;  // device
    const Long *yOffsets;  // device
    DimMap xm, ym;         // rank >= 1
    bool allPairs = false; // every run of x against every run of y (xDiv == yMod == runs of y): may be tiled
};
template <typename T>
bool launchReduce3(hipStream_t stream, int opNum, const T *x, const T *y, T *z, const T *extra, const Reduce3Launch &in,
                   Workspace ws);

// ---- special transforms ----------------------------------------------------------------------------
// numRows rows of `length` elements: row r starts at r * xRow (z: r * zRow), its elements are xEl (zEl) apart
struct SoftmaxPlan {
    Long numRows, length;
    Long xRow, xEl, zRow, zEl;
};
// opNum 38 SoftMax, 39 SoftMaxDerivative, 40 LogSoftMax
template <typename T> bool launchSoftmax(hipStream_t stream, int opNum, const T *x, T *z, const SoftmaxPlan &plan);
// For rows that do not fit the register-resident kernels of launchSoftmax (softmaxFitsRegisters false) and are few:
// launchSoftmaxStats (one pass of the reduction kernels, which cut long rows into slices) leaves the row maxima and the
// row sums of exp(x - max) (these in the compute type) in two per-row arrays, and launchSoftmaxFinish writes exp(x - max) / sum (38), its
// derivative p (1 - p) (39) or its logarithm (40)
template <typename T> bool softmaxFitsRegisters(const T *x, const T *z, const SoftmaxPlan &plan);
// The softmax family over contiguous rows (misaligned alike in x and z) that do not fit the register-resident kernels, in one pass:
// the blocks that hold the slices of a row exchange their maxima and sums through ws.slots.  False when the operands
// (or a workspace without slots) do not allow it; the caller then takes launchSoftmaxStats + launchSoftmaxFinish.
// How many polls a block of that kernel spends on a slice of its row that has not been published yet before it votes to
// abort the row (which the repair kernel then computes).  For tests of that path: 0 makes whatever is not there at the
// first look count as missing.  Default 5000.
void setCooperativeWaitLimit(int tries);
template <typename T> bool launchSoftmaxCooperative(hipStream_t stream, int opNum, const T *x, T *z, const SoftmaxPlan &plan, Workspace ws);
// The same exchange for an f-order matrix (rows adjacent in memory) with more columns than one block's slice of a group of
// rows: the blocks that share a group's columns cooperate.  True when the call was taken.
template <typename T> bool launchSoftmaxColCooperative(hipStream_t stream, int opNum, const T *x, T *z, const SoftmaxPlan &plan, Workspace ws);
template <typename T>
bool launchSoftmaxStats(hipStream_t stream, const T *x, T *maxima, typename Compute<T>::type *sums, const TadPlan &plan, Workspace ws);
template <typename T>
bool launchSoftmaxFinish(hipStream_t stream, int opNum, const T *x, T *z, const T *maxima, const typename Compute<T>::type *sums,
                         const SoftmaxPlan &plan);
// z = one-hot of the position stored (as a T) in index[0] / index[tad]; `zp` / `zt` walk z the way the index
// reduction walked x
template <typename T> void launchIsMaxFill(hipStream_t stream, T *z, const T *index, const FlatPlan &zp);
template <typename T> void launchIsMaxTadFill(hipStream_t stream, T *z, const T *index, const TadPlan &zt);

// ---- whole-array transforms (Col2Im 36, Im2col 37, Histogram 48, Reverse 70, Pooling2D 71) ---------------------
struct ReversePlan {
    Long n = 0;
    bool contiguous = false;  // x and z dense in one order (or x == z with unit stride): vector kernels
    bool swap = false;        // in place with an element-wise stride: exchange e and n - 1 - e for e < n / 2
    Long count = 0;           // mapped kernels: elements e < count are moved (n, or n / 2 in place)
    DimMap xm, zm;            // element e of x -> offset, element of z -> offset (each in its own order)
};
template <typename T> void launchReverse(hipStream_t stream, const T *x, T *z, const ReversePlan &plan);
// counts: histogramScratchBytes(..) of scratch; capacity = length of z (the bins that can be written)
template <typename T>
void launchHistogram(hipStream_t stream, const T *x, Long n, T *z, int capacity, const T *extra, unsigned *counts);
// bytes of `counts` that launchHistogram uses for n elements of the given size and a result of `capacity` bins
size_t histogramScratchBytes(Long n, int elementBytes, int capacity);
// An image [bS, iC, iH, iW] with strides imS, and either its column form [bS, iC, kH, kW, oH, oW] with strides colS
// (Im2col, Col2Im) or its pooled form [bS, iC, oH, oW] with strides colS[0..3] (Pooling2D).  Element counts stay below 2^31.
struct ConvGeometry {
    int bS, iC, iH, iW, kH, kW, oH, oW;
    Long imS[4], colS[6];
    FastDiv dOW, dOH, dKW, dKH, dIC, dIW, dIH;
    FastDiv dAux, dAux2;  // a launcher's own divisors (Im2col: 16-byte vectors per result row, planes per channel)
};
template <typename T> void launchIm2col(hipStream_t stream, const T *x, T *z, const T *extra, const ConvGeometry &g);
// clearFirst > 0: that many leading elements of z's buffer are cleared first and the sums are added onto what z holds
template <typename T> void launchCol2im(hipStream_t stream, const T *x, T *z, const T *extra, const ConvGeometry &g, Long clearFirst);
template <typename T> void launchPooling2d(hipStream_t stream, const T *x, T *z, const T *extra, const ConvGeometry &g);

// DropOut 43 / DropOutInverted 44 as transforms: element i of x (through xm) survives when a hash of (seed + i) falls
// below extra[0]
template <typename T>
void launchDropoutTransform(hipStream_t stream, bool inverted, const T *x, const DimMap &xm, T *z, const DimMap &zm,
                            const T *extra, Long n, unsigned long long seed);

// ---- data movement ---------------------------------------------------------------------------------
// The result of a concat as the kernel needs it: strides per dimension, the concatenated dimension, and for a
// contiguous C-order result the run geometry (inner = product of the dimensions after `dim`).
struct ConcatView {
    int rank, dim, zContig;
    Long zStride[kMaxDims];
    Long inner, dimTotal;
};
// Every pointer below is a device pointer (tables of pointers included), as in the reference's CUDA back end.
template <typename T>
void launchPullRows(hipStream_t stream, const T *x, T *z, Long n, const Long *indexes, const Long *tadInfo,
                    const Long *tadOffsets, const Long *zTadInfo, const Long *zTadOffsets);
template <typename T>
void launchTear(hipStream_t stream, const T *x, const Long *xInfo, T *const *targets, const Long *zInfo, const Long *tadInfo,
                const Long *tadOffsets, Long numTadsHint);
template <typename T>
void launchShuffle(hipStream_t stream, T *const *xs, const Long *const *xInfos, T *const *zs, int N, const int *map,
                   const Long *const *tadInfos, const Long *const *tadOffsets, Long numTadsHint);
// `scratch` is device memory of concatScratchBytes(numArrays) bytes; maxLength the element count of the largest input
size_t concatScratchBytes(int numArrays);
template <typename T>
void launchConcat(hipStream_t stream, const T *const *data, const Long *const *infos, T *z, const ConcatView &view,
                  int numArrays, Long maxLength, void *scratch);
// z[i * ews(zInfo)] = x[i * xe]; zInfo is a device shapeInfo, read by the kernel
template <typename T> void launchCopyToEws(hipStream_t stream, const T *x, Long xe, T *z, const Long *zInfo, Long n);
// z[r * zRowStride + c] = x[r + c * xColStride] for r < rows, c < cols, through LDS tiles
template <typename T>
void launchTransposeCopy(hipStream_t stream, const T *x, T *z, Long rows, Long cols, Long xColStride, Long zRowStride);
// z[i] = sum over the n buffers in the device table xs (average: / n); propagate: also written back to each of them
template <typename T> void launchAverage(hipStream_t stream, T *const *xs, T *z, int n, Long length, bool average, bool propagate);
// srcType / dstType: 3 half, 6 float, 7 double (type_conversions.h:11-18); false for any other pair
bool launchConvert(hipStream_t stream, int srcType, const void *x, Long n, int dstType, void *z);

// ---- random ----------------------------------------------------------------------------------------
// Device image of the generator state that getElement() needs (reference: helper_generator.h:61-74,
// 185-220).  Passed by value, so one op sees one consistent state.
struct RngState {
    const unsigned long long *buffer;  // device copy of the u64 buffer
    Long size;
    Long position;    // currentPosition
    Long generation;
    Long seed;
    Long amplifier;
    // Host-computed helpers for the divisions by launch-wide constants: 1 / size in double (quotient estimate
    // that the device corrects with the exact remainder) and floor((2^64 - 1) / d) for d = generation and
    // d = amplifier (0 when d < 1), which turn x / d into a 64-bit high multiplication plus one correction.
    double rSize;
    unsigned long long mGeneration, mAmplifier;
};
struct RandomPlan {
    Long n;
    // each operand: 1-D strided (ews >= 1 for all) or Fortran-order coordinate maps (cpu/random.cpp:46-76)
    bool strided;
    Long xEws, yEws, zEws;
    DimMap xm, ym, zm;
    Long yLength;  // Choice
};
template <typename T>
bool launchRandom(hipStream_t stream, int opNum, const RngState &rng, const T *x, const T *y, T *z, const T *args,
                  const RandomPlan &plan, int operands /* 1: z, 2: x,z, 3: x,y,z */, bool yIsZ);
// debugging / parity aid: out[i] = getElement(start + i)
void launchRngDump(hipStream_t stream, const RngState &rng, Long start, Long n, unsigned long long *out);
// plain copy with 16-byte vectors (bytes is rounded down to a multiple of 16 plus a byte tail)
void launchCopy(hipStream_t stream, void *dst, const void *src, Long bytes);
// measurement aid: copies an f-order float matrix in the tiles and block order of the cooperative f-order softmax kernel
void launchForderTileCopy(hipStream_t stream, const float *x, float *z, Long numRows, Long length);
// zero fill of `bytes` bytes (a multiple of 16, at a 16-byte boundary) by a kernel: safe to record where a memset node is not
void launchFill(hipStream_t stream, void *dst, size_t bytes);

}  // namespace nd4j_amd
