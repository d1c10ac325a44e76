// Host runtime shared by the boundary translation units: environment switches, extraPointers decoding,
// shapeInfo fetching, the per-stream workspace and the TAD cache.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "launch.h"
#include "shape_host.h"
#include "types.h"

namespace nd4j_amd {

// Runtime switches, the counterpart of nd4j::Environment (reference: blas/Environment.cpp:13-33).
struct Environment {
    std::atomic<bool> debug{false};
    std::atomic<bool> verbose{false};
    std::atomic<int> elementThreshold{1024};
    std::atomic<int> tadThreshold{8};
    std::atomic<int> gridLimit{8192};
    std::atomic<int> maxThreads{512};
};
Environment &environment();

// extraPointers slots of the reference's CUDA convention (blas/cuda/NativeOps.cu:1609-1624,1813-1823).
enum ExtraSlot {
    X_HOST_X_SHAPE = 0,
    X_STREAM = 1,
    X_DEVICE_ID = 2,
    X_ALLOCATION = 3,
    X_REDUCTION = 4,
    X_RESULT = 5,
    X_SPECIAL = 6,
    X_HOST_Y_SHAPE = 7,
    X_HOST_Z_SHAPE = 8,
    X_HOST_TAD_SHAPE = 9,
    X_DEV_TAD_SHAPE = 10,
    X_DEV_TAD_OFFSETS = 11,
    X_DEV_TAD_SHAPE_Z = 12,
    X_DEV_TAD_OFFSETS_Z = 13,
};

inline hipStream_t streamOf(Nd4jPointer *extra) { return extra ? reinterpret_cast<hipStream_t>(extra[X_STREAM]) : nullptr; }
inline void *slotOf(Nd4jPointer *extra, int slot) { return extra ? extra[slot] : nullptr; }

// true when the pointer refers to device memory that the host must not dereference
bool isDeviceMemory(const void *p);

// Returns a host-readable shapeInfo: the host copy in extraPointers[slot] when present, else the
// argument itself when it is host memory, else a copy fetched from the device into `storage` (this
// last case synchronises the stream).  Null when there is nothing to read.
const Long *hostShapeInfo(Nd4jPointer *extra, int slot, const Long *arg, std::vector<Long> &storage, hipStream_t s);

// How often hostShapeInfo / hostInts had to fetch from the device since the library was loaded: a caller that
// passes the host copies and TAD tables of the CUDA convention keeps this at zero on the array-result calls.
long long hostFetchCount();

// Host copy of a small int array argument (`dimension`), which is a device pointer on this convention.
bool hostInts(const int *arg, int count, std::vector<int> &out, hipStream_t s);

// Throws std::runtime_error when the launch failed; in debug mode also synchronises the stream and
// reports asynchronous errors (reference: include/helpers/DebugHelper.h:31-57, op_boilerplate.h:96-97).
void checkLaunch(const char *what, hipStream_t s);
// Synchronise + check, for scalar-returning members.
void syncAndCheck(const char *what, hipStream_t s);

void reportUnknownOp(const char *family, int opNum);

// Device scratch owned by the library, one per (device, stream), allocated on first use and kept.
Workspace workspaceFor(hipStream_t s, size_t minBytes);
// Adds the slots, counter and ticket of the one-launch whole-array reduction to `w`: a block of device memory per
// (device, stream) that only those reductions use, cleared when it is allocated.  Calls on one stream run one after the
// other, so they may share it (one host thread per stream: the ticket source is not synchronised).
void addFlatSlots(Workspace &w, hipStream_t s);
// true while `s` is being captured into a HIP graph
bool streamIsCapturing(hipStream_t s);
// 256 bytes of pinned, device-visible host memory per (device, stream): the kernels of the scalar-returning entry
// points write their result there (plainly at offset 0, and as ticket-tagged words at offset 128), so the host reads
// it without a copy.
void *pinnedScalarFor(hipStream_t s);
// The hand-over that goes with that slot: the tagged words and the next ticket of this (device, stream).  The kernel
// stores every 32 bits of the value together with the ticket in one 8-byte word; takeScalar returns once `bytes` bytes
// of the value have arrived that way, or, failing that, once the stream has drained (then it reads the plain copy), and
// throws on a HIP error: the host gets the value a few microseconds before the stream's own completion would reach it.
// Everything enqueued earlier on the stream has completed by then (stream order).  In debug mode it synchronises the
// stream instead.  One host thread per stream: two threads on one stream would share the slot and the tickets.
struct ScalarSignal {
    unsigned long long *words = nullptr;
    unsigned ticket = 0;
    const void *plain = nullptr;  // the start of the pinned block: the plainly stored copy of the value
    unsigned *fault = nullptr;    // the stream's fault word (see Workspace::fault)
};
ScalarSignal nextScalarSignal(hipStream_t s);
void takeScalar(const ScalarSignal &sig, hipStream_t s, const char *what, void *value, size_t bytes);

// Frees what the library keeps for a stream of the current device (workspace, reduction slots, pinned scalar block) once
// the stream has drained; a later call on the stream allocates afresh.  For hosts that create and destroy streams.
void releaseStreamResources(hipStream_t s);
// test aid: the last ticket handed out for the stream's reduction slots
void setSlotTicketForTesting(hipStream_t s, unsigned value);

// TAD tables resolved for a call: host shapeInfo of one TAD + device offsets.
struct ResolvedTad {
    const Long *hostInfo = nullptr;
    const Long *devOffsets = nullptr;
    Long numTads = 0;
    Long tadLength = 0;
    std::shared_ptr<const void> keep;  // keeps a cached table's host side alive while this call uses it
};
// Uses extraPointers[hostSlot]/[offsetSlot] when both are present; otherwise computes the TAD from the
// host xShapeInfo and `dimension` (fetched from the device if needed), uploads the offsets once and caches
// them by (shapeInfo, dimension).
bool resolveTad(Nd4jPointer *extra, int hostSlot, int offsetSlot, const Long *hostXInfo, const int *dimension,
                int dimLen, ResolvedTad &out, hipStream_t s);

// Whole-array special transforms reached through execTransform (opNums 38-41): SoftMax, SoftMaxDerivative,
// LogSoftMax, IsMax.  Returns false when opNum is not one of them.
template <typename T>
bool specialTransform(Nd4jPointer *extra, int opNum, T *x, const Long *hostXInfo, T *z, const Long *hostZInfo, T *params,
                      hipStream_t s);

// The other whole-array transforms reached through execTransform's shapeInfo form: Col2Im 36, Im2col 37, Histogram 48,
// Reverse 70, Pooling2D 71 (native_whole.cpp).  Returns false when opNum is not one of them; throws
// std::invalid_argument for arguments the op cannot take (wrong ranks, missing extraParams, 2^31 elements or more).
template <typename T>
bool wholeArrayTransform(int opNum, T *x, const Long *hostXInfo, T *z, const Long *hostZInfo, T *params, hipStream_t s);

// Whole-array reduce of a float array into z[0] (device) without allocating: see native_reduce.cpp.  Throws
// std::invalid_argument for what it does not accept (no host shapeInfo, more than 2^36 elements, unknown opNum).
void reduceFloatNoAlloc(Nd4jPointer *extra, int opNum, float *x, Long *xInfo, float *params, float *z);

}  // namespace nd4j_amd
