// Reduction skeletons shared by the reduce, index-reduce and summary-stats families.
//
// A policy `Pol` supplies the accumulator and its algebra:
//     typedef T (storage), C (compute), Acc
//     Acc  init(const T *first)            starting accumulator (may read the first element of the run)
//     void accumulate(Acc &, C v, Long i)  fold element i (its position inside the TAD / array)
//     Acc  combine(Acc a, Acc b)           merge two partial accumulators
//     T    finalize(Acc, Long n)           post-process into the stored result
//     void checkpoint(Acc &a)              called between groups of accumulate() calls; a policy may renormalise
//     void setTad(Long r)                  per-TAD hook (LogSumExp reads its shift from the result array)
//
// Kernels:
//   tadRowKernel<Pol, GROUP>  contiguous TADs (tadEws == 1): GROUP lanes walk one TAD with 16-byte loads,
//                             wave64 cross-lane merge, LDS only across waves.
//   tadColVecKernel<Pol>      strided TADs that are adjacent in memory: one lane per 16 bytes' worth of TADs,
//                             rows split over the waves of a block and over blockIdx.y (tadColFinish merges).
//   tadColKernel<Pol>         other strided TADs and short contiguous ones: one lane per TAD; the TAD length
//                             is split over blockIdx.y and merged by tadColFinish when split.
//   tadGeneralKernel<Pol>     block per TAD with a coordinate map.
//   flatKernel<Pol>           grid reduction over the whole array; the block that finishes last merges the blocks'
//                             results (flatFinish<Pol>: the same merge as a second launch, for callers without slots).
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "elementwise.cuh"
#include "types.h"
#include "view.h"

namespace nd4j_amd {

static constexpr int kWave = 64;

template <typename A> __device__ __forceinline__ A shflDownAny(A v, int delta) {
    static_assert(sizeof(A) % 4 == 0, "accumulator must be a multiple of 4 bytes");
    constexpr int W = sizeof(A) / 4;
    struct Words { int w[W]; };
    Words in = __builtin_bit_cast(Words, v);
    Words out;
#pragma unroll
    for (int i = 0; i < W; i++) out.w[i] = __shfl_down(in.w[i], delta, kWave);
    return __builtin_bit_cast(A, out);
}

// A policy may merge the lanes of a wave its own way (a member template waveMergeOwn<WIDTH>(acc), announced by a
// member constant ownWaveMerge): the summary statistics shuffle three of their seven doubles when they can.
template <class Pol, typename = void> struct HasOwnWaveMerge { static constexpr bool value = false; };
template <class Pol> struct HasOwnWaveMerge<Pol, decltype((void)Pol::ownWaveMerge)> { static constexpr bool value = Pol::ownWaveMerge; };

// A policy announces with a member constant kChains > 1 that a lane may keep several accumulators and combine() them.
template <class Pol, typename = void> struct PolChains { static constexpr int value = 1; };
template <class Pol> struct PolChains<Pol, decltype((void)Pol::kChains)> { static constexpr int value = Pol::kChains; };

// The most blocks a policy wants for the whole-array kernel (a member constant kFlatBlocks; kFlatMaxBlocks otherwise).
template <class Pol, typename = void> struct PolFlatBlocks { static constexpr int value = 2048; };
template <class Pol> struct PolFlatBlocks<Pol, decltype((void)Pol::kFlatBlocks)> { static constexpr int value = Pol::kFlatBlocks; };

// The blocks a policy wants in all for the strided vector kernel (a member constant kColBlocks; 2048 otherwise).
template <class Pol, typename = void> struct PolColBlocks { static constexpr int value = 2048; };
template <class Pol> struct PolColBlocks<Pol, decltype((void)Pol::kColBlocks)> { static constexpr int value = Pol::kColBlocks; };


// Folds an element whose index is higher than that of every element the accumulator has seen (the kernels walk their
// elements in ascending order wherever they can).  A policy may exploit that with a member accumulateAscending(): an
// index reduction then needs one comparison per element, where the general rule (better value, or the same value at a
// lower index) takes three and a handful of mask operations on the compute unit's one scalar unit - these kernels issued
// five scalar instructions per element of a wave that way, as many as a sum issues in all.
template <class Pol, typename = void> struct HasAscending { static constexpr bool value = false; };
template <class Pol> struct HasAscending<Pol, decltype((void)Pol::hasAscending)> { static constexpr bool value = Pol::hasAscending; };
template <class Pol>
__device__ __forceinline__ void foldNext(const Pol &pol, typename Pol::Acc &acc, typename Pol::C v, Long i) {
    if constexpr (HasAscending<Pol>::value) pol.accumulateAscending(acc, v, i);
    else pol.accumulate(acc, v, i);
}

// Merge over the lanes of one wave; lane 0 (of each WIDTH-lane segment) ends up with the result.
template <class Pol, int WIDTH = kWave>
__device__ __forceinline__ typename Pol::Acc waveMerge(const Pol &pol, typename Pol::Acc a) {
    if constexpr (HasOwnWaveMerge<Pol>::value) {
        return pol.template waveMergeOwn<WIDTH>(a);
    } else {
#pragma unroll
        for (int d = WIDTH / 2; d >= 1; d >>= 1) {
            typename Pol::Acc o = shflDownAny(a, d);
            a = pol.combine(a, o);
        }
        return a;
    }
}

// Merge over a whole 256-thread block; thread 0 gets the result.  `smem` holds kBlock/kWave accumulators.
template <class Pol>
__device__ __forceinline__ typename Pol::Acc blockMerge(const Pol &pol, typename Pol::Acc a, typename Pol::Acc *smem) {
    a = waveMerge<Pol>(pol, a);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    __syncthreads();  // smem may still be read from a previous round
    if (lane == 0) smem[wave] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kBlock / kWave; w++) a = pol.combine(a, smem[w]);
    }
    return a;
}

// Folds n contiguous elements starting at `p` (they are elements base, base + 1, .. of their run) using `lanes`
// cooperating lanes, this lane being `lane`.
template <class Pol>
__device__ __forceinline__ void foldContiguous(const Pol &pol, typename Pol::Acc &acc, const typename Pol::T *p, Long n,
                                               int lane, int lanes, Long base = 0) {
    typedef typename Pol::T T;
    constexpr int VEC = Pack<T>::N;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
    Long head = 0;
    if ((addr & (sizeof(T) - 1)) == 0) head = (Long)(((16 - (addr & 15)) & 15) / sizeof(T));
    else head = n;  // cannot be vectorised
    if (head > n) head = n;
    const Long nvec = (n - head) / VEC;
    // The elements before the first and after the last aligned vector (fewer than 2 VEC when the run can be vectorised at
    // all): one per lane, requested before the vectors so that a run costs one round trip to memory, not three.
    const Long tail0 = head + nvec * VEC, edges = head + (n - tail0);
    const bool oneEach = edges <= lanes;
    const bool hasEdge = oneEach && lane < edges;
    const Long edgeAt = lane < head ? lane : tail0 + (lane - head);
    T edge;
    if (hasEdge) edge = p[edgeAt];
    if (!oneEach) {
        for (Long i = lane; i < head; i += lanes) { pol.accumulate(acc, toCompute(p[i]), base + i); pol.checkpoint(acc); }
    }
    // (a lane's elements are folded in ascending order: its head element first, its tail element last)
    if (hasEdge && lane < head) { foldNext(pol, acc, toCompute(edge), base + edgeAt); pol.checkpoint(acc); }
    const Pack<T> *pv = reinterpret_cast<const Pack<T> *>(p + head);
    Long v = lane;
    // Four independent 16-byte loads in flight per lane, then the arithmetic.  Each of the four is guarded on its own: a
    // lane whose last batch is short still runs it with the rest of its wave (an all-or-nothing batch sent such lanes
    // through a second, vector-by-vector loop that the whole wave had to sit through; a separate unguarded copy of the
    // batch for the full ones measured slower again, for the code it adds).
    for (; v < nvec; v += 4 * (Long)lanes) {
        Pack<T> pk[4];
        // (the loads themselves are unconditional - a vector beyond the end re-reads the last one and is not folded: a
        // load inside a branch of its own makes the compiler wait for the loads before it, one round trip after the other)
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const Long vu = v + u * (Long)lanes;
            pk[u] = loadPack(pv + (vu < nvec ? vu : nvec - 1));
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (v + u * (Long)lanes < nvec) {
#pragma unroll
                for (int e = 0; e < VEC; e++) foldNext(pol, acc, toCompute(pk[u].v[e]), base + head + (v + u * (Long)lanes) * VEC + e);
                pol.checkpoint(acc);
            }
        }
    }
    if (hasEdge && lane >= head) { foldNext(pol, acc, toCompute(edge), base + edgeAt); pol.checkpoint(acc); }
    if (!oneEach) {
        for (Long i = tail0 + lane; i < n; i += lanes) { foldNext(pol, acc, toCompute(p[i]), base + i); pol.checkpoint(acc); }
    }
}

template <class Pol, int GROUP>
__global__ void __launch_bounds__(kBlock) tadRowKernel(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                       const Long *offsets, Long tadLength, Long numTads) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::Acc Acc;
    constexpr int GROUPS = kBlock / GROUP;
    __shared__ Acc smem[kBlock / kWave];
    const int g = threadIdx.x / GROUP, lane = threadIdx.x % GROUP;
    // GROUP == kBlock: every thread of the block runs the same trip count, so blockMerge may synchronise
    for (Long r0 = (Long)blockIdx.x * GROUPS; r0 < numTads; r0 += (Long)gridDim.x * GROUPS) {
        const Long r = r0 + g;
        const bool live = r < numTads;
        Acc acc;
        if (live) {
            pol.setTad(r, z);
            const typename Pol::T *tx = x + offsets[r];
            acc = pol.init(tx);
            foldContiguous<Pol>(pol, acc, tx, tadLength, lane, GROUP);
        }
        if (GROUP == kBlock) {
            acc = blockMerge<Pol>(pol, acc, smem);
        } else {
            if (live) acc = waveMerge<Pol, GROUP>(pol, acc);
        }
        if (live && lane == 0) z[r] = pol.finalize(acc, tadLength);
    }
}

// Strided TADs: thread t <-> TAD t, rows [rowsPerSplit * blockIdx.y, ...) of each TAD.
// MAPPED: TADs over several dimensions whose innermost one is strided (no vectors to be had along a TAD): element j of a
// TAD lies at the offset the coordinate map gives - the same for every lane, so one division chain serves the 64 TADs
// of a wave - and neighbouring TADs still coalesce wherever they are neighbours in memory.
template <class Pol, bool MAPPED = false>
__global__ void __launch_bounds__(kBlock) tadColKernel(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                       typename Pol::Acc *partials, const Long *offsets, Long tadLength,
                                                       Long numTads, Long tadEws, Long rowsPerSplit, DimMap tm = DimMap()) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::Acc Acc;
    const Long t = (Long)blockIdx.x * kBlock + threadIdx.x;
    if (t >= numTads) return;
    pol.setTad(t, z);
    const typename Pol::T *base = x + offsets[t];
    Acc acc = pol.init(base);
    // Split y takes the rows y, y + splits, y + 2 splits, ...: the blocks that run at the same time then read
    // neighbouring rows - one compact stretch of memory - instead of stretches a whole row range apart.
    (void)rowsPerSplit;
    const Long S = gridDim.y;
    Long j = blockIdx.y;
    auto at = [&](Long row) -> Long { return MAPPED ? mapOffset32(tm, (unsigned)row) : row * tadEws; };
    for (; j + 7 * S < tadLength; j += 8 * S) {
        typename Pol::T v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = base[at(j + u * S)];
#pragma unroll
        for (int u = 0; u < 8; u++) foldNext(pol, acc, toCompute(v[u]), j + u * S);
        pol.checkpoint(acc);
    }
    for (; j < tadLength; j += S) { foldNext(pol, acc, toCompute(base[at(j)]), j); pol.checkpoint(acc); }
    if (gridDim.y == 1) z[t] = pol.finalize(acc, tadLength);
    else partials[(Long)blockIdx.y * numTads + t] = acc;
}

// Hands a scalar result to a host that is waiting for it: the value goes out in 8-byte words of pinned host memory, each
// the call's ticket (upper half) with 32 bits of the value (lower half), each one system-scope store.  The host takes
// the value once every word shows the ticket; a word is complete or absent, so no fence (on this chip: a write-back of
// the whole L2) has to separate value and signal.
template <typename T> __device__ __forceinline__ void signalResult(unsigned long long *signal, unsigned ticket, T value) {
    if (signal == nullptr) return;
    constexpr int W = (sizeof(T) + 3) / 4;
    struct Words { unsigned w[W]; };
    Words in;
    if constexpr (sizeof(T) == 2) in.w[0] = __builtin_bit_cast(unsigned short, value);
    else in = __builtin_bit_cast(Words, value);
#pragma unroll
    for (int i = 0; i < W; i++)
        __hip_atomic_store(signal + i, ((unsigned long long)ticket << 32) | in.w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

static constexpr unsigned kFlatGroup = 32;          // blocks per first-level counter
static constexpr unsigned kFlatCounterStride = 32;  // counters are this many 32-bit words (128 bytes) apart
static constexpr unsigned kFlatMaxBlocks = 2048;    // 1 + kFlatMaxBlocks / kFlatGroup counters exist
// How many 32-bit words of a policy's accumulator travel through the slots: all of them, unless the policy says that
// only the first kSlotWords matter (trailing padding stays at home; the receiver fills it with zeros).
template <class Pol, typename = void> struct SlotWords { static constexpr int value = sizeof(typename Pol::Acc) / 4; };
template <class Pol> struct SlotWords<Pol, decltype((void)Pol::kSlotWords)> { static constexpr int value = Pol::kSlotWords; };

template <typename A, int W = sizeof(A) / 4>
__device__ __forceinline__ void publishSlots(unsigned long long *slot, const A &a, unsigned ticket) {
    static_assert(sizeof(A) % 4 == 0, "accumulator must be a multiple of 4 bytes");
    struct Words { unsigned w[sizeof(A) / 4]; };
    const Words in = __builtin_bit_cast(Words, a);
#pragma unroll
    for (int i = 0; i < W; i++)
        __hip_atomic_store(slot + i, ((unsigned long long)ticket << 32) | in.w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// One word of a slot group: waits (bounded) until it carries `ticket`, starting from the value `v` already loaded.  Only
// called for groups whose writer has already issued its stores, so the wait ends as soon as they land.
// `missing` is set when the wait ran out (seconds: only a launch that has gone wrong gets there).
__device__ __forceinline__ unsigned awaitSlot(const unsigned long long *slot, unsigned long long v, unsigned ticket, bool &missing) {
    for (int tries = 0; (unsigned)(v >> 32) != ticket && tries < (1 << 22); tries++) {
        __builtin_amdgcn_s_sleep(1);
        v = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if ((unsigned)(v >> 32) != ticket) missing = true;
    return (unsigned)v;
}
// What the merging block does when a slot never arrived (all its threads call this together): true tells the caller to
// store NaN instead of a number made of stale words; the stream's fault word, when there is one, lets the host report it.
__device__ __forceinline__ bool slotsWereMissing(bool missing, unsigned *fault) {
    const bool any = __syncthreads_or(missing ? 1 : 0) != 0;
    if (any && threadIdx.x == 0 && fault != nullptr) __hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    return any;
}
template <typename T> __device__ __forceinline__ T notANumber() { return fromCompute<T>((typename Compute<T>::type)__builtin_nanf("")); }
// Merges the slot groups first, first + stride, ... (count of them in all) into acc, in that order.  The loads of
// several groups are issued together: they bypass the caches, and one after the other their latencies would add up to
// more than the second launch they replace.
template <class Pol>
__device__ __forceinline__ bool mergeSlots(const Pol &pol, typename Pol::Acc &acc, const unsigned long long *slots, int first,
                                           int stride, int count, unsigned ticket) {
    bool missing = false;
    typedef typename Pol::Acc Acc;
    constexpr int W = SlotWords<Pol>::value;
    constexpr int G = W <= 2 ? 8 : (W <= 4 ? 4 : 2);
    struct Words { unsigned w[sizeof(Acc) / 4]; };
    for (int i0 = first; i0 < count; i0 += stride * G) {
        unsigned long long v[G][W];
#pragma unroll
        for (int g = 0; g < G; g++) {
            const int i = i0 + g * stride;
            if (i < count) {
#pragma unroll
                for (int w = 0; w < W; w++) v[g][w] = __hip_atomic_load(slots + (size_t)i * W + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            const int i = i0 + g * stride;
            if (i < count) {
                Words out = {};
#pragma unroll
                for (int w = 0; w < W; w++) out.w[w] = awaitSlot(slots + (size_t)i * W + w, v[g][w], ticket, missing);
                acc = pol.combine(acc, __builtin_bit_cast(Acc, out));
            }
        }
    }
    return missing;
}

// One thread of every block of a one-dimensional grid (of at most kFlatMaxBlocks blocks) calls this once, after it has
// published the block's slots: true in the block that counts itself in last.  The counters are back at zero by then.
// Atomics on one address are served one after the other, some 15 ns apiece: two thousand blocks on a single counter
// cost more than the reduction itself.  So blocks count in groups of kFlatGroup, each group on a counter of its own (in
// a memory channel of its own), and only the last block of each group goes on to the top counter.
__device__ __forceinline__ bool countedInLast(unsigned *counter) {
    const unsigned group = blockIdx.x / kFlatGroup, groups = (gridDim.x + kFlatGroup - 1) / kFlatGroup;
    const unsigned members = group + 1 < groups ? kFlatGroup : gridDim.x - group * kFlatGroup;
    unsigned *mine = counter + (size_t)(1 + group) * kFlatCounterStride;
    bool last = __hip_atomic_fetch_add(mine, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == members - 1;
    if (last) {
        __hip_atomic_store(mine, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == groups - 1;
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return last;
}

// Strided TADs whose neighbours are neighbours in memory (columns of a c-order matrix, rows of an f-order
// one): every lane owns Pack<T>::N adjacent TADs and reads them with one 16-byte load per row, so a wave
// covers a contiguous kilobyte per row.  The waves of a block (four, or eight) take the rows of the block's row
// range and merge through LDS.  A block's rows are [rowsPerSplit * blockIdx.y, ...) or, with `dealt` rows to a batch, the
// batches blockIdx.y, blockIdx.y + gridDim.y, ... of the TAD; the row ranges are merged by the last block of the column
// tile to finish (when `slots` are given: one launch) or by tadColFinish.
// Lanes whose TADs are not adjacent / aligned (checked against the offsets table) walk them one by one.
// (The four waves side by side instead - 4 KiB of every row to a block, each wave walking all the rows of the range, no
// merge through LDS - was slower: 52.6 against 48.6 us for sums along dim 0 of [16384, 4096], twice as slow for the
// summary statistics.)
// MAPPED: the same for TADs over several dimensions whose innermost one is strided: row j of the TADs lies where the
// coordinate map puts it (every stride of the map a multiple of the vector width, so that the vectors stay aligned);
// a row's divisions are shared by the Pack::N TADs of a lane.
// BLK: threads of a block (256, or 512 where the host finds that to pay).
template <class Pol, bool MAPPED = false, int BLK = kBlock>
__global__ void __launch_bounds__(BLK) tadColVecKernel(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                       typename Pol::Acc *partials, const Long *offsets, Long tadLength,
                                                       Long numTads, Long tadEws, Long rowsPerSplit, DimMap tm = DimMap(),
                                                       unsigned long long *slots = nullptr, unsigned *counter = nullptr,
                                                       unsigned slotTicket = 0, unsigned *fault = nullptr, Long dealt = 0) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::T T;
    typedef typename Pol::Acc Acc;
    constexpr int VEC = Pack<T>::N;
    constexpr int WAVES = BLK / kWave;
    constexpr int W = SlotWords<Pol>::value;
    constexpr int TILE = VEC * kWave;  // TADs of a column tile
    // (accumulators of 16 bytes or more - index pairs, moments - are merged by halving the waves, all owned TADs at once:
    // three rounds of combines side by side instead of seven on the first wave for each owned TAD in turn)
    constexpr bool TREE = sizeof(Acc) >= 16 && WAVES >= 4 && (WAVES & (WAVES - 1)) == 0;
    __shared__ Acc smem[TREE ? (WAVES / 2) * kWave * VEC : (WAVES - 1) * kWave];
    __shared__ int mergeHere;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const Long t0 = ((Long)blockIdx.x * kWave + lane) * VEC;
    const bool live = t0 < numTads;
    const Long j0 = (Long)blockIdx.y * rowsPerSplit;
    Long j1 = j0 + rowsPerSplit;
    if (j1 > tadLength) j1 = tadLength;
    Acc acc[VEC];
    Pol pe[VEC];
    if (live) {
        Long off[VEC];
        bool vec = t0 + VEC <= numTads;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            off[e] = (t0 + e < numTads) ? offsets[t0 + e] : 0;
            pe[e] = pol;
            if (t0 + e < numTads) pe[e].setTad(t0 + e, z);
            acc[e] = pe[e].init(x + off[e]);
            if (e > 0 && off[e] != off[0] + e) vec = false;
        }
        if ((reinterpret_cast<uintptr_t>(x + off[0]) & 15) != 0 || (!MAPPED && (tadEws % VEC) != 0)) vec = false;
        auto rowAt = [&](Long row) -> Long { return MAPPED ? mapOffset32(tm, (unsigned)row) : row * tadEws; };
        if (vec) {
            const T *base = x + off[0];
            // Row ranges start a power-of-two number of bytes apart, so blocks that all began at the top of their range
            // would keep hitting the same few memory channels: each range is walked from a different row, wrapping round.
            const Long span = j1 - j0;
            const Long turn = span >= 8 * WAVES ? (((Long)blockIdx.y * 3) % (span / (4 * WAVES))) * (4 * WAVES) : 0;
            // (the first part is walked in ascending order from fresh accumulators; the second part's rows lie before the
            // first's, so its elements are folded by the general rule.  Issuing the next batch's loads before the current
            // batch is folded measured no better: sums 42.9 -> 43.8 us, variance 48.6 -> 48.0, mapped TADs 44.9 -> 47.3)
            auto walk = [&](Long a, Long b, auto ascending) {
                Long j = a + wave;
                for (; j + 3 * WAVES < b; j += 4 * WAVES) {
                    Pack<T> pk[4];
#pragma unroll
                    for (int u = 0; u < 4; u++) pk[u] = loadPack(reinterpret_cast<const Pack<T> *>(base + rowAt(j + u * WAVES)));
#pragma unroll
                    for (int u = 0; u < 4; u++) {
#pragma unroll
                        for (int e = 0; e < VEC; e++) {
                            if constexpr (decltype(ascending)::value) foldNext(pe[e], acc[e], toCompute(pk[u].v[e]), j + u * WAVES);
                            else pe[e].accumulate(acc[e], toCompute(pk[u].v[e]), j + u * WAVES);
                        }
                    }
#pragma unroll
                    for (int e = 0; e < VEC; e++) pe[e].checkpoint(acc[e]);
                }
                for (; j < b; j += WAVES) {
                    Pack<T> pk = loadPack(reinterpret_cast<const Pack<T> *>(base + rowAt(j)));
#pragma unroll
                    for (int e = 0; e < VEC; e++) {
                        if constexpr (decltype(ascending)::value) foldNext(pe[e], acc[e], toCompute(pk.v[e]), j);
                        else pe[e].accumulate(acc[e], toCompute(pk.v[e]), j);
                        pe[e].checkpoint(acc[e]);
                    }
                }
            };
            if (dealt > 0) {
                for (Long q = blockIdx.y; q * dealt < tadLength; q += gridDim.y) {
                    const Long a = q * dealt, b = a + dealt < tadLength ? a + dealt : tadLength;
                    if constexpr (HasAscending<Pol>::value) walk(a, b, std::true_type());
                    else walk(a, b, std::false_type());
                }
            } else if constexpr (HasAscending<Pol>::value) {
                walk(j0 + turn, j1, std::true_type());
                walk(j0, j0 + turn, std::false_type());
            } else {
                for (int part = 0; part < 2; part++) walk(part == 0 ? j0 + turn : j0, part == 0 ? j1 : j0 + turn, std::false_type());
            }
        } else {
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                if (t0 + e >= numTads) continue;
                const T *base = x + off[e];
                if (dealt > 0) {
                    for (Long q = blockIdx.y; q * dealt < tadLength; q += gridDim.y) {
                        const Long a = q * dealt, b = a + dealt < tadLength ? a + dealt : tadLength;
                        for (Long j = a + wave; j < b; j += WAVES) { foldNext(pe[e], acc[e], toCompute(base[rowAt(j)]), j); pe[e].checkpoint(acc[e]); }
                    }
                    continue;
                }
                for (Long j = j0 + wave; j < j1; j += WAVES) { foldNext(pe[e], acc[e], toCompute(base[rowAt(j)]), j); pe[e].checkpoint(acc[e]); }
            }
        }
    }
    if constexpr (TREE) {
        for (int half = WAVES / 2; half >= 1; half >>= 1) {
            __syncthreads();
            if (wave >= half && wave < 2 * half) {
#pragma unroll
                for (int e = 0; e < VEC; e++) smem[((wave - half) * VEC + e) * kWave + lane] = acc[e];
            }
            __syncthreads();
            if (wave < half && live) {
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    if (t0 + e < numTads) acc[e] = pe[e].combine(acc[e], smem[(wave * VEC + e) * kWave + lane]);
            }
        }
    }
    // merge the waves, one owned TAD at a time (keeps the LDS footprint at one accumulator per lane of the other waves)
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        if constexpr (!TREE) {
            __syncthreads();
            if (wave > 0) smem[(wave - 1) * kWave + lane] = acc[e];
            __syncthreads();
        }
        if (wave == 0 && live && t0 + e < numTads) {
            Acc a = acc[e];
            if constexpr (!TREE) {
#pragma unroll
                for (int w = 0; w < WAVES - 1; w++) a = pe[e].combine(a, smem[w * kWave + lane]);
            }
            if (gridDim.y == 1) z[t0 + e] = pe[e].finalize(a, tadLength);
            else if (slots != nullptr)
                publishSlots<Acc, W>(slots + (((size_t)blockIdx.x * gridDim.y + blockIdx.y) * TILE + e * kWave + lane) * W, a, slotTicket);
            else partials[(Long)blockIdx.y * numTads + t0 + e] = a;
        }
    }
    if (gridDim.y == 1 || slots == nullptr) return;
    if constexpr (W <= 2) {  // (the host asks for this form only with accumulators of one or two words)
    // One launch: the row ranges of a column tile count themselves in on the tile's counter once their slots are on the
    // way, and the block that comes last merges the tile - a thread per TAD, the ranges in order, 16 slot groups in
    // flight - and writes its results.  (Tiles finish at different times: only the last one's merge is not hidden.)
    if (threadIdx.x == 0) {
        unsigned *mine = counter + (size_t)blockIdx.x * kFlatCounterStride;
        const bool last = __hip_atomic_fetch_add(mine, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.y - 1;
        if (last) __hip_atomic_store(mine, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        mergeHere = last ? 1 : 0;
    }
    __syncthreads();
    if (!mergeHere) return;
    struct Words { unsigned w[sizeof(Acc) / 4]; };
    constexpr int G = W <= 1 ? 16 : (W <= 2 ? 8 : 4);
    // PARTS threads share a TAD when the block has more threads than the tile has TADs: each takes every PARTS-th batch of
    // G row ranges, the first of them merges what the others hand over through LDS
    constexpr int PARTS = BLK > TILE ? BLK / TILE : 1;
    static_assert(PARTS == 1 || (!TREE && (PARTS - 1) * TILE <= (WAVES - 1) * kWave), "the hand-over reuses the waves' merge area");
    const int splits = (int)gridDim.y;
    __syncthreads();  // (the waves' merge area is free from here on)
    for (int k0 = 0; k0 < TILE * PARTS; k0 += BLK) {
        const int k = (k0 + (int)threadIdx.x) % TILE, part = (k0 + (int)threadIdx.x) / TILE;
        const Long t = ((Long)blockIdx.x * kWave + k % kWave) * VEC + k / kWave;
        const bool mineLive = t < numTads && part < PARTS;
        const unsigned long long *mine = slots + ((size_t)blockIdx.x * splits * TILE + k) * W;
        Pol pm = pol;
        if (mineLive) pm.setTad(t, z);
        Acc a;
        bool have = false, missing = false;
        if (mineLive) {
            for (int b0 = part * G; b0 < splits; b0 += PARTS * G) {
                unsigned long long v[G][W];
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const int b = b0 + g < splits ? b0 + g : splits - 1;
#pragma unroll
                    for (int w = 0; w < W; w++) v[g][w] = __hip_atomic_load(mine + (size_t)b * TILE * W + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int g = 0; g < G; g++) {
                    if (b0 + g < splits) {
                        Words out = {};
#pragma unroll
                        for (int w = 0; w < W; w++) out.w[w] = awaitSlot(mine + (size_t)(b0 + g) * TILE * W + w, v[g][w], slotTicket, missing);
                        const Acc piece = __builtin_bit_cast(Acc, out);
                        a = have ? pm.combine(a, piece) : piece;
                        have = true;
                    }
                }
            }
        }
        if constexpr (PARTS > 1) {
            __shared__ int handed[(PARTS - 1) * TILE];  // 0: nothing, 1: an accumulator, 2: a slot was missing
            if (mineLive && part > 0) {
                if (have) smem[(part - 1) * TILE + k] = a;
                handed[(part - 1) * TILE + k] = missing ? 2 : (have ? 1 : 0);
            }
            __syncthreads();
            if (mineLive && part == 0) {
#pragma unroll
                for (int q = 1; q < PARTS; q++) {
                    const int h = handed[(q - 1) * TILE + k];
                    if (h == 2) missing = true;
                    else if (h == 1) { a = have ? pm.combine(a, smem[(q - 1) * TILE + k]) : smem[(q - 1) * TILE + k]; have = true; }
                }
            }
        }
        if (mineLive && part == 0) {
            if (missing && fault != nullptr) __hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            z[t] = missing ? notANumber<T>() : pm.finalize(a, tadLength);
        }
    }
    }
}

// Strided TADs of which only a few are neighbours in memory: the last dimension that is kept is the contiguous one and
// short (`inner` elements, fewer than a wave's 64 vectors), as when the rows of the 56 x 56 planes of an image batch are
// summed.  A wave of the kernel above would straddle several such groups with every load.  Here a block takes one group -
// TADs a * inner .. a * inner + inner - 1 - and walks it plane by plane: thread = (row lane, vector of the row), so that what
// the block has in flight is one contiguous stretch wherever the rows of a plane follow one another.  Row j of a TAD (j
// counts the TAD's elements in C order) lies at outer(j / planeRows) + (j % planeRows) * rowStride, the map's innermost
// dimension being the plane's rows.  Row ranges (blockIdx.y) leave their accumulators in partials[range * numTads + tad]
// for tadColFinish.  Nothing is assumed about the offsets table beyond what the vector loads need, which is checked here:
// a thread whose TADs are not neighbours, or not aligned, reads them element by element.
__device__ __forceinline__ Long outerRowsOffset(const DimMap &m, unsigned idx) {
    if (m.rank < 2) return 0;
    Long off = 0;
    for (int d = m.rank - 2; d > 0; d--) {
        const unsigned q = idx / m.shape[d];
        off += (Long)(idx - q * m.shape[d]) * m.stride[d];
        idx = q;
    }
    return off + (Long)idx * m.stride[0];
}
template <class Pol>
__global__ void __launch_bounds__(kBlock) tadPlaneKernel(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                        typename Pol::Acc *partials, const Long *offsets, Long tadLength,
                                                        Long numTads, unsigned inner, unsigned groups, DimMap tm,
                                                        FastDiv planeRows, Long rowStride, Long rowsPerSplit) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::T T;
    typedef typename Pol::Acc Acc;
    constexpr int VEC = Pack<T>::N;
    static_assert(sizeof(Acc) * kBlock * VEC <= 32768, "the merge area holds every thread's accumulators");
    __shared__ Acc smem[kBlock * VEC];
    const unsigned vpr = inner / VEC;           // vectors of a row
    const unsigned lanes = kBlock / vpr;        // rows in flight per round
    const unsigned cv = threadIdx.x % vpr, rl = threadIdx.x / vpr;
    const bool active = rl < lanes;
    const Long j0 = (Long)blockIdx.y * rowsPerSplit;
    Long j1 = j0 + rowsPerSplit;
    if (j1 > tadLength) j1 = tadLength;
    auto rowAt = [&](Long j) -> Long {
        unsigned ji;
        const unsigned jo = planeRows.divmod((unsigned)j, ji);
        return outerRowsOffset(tm, jo) + (Long)ji * rowStride;
    };
    for (unsigned a = blockIdx.x; a < groups; a += gridDim.x) {
        const Long t0 = (Long)a * inner + (Long)cv * VEC;
        Acc acc[VEC];
        Pol pe[VEC];
        if (active) {
            Long off[VEC];
            bool vec = true;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                off[e] = offsets[t0 + e];
                pe[e] = pol;
                pe[e].setTad(t0 + e, z);
                acc[e] = pe[e].init(x + off[e]);
                if (e > 0 && off[e] != off[0] + e) vec = false;
            }
            if ((reinterpret_cast<uintptr_t>(x + off[0]) & 15) != 0) vec = false;
            if (vec) {
                const T *base = x + off[0];
                Long j = j0 + rl;
                for (; j < j1; j += 4 * (Long)lanes) {
                    Pack<T> pk[4];
                    // (unconditional loads on clamped rows, the guard at the use: a load in a branch of its own would wait for
                    // the loads before it)
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const Long ju = j + u * (Long)lanes;
                        pk[u] = loadPack(reinterpret_cast<const Pack<T> *>(base + rowAt(ju < j1 ? ju : j1 - 1)));
                    }
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const Long ju = j + u * (Long)lanes;
                        if (ju < j1) {
#pragma unroll
                            for (int e = 0; e < VEC; e++) foldNext(pe[e], acc[e], toCompute(pk[u].v[e]), ju);
                        }
                    }
#pragma unroll
                    for (int e = 0; e < VEC; e++) pe[e].checkpoint(acc[e]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    const T *base = x + off[e];
                    for (Long j = j0 + rl; j < j1; j += lanes) { foldNext(pe[e], acc[e], toCompute(base[rowAt(j)]), j); pe[e].checkpoint(acc[e]); }
                }
            }
        }
        // every TAD of the group is merged by a thread of its own, over the row lanes that hold a part of it
        __syncthreads();  // (the area may still be read for the group before)
        if (active) {
#pragma unroll
            for (int e = 0; e < VEC; e++) smem[threadIdx.x * VEC + e] = acc[e];
        }
        __syncthreads();
        if (threadIdx.x < inner) {
            const Long t = (Long)a * inner + threadIdx.x;
            Pol pm = pol;
            pm.setTad(t, z);
            // (lanes beyond the range's rows hold fresh accumulators, which merge like any other)
            Acc m = smem[threadIdx.x];  // row lane 0: thread cv, element e at cv * VEC + e
            for (unsigned r = 1; r < lanes; r++) m = pm.combine(m, smem[(size_t)r * inner + threadIdx.x]);
            if (gridDim.y == 1) z[t] = pm.finalize(m, tadLength);
            else partials[(Long)blockIdx.y * numTads + t] = m;
        }
    }
}

// A few very long contiguous TADs: blockIdx.x is the TAD, blockIdx.y one slice of it; the slices' accumulators go to
// partials[slice * numTads + tad] and are merged by tadColFinish.  (One block per TAD would leave most of the chip idle.)
template <class Pol>
__global__ void __launch_bounds__(kBlock) tadRowSliceKernel(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                            typename Pol::Acc *partials, const Long *offsets, Long tadLength,
                                                            Long numTads, Long sliceLength) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::Acc Acc;
    __shared__ Acc smem[kBlock / kWave];
    const Long r = blockIdx.x;
    const Long f0 = (Long)blockIdx.y * sliceLength;
    Long f1 = f0 + sliceLength;
    if (f1 > tadLength) f1 = tadLength;
    pol.setTad(r, z);
    const typename Pol::T *tx = x + offsets[r];
    Acc acc = pol.init(tx);
    if (f0 < f1) foldContiguous<Pol>(pol, acc, tx + f0, f1 - f0, (int)threadIdx.x, kBlock, f0);
    acc = blockMerge<Pol>(pol, acc, smem);
    if (threadIdx.x == 0) partials[(Long)blockIdx.y * numTads + r] = acc;
}

// Merges the slices of tadRowSliceKernel: one block per TAD, its threads take every kBlock-th slice and merge through
// the wave butterflies and LDS (there are few TADs and up to thousands of slices).
template <class Pol>
__global__ void __launch_bounds__(kBlock) tadSliceFinish(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                         const typename Pol::Acc *__restrict__ partials, const Long *offsets,
                                                         Long tadLength, Long numTads, int slices) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::Acc Acc;
    __shared__ Acc smem[kBlock / kWave];
    const Long r = blockIdx.x;
    pol.setTad(r, z);
    Acc acc = pol.init(x + offsets[r]);  // what a lane that saw nothing holds, as in the slices themselves
    for (int sl = threadIdx.x; sl < slices; sl += kBlock) acc = pol.combine(acc, partials[(Long)sl * numTads + r]);
    acc = blockMerge<Pol>(pol, acc, smem);
    if (threadIdx.x == 0) z[r] = pol.finalize(acc, tadLength);
}

// Merges the `splits` partial accumulators of each TAD: 16 TADs per block (a 64-byte stretch of each split's row of
// partials), the block's 16 groups of lanes take every 16th split, all of a thread's loads in flight together, then one
// pass through LDS.  (64 TADs per block left the 4096 results of a [16384, 4096] reduction to 64 blocks, each thread
// walking 32 splits one after the other: 5 to 6 us for 2 MB that the caches hold; this takes half of that.)
static constexpr int kFinishLanes = 16;
template <class Pol>
__global__ void __launch_bounds__(kBlock) tadColFinish(Pol pol, typename Pol::T *z,
                                                       const typename Pol::Acc *__restrict__ partials, Long tadLength,
                                                       Long numTads, int splits) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::Acc Acc;
    constexpr int LANES = kFinishLanes, GROUPS = kBlock / LANES;
    __shared__ Acc smem[kBlock];
    const int lane = threadIdx.x % LANES, grp = threadIdx.x / LANES;
    const Long t = (Long)blockIdx.x * LANES + lane;
    const bool live = t < numTads && grp < splits;
    Acc acc;
    if (live) {
        acc = partials[(Long)grp * numTads + t];
#pragma unroll 8
        for (int s = grp + GROUPS; s < splits; s += GROUPS) acc = pol.combine(acc, partials[(Long)s * numTads + t]);
        smem[threadIdx.x] = acc;
    }
    __syncthreads();
    if (live && grp == 0) {
        pol.setTad(t, z);
        for (int g = 1; g < GROUPS && g < splits; g++) acc = pol.combine(acc, smem[g * LANES + lane]);
        z[t] = pol.finalize(acc, tadLength);
    }
}

// TADs over several dimensions (their shapeInfo carries no element-wise stride) whose innermost dimension, after the
// map has been canonicalised, is contiguous: a TAD is a set of runs of runLength elements, placed by the outer dimensions
// of the map.  TEAM lanes share a TAD - or a slice of one (blockIdx.y) when the TADs are few and long - and take its
// 16-byte vectors in turn, four in flight per lane; a vector's place costs one division by the number of vectors in a
// run plus one per outer dimension beyond the first: divisions per vector, none per element.  The last vector of a run
// is short when runLength is not a multiple of the vector width; vectors need no alignment beyond the element's own.
template <class Pol, int TEAM>
__global__ void __launch_bounds__(kBlock) tadRunsKernel(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                        typename Pol::Acc *partials, const Long *offsets, DimMap tm,
                                                        Long tadLength, Long numTads, unsigned runLength, FastDiv perRun,
                                                        unsigned unitsPerTad, unsigned unitsPerSlice) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::T T;
    typedef typename Pol::Acc Acc;
    constexpr int VEC = Pack<T>::N;
    constexpr int TEAMS = kBlock / TEAM;
    __shared__ Acc smem[kBlock / kWave];
    const int team = threadIdx.x / TEAM, lane = threadIdx.x % TEAM;
    const unsigned u0 = blockIdx.y * unitsPerSlice;
    const unsigned u1 = unitsPerTad - u0 < unitsPerSlice ? unitsPerTad : u0 + unitsPerSlice;
    const int outer = tm.rank - 1;  // dimensions that place a run
    for (Long r0 = (Long)blockIdx.x * TEAMS; r0 < numTads; r0 += (Long)gridDim.x * TEAMS) {
        const Long r = r0 + team;
        const bool live = r < numTads;
        Acc acc;
        if (live) {
            pol.setTad(r, z);
            const T *tx = x + offsets[r];
            acc = pol.init(tx);
            if (runLength >= (unsigned)VEC) {
                // Every unit is one 16-byte load, requested unconditionally (a load inside a branch of its own would make the
                // compiler wait for the loads before it): a unit beyond the slice re-reads the slice's last one and is not
                // folded, and the short last unit of a run loads the VEC elements that END with the run and skips those
                // that the unit before it has folded.
                for (unsigned u = u0 + lane; u < u1; u += 4 * TEAM) {
                    Pack<T> pk[4];
                    unsigned first[4], skip[4];
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const unsigned uu = u + k * TEAM;
                        unsigned c;
                        unsigned m = perRun.divmod(uu < u1 ? uu : u1 - 1, c);
                        const unsigned begin = c * VEC + VEC <= runLength ? c * VEC : runLength - VEC;
                        skip[k] = uu < u1 ? c * VEC - begin : (unsigned)VEC;
                        first[k] = m * runLength + begin;
                        Long off = (Long)begin;
                        for (int d = outer - 1; d > 0; d--) {
                            const unsigned q = m / tm.shape[d];
                            off += (Long)(m - q * tm.shape[d]) * tm.stride[d];
                            m = q;
                        }
                        off += (Long)m * tm.stride[0];
                        pk[k] = streamPackAnywhere(tx + off);
                    }
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        if (skip[k] == 0) {
#pragma unroll
                            for (int e = 0; e < VEC; e++) foldNext(pol, acc, toCompute(pk[k].v[e]), (Long)first[k] + e);
                            pol.checkpoint(acc);
                        } else if (skip[k] < (unsigned)VEC) {
#pragma unroll
                            for (int e = 0; e < VEC; e++)
                                if ((unsigned)e >= skip[k]) foldNext(pol, acc, toCompute(pk[k].v[e]), (Long)first[k] + e);
                            pol.checkpoint(acc);
                        }
                    }
                }
            } else {
                // runs shorter than a vector: element by element
                for (unsigned u = u0 + lane; u < u1; u += TEAM) {
                    unsigned c;
                    unsigned m = perRun.divmod(u, c);  // (one unit per run: c == 0)
                    const unsigned first = m * runLength;
                    Long off = 0;
                    for (int d = outer - 1; d > 0; d--) {
                        const unsigned q = m / tm.shape[d];
                        off += (Long)(m - q * tm.shape[d]) * tm.stride[d];
                        m = q;
                    }
                    off += (Long)m * tm.stride[0];
                    for (unsigned e = 0; e < runLength; e++) foldNext(pol, acc, toCompute(tx[off + e]), (Long)first + e);
                    pol.checkpoint(acc);
                }
            }
        }
        if (TEAM == kBlock) {
            acc = blockMerge<Pol>(pol, acc, smem);  // one TAD per block: every thread runs the same trips
        } else {
            if (live) acc = waveMerge<Pol, TEAM>(pol, acc);
        }
        if (live && lane == 0) {
            if (gridDim.y == 1) z[r] = pol.finalize(acc, tadLength);
            else partials[(Long)blockIdx.y * numTads + r] = acc;
        }
    }
}

template <class Pol>
__global__ void __launch_bounds__(kBlock) tadGeneralKernel(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                           const Long *offsets, DimMap tm, Long tadLength, Long numTads) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::Acc Acc;
    __shared__ Acc smem[kBlock / kWave];
    for (Long r = blockIdx.x; r < numTads; r += gridDim.x) {
        pol.setTad(r, z);
        const typename Pol::T *tx = x + offsets[r];
        Acc acc = pol.init(tx);
        for (Long f = threadIdx.x; f < tadLength; f += kBlock)
            { foldNext(pol, acc, toCompute(tx[mapOffset32(tm, (unsigned)f)]), f); pol.checkpoint(acc); }
        acc = blockMerge<Pol>(pol, acc, smem);
        if (threadIdx.x == 0) z[r] = pol.finalize(acc, tadLength);
    }
}

// The full-array reduction: block b folds the chunks b, b+grid, ... of kBlock*kUnroll vectors.
// A one-block launch (small arrays) finishes by itself.  With several blocks and `slots` given, every block publishes
// its accumulator in its slot group and takes a number from `counter`; the block that draws the last number has seen
// every other block issue its stores, waits for them to land, merges all groups in block order and writes the result
// (the counters are back at zero by then): one launch.  Without `slots` the accumulators go to `partials` and flatFinish
// merges them in a second launch.
template <class Pol>
__global__ void __launch_bounds__(kBlock) flatKernel(Pol pol, const typename Pol::T *x, typename Pol::Acc *partials,
                                                     Long n, int strided, Long ews, DimMap xm, typename Pol::T *z,
                                                     unsigned long long *signal, unsigned ticket, unsigned long long *slots,
                                                     unsigned *counter, unsigned slotTicket, unsigned *fault = nullptr) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::T T;
    typedef typename Pol::Acc Acc;
    __shared__ Acc smem[kBlock / kWave];
    __shared__ int mergeHere;
    pol.setTad(0, nullptr);
    Acc acc = pol.init(x);
    if (strided && ews == 1) {
        constexpr int VEC = Pack<T>::N;
        const uintptr_t addr = reinterpret_cast<uintptr_t>(x);
        Long head = ((addr & (sizeof(T) - 1)) == 0) ? (Long)(((16 - (addr & 15)) & 15) / sizeof(T)) : n;
        if (head > n) head = n;
        const Long nvec = (n - head) / VEC;
        const Pack<T> *xv = reinterpret_cast<const Pack<T> *>(x + head);
        const Long chunk = (Long)kBlock * kUnroll;
        // A policy whose accumulators may be regrouped freely (kChains > 1: its combine() is its update) gets one
        // accumulator per vector in flight: one accumulator makes every element wait for the one before it (a compare and a
        // select for a maximum, three selects for an index), and with the few waves per SIMD of this launch nothing else
        // fills the gaps - the maximum over 2^26 floats took 85 us with 512 blocks where the sum took 48.
        constexpr int CH = PolChains<Pol>::value > 1 ? 4 : 1;
        Acc more[CH > 1 ? CH - 1 : 1];
        if (CH > 1) {
#pragma unroll
            for (int c = 0; c < CH - 1; c++) more[c] = pol.init(x);
        }
        // (every block takes every gridDim.x-th chunk; one contiguous range per block measured 1 to 2 % slower)
        const Long bFirst = (Long)blockIdx.x * chunk, bEnd = nvec, bStep = (Long)gridDim.x * chunk;
        for (Long b = bFirst; b < bEnd; b += bStep) {
            Pack<T> pk[kUnroll];
            // (unconditional loads, see foldContiguous: out-of-range lanes re-read the last vector and do not fold it)
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                Long v = b + u * kBlock + threadIdx.x;
                pk[u] = loadPack(xv + (v < nvec ? v : nvec - 1));
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                Long v = b + u * kBlock + threadIdx.x;
                if (v < nvec) {
                    Acc &to = (CH > 1 && u % CH > 0) ? more[u % CH - 1] : acc;
#pragma unroll
                    for (int e = 0; e < VEC; e++) foldNext(pol, to, toCompute(pk[u].v[e]), head + v * VEC + e);
                    pol.checkpoint(to);
                }
            }
        }
        if (CH > 1) {
#pragma unroll
            for (int c = 0; c < CH - 1; c++) acc = pol.combine(acc, more[c]);
        }
        if (blockIdx.x == 0) {
            for (Long i = threadIdx.x; i < head; i += kBlock) {
                pol.accumulate(acc, toCompute(x[i]), i);
                pol.checkpoint(acc);
            }
            for (Long i = head + nvec * VEC + threadIdx.x; i < n; i += kBlock) {
                pol.accumulate(acc, toCompute(x[i]), i);
                pol.checkpoint(acc);
            }
        }
    } else if (strided) {
        for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += (Long)gridDim.x * kBlock)
            { foldNext(pol, acc, toCompute(x[i * ews]), i); pol.checkpoint(acc); }
    } else {
        for (Long i = (Long)blockIdx.x * kBlock + threadIdx.x; i < n; i += (Long)gridDim.x * kBlock)
            { foldNext(pol, acc, toCompute(x[mapOffsetAny(xm, i)]), i); pol.checkpoint(acc); }
    }
    acc = blockMerge<Pol>(pol, acc, smem);
    if (gridDim.x == 1) {
        if (threadIdx.x == 0) {
            const T r = pol.finalize(acc, n);
            z[0] = r;
            signalResult(signal, ticket, r);
        }
        return;
    }
    if (slots == nullptr) {
        if (threadIdx.x == 0) partials[blockIdx.x] = acc;
        return;
    }
    constexpr int W = SlotWords<Pol>::value;
    if (threadIdx.x == 0) {
        publishSlots<Acc, W>(slots + (size_t)blockIdx.x * W, acc, slotTicket);
        mergeHere = countedInLast(counter);
    }
    __syncthreads();
    if (!mergeHere) return;
    acc = pol.init(x);
    const bool missing = slotsWereMissing(mergeSlots<Pol>(pol, acc, slots, threadIdx.x, kBlock, (int)gridDim.x, slotTicket), fault);
    acc = blockMerge<Pol>(pol, acc, smem);
    if (threadIdx.x == 0) {
        const typename Pol::T r = missing ? notANumber<T>() : pol.finalize(acc, n);
        z[0] = r;
        signalResult(signal, ticket, r);
    }
}

// Second launch of the two-launch form: one block merges the per-block partials.
template <class Pol>
__global__ void __launch_bounds__(kBlock) flatFinish(Pol pol, const typename Pol::T *x, typename Pol::T *z,
                                                     const typename Pol::Acc *partials, int count, Long n,
                                                     unsigned long long *signal, unsigned ticket) {
    if (Pol::tables) lm::loadTables();
    typedef typename Pol::Acc Acc;
    __shared__ Acc smem[kBlock / kWave];
    pol.setTad(0, nullptr);
    Acc acc = pol.init(x);
    for (int i = threadIdx.x; i < count; i += kBlock) acc = pol.combine(acc, partials[i]);
    acc = blockMerge<Pol>(pol, acc, smem);
    if (threadIdx.x == 0) {
        const typename Pol::T r = pol.finalize(acc, n);
        z[0] = r;
        signalResult(signal, ticket, r);
    }
}

// ---- host launch logic shared by the three families ---------------------------------------------------
template <class Pol>
inline void runTadReduce(hipStream_t s, Pol pol, const typename Pol::T *x, typename Pol::T *z, const TadPlan &pl,
                         Workspace ws) {
    typedef typename Pol::Acc Acc;
    if (pl.numTads <= 0) return;
    if (pl.kind == TadPlan::ROW && pl.tadLength >= 16384 && pl.numTads <= 1024) {
        // few long TADs: slices of at least 4096 elements, about 2048 blocks in all
        Long slices = 2048 / pl.numTads;
        const Long maxSlices = pl.tadLength / 4096;
        if (slices > maxSlices) slices = maxSlices;
        if (slices > 65535) slices = 65535;
        while (slices > 1 && (size_t)slices * (size_t)pl.numTads * sizeof(Acc) > ws.bytes) slices /= 2;
        if (slices >= 2) {
            Long sliceLength = (pl.tadLength + slices - 1) / slices;
            sliceLength = (sliceLength + 63) / 64 * 64;  // slices start on 16-byte boundaries whenever the TAD does
            slices = (pl.tadLength + sliceLength - 1) / sliceLength;
            Acc *partials = reinterpret_cast<Acc *>(ws.ptr);
            ND4J_LAUNCH((tadRowSliceKernel<Pol>), dim3((unsigned)pl.numTads, (unsigned)slices), dim3(kBlock), 0, s, pol, x, z,
                               partials, pl.offsets, pl.tadLength, pl.numTads, sliceLength);
            ND4J_LAUNCH((tadSliceFinish<Pol>), dim3((unsigned)pl.numTads), dim3(kBlock), 0, s, pol, x, z, partials,
                               pl.offsets, pl.tadLength, pl.numTads, (int)slices);
            return;
        }
    }
    if (pl.kind == TadPlan::ROW && pl.tadLength >= 32) {
        // (a whole block per TAD from 4096 elements on - a batch of four vectors per lane: sums and maxima along the rows
        // of [16384, 4096] 42.6 -> 41.2 us against a wave per row; from 2048 on the rows of [32768, 2048] lose: 86 -> 108)
        if (pl.tadLength >= 4096) {
            int grid = gridFor(pl.numTads, 1, kGridCap);
            ND4J_LAUNCH((tadRowKernel<Pol, kBlock>), dim3(grid), dim3(kBlock), 0, s, pol, x, z, pl.offsets,
                               pl.tadLength, pl.numTads);
        } else if (pl.tadLength >= 256) {
            int grid = gridFor(pl.numTads, kBlock / 64, kGridCap);
            ND4J_LAUNCH((tadRowKernel<Pol, 64>), dim3(grid), dim3(kBlock), 0, s, pol, x, z, pl.offsets,
                               pl.tadLength, pl.numTads);
        } else {
            int grid = gridFor(pl.numTads, kBlock / 16, kGridCap);
            ND4J_LAUNCH((tadRowKernel<Pol, 16>), dim3(grid), dim3(kBlock), 0, s, pol, x, z, pl.offsets,
                               pl.tadLength, pl.numTads);
        }
        return;
    }
    // (the vector loads need every row of the TADs' common pitch to start on a 16-byte boundary: a pitch that is not a
    // multiple of the vector width goes to the lane-per-TAD kernel below, whose neighbouring lanes read neighbouring
    // elements)
    {
        // Strided TADs in groups of fewer neighbours than a wave has vectors, and at least ten rounds of rows for the block:
        // the plane kernel.  In us against the kernels below - sums over dimensions {0,2} of [128,128,56,56]: 36.1 / 43.4, index
        // of the maximum 40.3 / 52.8; sums over dimension 1 of [4096,128,100]: 33.8 / 41.1, of [6000,40,252]: 42.0 / 49.7, of
        // [8,100000,32]: 22.9 / 28.8, of [4096,128,128]: 42.3 / 42.9.  Shorter ranges lose (three rounds, dimension 2 of the
        // first array: 43.0 against 42.5 for sums, 79 against 47 for the index; two rounds, [4096,128,16]: 21 against 9), and
        // so do the statistics' moments (66 against 53-60), whose merge is the expensive part: both stay below.
        constexpr int VEC = Pack<typename Pol::T>::N;
        const bool stridedTads = pl.kind == TadPlan::COL || (pl.kind == TadPlan::GENERAL && pl.runLength == 0 && pl.tm.rank >= 1);
        if constexpr (sizeof(Acc) <= 16)
        if (stridedTads && pl.keptInner >= 4u * VEC && pl.keptInner % VEC == 0 && pl.keptInner / VEC < (unsigned)kWave &&
            pl.otherStrides % VEC == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && pl.numTads % pl.keptInner == 0 &&
            pl.tadLength <= 0x7fffffffLL) {
            const unsigned lanes = kBlock / (pl.keptInner / VEC);
            DimMap tm = pl.tm;
            if (pl.kind == TadPlan::COL) { tm.rank = 1; tm.shape[0] = (unsigned)pl.tadLength; tm.stride[0] = pl.tadEws; }
            const unsigned planeRows = tm.shape[tm.rank - 1];
            const Long rowStride = tm.stride[tm.rank - 1];
            if (pl.tadLength >= 10 * (Long)lanes && rowStride % VEC == 0) {
                const Long groups = pl.numTads / pl.keptInner;
                // 512 blocks or more (1024 for index pairs), a range no shorter than ten rounds of the block's row lanes, whole planes
                // where it has several
                // (sums over {0,2} of [128,128,56,56] with 256 / 512 / 1024 / 2048 / 4096 blocks: 50.0 / 34.1 / 34.8 / 36.5 / 34.9 us; the
                // index of the maximum: 61.5 / 41.0 / 38.6 / 39.9)
                const Long tgt = sizeof(Acc) <= 8 ? 512 : 1024;
                Long splits = groups >= tgt ? 1 : (tgt + groups - 1) / groups;
                const Long maxByRows = pl.tadLength / (10 * (Long)lanes) > 1 ? pl.tadLength / (10 * (Long)lanes) : 1;
                if (splits > maxByRows) splits = maxByRows;
                if (splits > 65535) splits = 65535;
                while (splits > 1 && (size_t)splits * (size_t)pl.numTads * sizeof(Acc) > ws.bytes) splits /= 2;
                Long rowsPerSplit = (pl.tadLength + splits - 1) / splits;
                if (rowsPerSplit > (Long)planeRows) rowsPerSplit = (rowsPerSplit + planeRows - 1) / planeRows * planeRows;
                splits = (pl.tadLength + rowsPerSplit - 1) / rowsPerSplit;
                Acc *partials = reinterpret_cast<Acc *>(ws.ptr);
                const unsigned gx = (unsigned)(groups < (1 << 20) ? groups : (1 << 20));
                ND4J_LAUNCH((tadPlaneKernel<Pol>), dim3(gx, (unsigned)splits), dim3(kBlock), 0, s, pol, x, z, partials, pl.offsets,
                            pl.tadLength, pl.numTads, pl.keptInner, (unsigned)groups, tm, FastDiv(planeRows), rowStride, rowsPerSplit);
                if (splits > 1)
                    ND4J_LAUNCH((tadColFinish<Pol>), dim3((unsigned)((pl.numTads + kFinishLanes - 1) / kFinishLanes)), dim3(kBlock), 0, s,
                                pol, z, partials, pl.tadLength, pl.numTads, (int)splits);
                return;
            }
        }
    }
    bool mappedVec = pl.kind == TadPlan::GENERAL && pl.runLength == 0 && pl.numTads >= 2 * kWave * Pack<typename Pol::T>::N &&
                     (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    for (int d = 0; mappedVec && d < pl.tm.rank; d++) mappedVec = pl.tm.stride[d] % Pack<typename Pol::T>::N == 0;
    if (mappedVec || (pl.kind == TadPlan::COL && pl.numTads >= 2 * kWave * Pack<typename Pol::T>::N &&
        pl.tadEws % Pack<typename Pol::T>::N == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0)) {
        // lane per Pack::N adjacent TADs, 64 lanes per block column, rows split over the block's waves and blockIdx.y
        constexpr int VEC = Pack<typename Pol::T>::N;
        int gx = (int)((pl.numTads + (Long)kWave * VEC - 1) / ((Long)kWave * VEC));
        // Plain strided TADs: 256 blocks of 512 threads, whatever the policy (one block per compute unit: eight waves with four
        // 16-byte loads in flight each keep the memory busy, and every block less is a row of partial results less to merge).
        // Measured on [16384, 4096] along dimension 0 (16 column tiles) and on an f-order [32768, 2048] along dimension 1
        // (128 tiles), in us: sums 42.9 / 41.8, index of the maximum 46.0, variance - / 48.6; with 256 threads and 512
        // (sums), 2048 (index) or 1024 (statistics) blocks 45.6 / 44.0, 49.3 and 49.1; 512 or 1024 blocks of 512 threads
        // are slower for all of them.  Mapped TADs keep 256 threads and the policy's kColBlocks (1024 at least).
        const bool wide = !mappedVec;
        const int waves = wide ? 8 : kBlock / kWave;
        // (mapped TADs: at least 1024 blocks - sums over dimensions {0,2} of [128,128,56,56] 45.2 us with 512, 43.2 with 1024,
        // 46.9 with 2048, 66 with 256)
        constexpr int kMappedBlocks = PolColBlocks<Pol>::value < 1024 ? 1024 : PolColBlocks<Pol>::value;
        Long splits = (wide ? 256 : kMappedBlocks) / gx;
        if (splits < 1) splits = 1;
        Long maxSplitsByRows = (pl.tadLength + 16 * waves - 1) / (16 * waves);  // at least 16 rows per wave
        if (splits > maxSplitsByRows) splits = maxSplitsByRows;
        if (splits > 65535) splits = 65535;
        size_t need = (size_t)splits * (size_t)pl.numTads * sizeof(Acc);
        while (splits > 1 && need > ws.bytes) { splits /= 2; need = (size_t)splits * (size_t)pl.numTads * sizeof(Acc); }
        if (splits < 1) splits = 1;
        Long rowsPerSplit = (pl.tadLength + splits - 1) / splits;
        splits = (pl.tadLength + rowsPerSplit - 1) / rowsPerSplit;
        if (splits < 1) splits = 1;
        Acc *partials = reinterpret_cast<Acc *>(ws.ptr);
        // One launch when the accumulators are one or two slot words, the tiles' counters exist (128 of them) and the slots
        // hold a group per (tile, row range, TAD); otherwise the row ranges are merged by a second launch.  (What the second
        // launch costs is small: sums along dimension 0 of [16384, 4096] take 45.6 us either way, maxima along dimension 1
        // of an f-order [32768, 2048] 41.9 in one launch and 42.5 in two.  Accumulators of more words - index pairs, the
        // statistics' moments - would have a tile's last block collect hundreds of words per thread: they keep the second
        // launch, which spreads that over the chip - measured: index of the maximum 45.8 us in two launches, 46.7 in one;
        // variance, with its moments cut down to the seven words of an open run, 47.3 against 49.8.)
        constexpr int W = SlotWords<Pol>::value;
        const bool oneLaunch = splits > 1 && W <= 2 && ws.slots != nullptr && ws.counter != nullptr && ws.slotTicketSource != nullptr &&
                               gx <= 128 && (size_t)gx * (size_t)splits * kWave * VEC * W * sizeof(unsigned long long) <= ws.slotBytes;
        // With eight row ranges or more a tile's rows are dealt to them a batch at a time (what all blocks have in flight is
        // then one stretch of memory): 45.6 -> 42.9 us for the sums over 16 tiles above, 51 -> 46 for the index of the
        // maximum; with two ranges (128 tiles) it changes nothing for sums and costs the statistics 3 us, so few ranges keep
        // a contiguous share each.
        Long dealt = wide && splits >= 8 ? 4 * waves : 0;
        unsigned long long *slots = oneLaunch ? ws.slots : nullptr;
        const unsigned slotTicket = oneLaunch ? ws.nextSlotTicket() : 0u;
        if (mappedVec)
            ND4J_LAUNCH((tadColVecKernel<Pol, true>), dim3(gx, (unsigned)splits), dim3(kBlock), 0, s, pol, x, z, partials,
                               pl.offsets, pl.tadLength, pl.numTads, (Long)0, rowsPerSplit, pl.tm, slots, ws.counter, slotTicket, ws.fault,
                               dealt);
        else
            ND4J_LAUNCH((tadColVecKernel<Pol, false, 512>), dim3(gx, (unsigned)splits), dim3(512), 0, s, pol, x, z, partials,
                               pl.offsets, pl.tadLength, pl.numTads, pl.tadEws, rowsPerSplit, DimMap(), slots, ws.counter, slotTicket,
                               ws.fault, dealt);
        if (splits > 1 && !oneLaunch)
            ND4J_LAUNCH((tadColFinish<Pol>), dim3((unsigned)((pl.numTads + kFinishLanes - 1) / kFinishLanes)), dim3(kBlock), 0, s, pol,
                               z, partials, pl.tadLength, pl.numTads, (int)splits);
        return;
    }
    const bool mappedLanes = pl.kind == TadPlan::GENERAL && pl.runLength == 0 && pl.numTads >= kWave;
    if (pl.kind == TadPlan::ROW || pl.kind == TadPlan::COL || mappedLanes) {
        // one lane per TAD; split the TAD length so that the grid fills the chip
        int gx = (int)((pl.numTads + kBlock - 1) / kBlock);
        Long splits = 2048 / gx;
        if (splits < 1) splits = 1;
        Long maxSplitsByRows = (pl.tadLength + 31) / 32;  // at least 32 rows per split
        if (splits > maxSplitsByRows) splits = maxSplitsByRows;
        size_t need = (size_t)splits * (size_t)pl.numTads * sizeof(Acc);
        while (splits > 1 && need > ws.bytes) { splits /= 2; need = (size_t)splits * (size_t)pl.numTads * sizeof(Acc); }
        if (splits < 1) splits = 1;
        Long rowsPerSplit = (pl.tadLength + splits - 1) / splits;
        splits = (pl.tadLength + rowsPerSplit - 1) / rowsPerSplit;
        if (splits < 1) splits = 1;
        Acc *partials = reinterpret_cast<Acc *>(ws.ptr);
        if (mappedLanes)
            ND4J_LAUNCH((tadColKernel<Pol, true>), dim3(gx, (unsigned)splits), dim3(kBlock), 0, s, pol, x, z, partials,
                               pl.offsets, pl.tadLength, pl.numTads, (Long)0, rowsPerSplit, pl.tm);
        else
        ND4J_LAUNCH((tadColKernel<Pol>), dim3(gx, (unsigned)splits), dim3(kBlock), 0, s, pol, x, z, partials,
                           pl.offsets, pl.tadLength, pl.numTads, pl.tadEws, rowsPerSplit, DimMap());
        if (splits > 1)
            ND4J_LAUNCH((tadColFinish<Pol>), dim3((unsigned)((pl.numTads + kFinishLanes - 1) / kFinishLanes)), dim3(kBlock), 0, s, pol,
                               z, partials, pl.tadLength, pl.numTads, (int)splits);
        return;
    }
    if (pl.runLength > 0 && pl.tm.rank >= 2) {
        // several dimensions, the innermost contiguous: vectors along the runs
        constexpr int VEC = Pack<typename Pol::T>::N;
        const unsigned unitsPerRun = (pl.runLength + VEC - 1) / VEC;
        const unsigned unitsPerTad = (unsigned)(pl.tadLength / pl.runLength) * unitsPerRun;
        const FastDiv perRun(unitsPerRun);
        Acc *partials = reinterpret_cast<Acc *>(ws.ptr);
        if (unitsPerTad >= 2048) {
            // a block per TAD; few TADs are cut into slices of whole rounds (four vectors per thread), four rounds or more
            // each, about 2048 blocks in all (4096 or 8192 blocks and slices of one or two rounds measured the same for sums
            // and 10 % slower for the summary statistics, whose accumulators cost more to merge)
            const int tuneRounds = 4, tuneBlocks = 2048;
            const unsigned round = 4 * kBlock;
            Long slices = pl.numTads < tuneBlocks ? (tuneBlocks + pl.numTads - 1) / pl.numTads : 1;
            const Long maxSlices = unitsPerTad / (tuneRounds * round);
            if (slices > maxSlices) slices = maxSlices;
            if (slices > 65535) slices = 65535;
            while (slices > 1 && (size_t)slices * (size_t)pl.numTads * sizeof(Acc) > ws.bytes) slices /= 2;
            if (slices < 1) slices = 1;
            unsigned perSlice = (unsigned)((unitsPerTad + slices - 1) / slices);
            if (slices > 1) perSlice = (perSlice + round - 1) / round * round;
            slices = (unitsPerTad + perSlice - 1) / perSlice;
            const int gx = (int)(pl.numTads < kGridCap ? pl.numTads : kGridCap);
            ND4J_LAUNCH((tadRunsKernel<Pol, kBlock>), dim3(gx, (unsigned)slices), dim3(kBlock), 0, s, pol, x, z, partials, pl.offsets,
                               pl.tm, pl.tadLength, pl.numTads, pl.runLength, perRun, unitsPerTad, perSlice);
            if (slices > 1)
                ND4J_LAUNCH((tadSliceFinish<Pol>), dim3((unsigned)pl.numTads), dim3(kBlock), 0, s, pol, x, z, partials, pl.offsets,
                                   pl.tadLength, pl.numTads, (int)slices);
        } else if (unitsPerTad >= 64) {
            ND4J_LAUNCH((tadRunsKernel<Pol, 64>), dim3(gridFor(pl.numTads, kBlock / 64, kGridCap)), dim3(kBlock), 0, s, pol, x, z,
                               partials, pl.offsets, pl.tm, pl.tadLength, pl.numTads, pl.runLength, perRun, unitsPerTad, unitsPerTad);
        } else {
            ND4J_LAUNCH((tadRunsKernel<Pol, 16>), dim3(gridFor(pl.numTads, kBlock / 16, kGridCap)), dim3(kBlock), 0, s, pol, x, z,
                               partials, pl.offsets, pl.tm, pl.tadLength, pl.numTads, pl.runLength, perRun, unitsPerTad, unitsPerTad);
        }
        return;
    }
    int grid = gridFor(pl.numTads, 1, kGridCap);
    ND4J_LAUNCH((tadGeneralKernel<Pol>), dim3(grid), dim3(kBlock), 0, s, pol, x, z, pl.offsets, pl.tm, pl.tadLength,
                       pl.numTads);
}

template <class Pol>
inline void runFlatReduce(hipStream_t s, Pol pol, const typename Pol::T *x, typename Pol::T *z, const FlatPlan &pl,
                          Workspace ws) {
    typedef typename Pol::Acc Acc;
    typedef typename Pol::T T;
    Long perBlock = (Long)kBlock * kUnroll * Pack<T>::N;
    // (how many blocks serve best differs by policy - kFlatBlocks: with a thread's four loads in flight together, two
    // blocks per compute unit stream 2^26 floats as fast as eight do, and every block less is a slot less for the last
    // block to collect: sums and maxima 49 us per synchronous call with 512 blocks, 50 to 52 with 1024 or 2048; index
    // reductions, whose accumulators are three slot words, 53 us with 768, 54 with 1024, 56 with 2048, 71 with 512)
    int grid = gridFor(pl.n, perBlock, PolFlatBlocks<Pol>::value);
    const bool oneLaunch = ws.slots != nullptr && ws.counter != nullptr && ws.slotTicketSource != nullptr;
    size_t maxBlocks = oneLaunch ? ws.slotBytes / (SlotWords<Pol>::value * sizeof(unsigned long long)) : ws.bytes / sizeof(Acc);
    if ((size_t)grid > maxBlocks) grid = (int)maxBlocks;
    if (grid < 1) grid = 1;
    Acc *partials = reinterpret_cast<Acc *>(ws.ptr);
    ND4J_LAUNCH((flatKernel<Pol>), dim3(grid), dim3(kBlock), 0, s, pol, x, partials, pl.n, pl.strided ? 1 : 0,
                       pl.ews, pl.xm, z, ws.signal, ws.ticket, oneLaunch ? ws.slots : nullptr, ws.counter,
                       oneLaunch && grid > 1 ? ws.nextSlotTicket() : 0u, ws.fault);
    if (grid > 1 && !oneLaunch)
        ND4J_LAUNCH((flatFinish<Pol>), dim3(1), dim3(kBlock), 0, s, pol, x, z, partials, grid, pl.n, ws.signal, ws.ticket);
}

}  // namespace nd4j_amd
