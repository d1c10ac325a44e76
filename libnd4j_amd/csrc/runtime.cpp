#include "runtime.h"

#include <chrono>
#include <cstring>

#include <map>
#include <mutex>
#include <utility>

namespace nd4j_amd {

Environment &environment() {
    static Environment env;
    return env;
}

bool launchesAreVerbose() { return environment().verbose.load(std::memory_order_relaxed) && environment().debug.load(std::memory_order_relaxed); }
void printLaunch(const char *kernel, dim3 grid, dim3 block, size_t ldsBytes) {
    std::printf("Launch: %s gridSize: [%u, %u, %u], blockSize: [%u], dynamic shmem: [%zu]\n", kernel, grid.x, grid.y, grid.z, block.x,
                ldsBytes);
    std::fflush(stdout);
}

bool isDeviceMemory(const void *p) {
    if (p == nullptr) return false;
    hipPointerAttribute_t attr;
    hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();  // plain (unregistered) host memory reports an error: clear it
        return false;
    }
    return attr.type == hipMemoryTypeDevice;
}

static void throwHip(const char *what, hipError_t e) {
    throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// Calls that had to read a shapeInfo or a dimension array back from the device (each one a stream synchronisation)
static std::atomic<long long> gHostFetches{0};
long long hostFetchCount() { return gHostFetches.load(); }

const Long *hostShapeInfo(Nd4jPointer *extra, int slot, const Long *arg, std::vector<Long> &storage, hipStream_t s) {
    if (void *h = slotOf(extra, slot)) return reinterpret_cast<const Long *>(h);
    if (arg == nullptr) return nullptr;
    if (!isDeviceMemory(arg)) return arg;
    gHostFetches++;
    Long rank = 0;
    hipError_t e = hipMemcpyAsync(&rank, arg, sizeof(Long), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) throwHip("fetching shapeInfo rank", e);
    if (rank < 0 || rank > kMaxRank) throw std::runtime_error("shapeInfo rank out of range");
    storage.resize(siLength((int)rank));
    e = hipMemcpyAsync(storage.data(), arg, storage.size() * sizeof(Long), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) throwHip("fetching shapeInfo", e);
    return storage.data();
}

bool hostInts(const int *arg, int count, std::vector<int> &out, hipStream_t s) {
    out.clear();
    if (arg == nullptr || count <= 0) return false;
    out.resize(count);
    if (!isDeviceMemory(arg)) {
        for (int i = 0; i < count; i++) out[i] = arg[i];
        return true;
    }
    gHostFetches++;
    hipError_t e = hipMemcpyAsync(out.data(), arg, count * sizeof(int), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) throwHip("fetching dimension", e);
    return true;
}

// A kernel whose merging block gave up waiting for another block's partial result stores a non-zero word in the stream's
// pinned block (and NaN as its result): reported by the next call on the stream that looks (scalar-returning calls, and
// every call in debug mode).
static void throwOnFault(unsigned *fault, const char *what) {
    if (fault == nullptr) return;
    volatile unsigned *f = fault;
    if (*f == 0) return;
    *f = 0;
    throw std::runtime_error(std::string(what) + ": a block's partial result did not reach the block that merges them "
                             "(a whole-array reduction on this stream gave up after its bounded wait); its result is NaN");
}
static unsigned *faultWordIfAny(hipStream_t s);

void checkLaunch(const char *what, hipStream_t s) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) throwHip(what, e);
    if (environment().debug.load()) {
        e = hipStreamSynchronize(s);
        if (e != hipSuccess) throwHip(what, e);
        throwOnFault(faultWordIfAny(s), what);
    }
}

bool streamIsCapturing(hipStream_t s) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capture) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return capture != hipStreamCaptureStatusNone;
}

void syncAndCheck(const char *what, hipStream_t s) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) throwHip(what, e);
    if (streamIsCapturing(s)) return;  // nothing runs yet that could be waited for; the graph's launch is what the caller waits on
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) throwHip(what, e);
}

void reportUnknownOp(const char *family, int opNum) {
    // the reference prints and carries on without touching the output (op_boilerplate.h:1148)
    printf("[ERROR] Unknown opNum=%d for %s on %s:%d\n", opNum, family, __FILE__, __LINE__);
    fflush(stdout);
}

namespace {
std::mutex gMutex;
std::map<std::pair<int, hipStream_t>, Workspace> gWorkspaces;

struct CachedTad {
    TadPack pack;
    Long *devOffsets = nullptr;
    Long tadLength = 0;
    ~CachedTad() { if (devOffsets != nullptr) (void)hipFree(devOffsets); }
};
std::map<std::vector<Long>, std::shared_ptr<CachedTad> > gTadCache;
size_t gTadCacheBytes = 0;
// Beyond this the cache is emptied (after the devices have drained: queued kernels may still read the tables).
// Callers that pass their own TAD tables, as nd4j does, never fill it.
const size_t kTadCacheLimitBytes = (size_t)1 << 30;
const size_t kTadCacheLimitEntries = 16384;

// Empties the cache into `old`, which the caller destroys after it has let go of gMutex: an entry's device table is
// released by hipFree, which waits for the device's outstanding work first (kernels queued by calls that have already
// returned may still read the table), and that wait must not hold up every other thread of the library.  A call that
// still holds an entry keeps it alive until it returns.
void takeTadCacheLocked(std::map<std::vector<Long>, std::shared_ptr<CachedTad> > &old) {
    old.swap(gTadCache);
    gTadCacheBytes = 0;
}
}  // namespace

Workspace workspaceFor(hipStream_t s, size_t minBytes) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    std::lock_guard<std::mutex> lock(gMutex);
    Workspace &w = gWorkspaces[std::make_pair(dev, s)];
    if (w.ptr != nullptr && w.bytes >= minBytes) return w;
    // (allocating - and waiting for the stream before the old block is freed - is not something a stream under capture
    // can do: say so, instead of leaving the capture broken by the calls below)
    if (streamIsCapturing(s))
        throw std::runtime_error("the stream is being captured and its workspace does not exist yet or is too small: make the "
                                 "same call once on this stream before the capture begins");
    size_t want = minBytes < (size_t)(8u << 20) ? (size_t)(8u << 20) : minBytes;
    if (w.ptr != nullptr) {
        // earlier work on this stream may still use the old block
        (void)hipStreamSynchronize(s);
        (void)hipFree(w.ptr);
        w.ptr = nullptr;
        w.bytes = 0;
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) throwHip("workspace allocation", e);
    w.ptr = p;
    w.bytes = want;
    return w;
}

namespace {
struct PinnedSlot {
    void *block = nullptr;  // 256 bytes: value at 0, tagged words at 128, fault word at kPinnedFaultOffset
    unsigned ticket = 0;
};
const size_t kPinnedFaultOffset = 192;
std::map<std::pair<int, hipStream_t>, PinnedSlot> gPinnedSlots;
PinnedSlot &pinnedSlotLocked(hipStream_t s) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    PinnedSlot &p = gPinnedSlots[std::make_pair(dev, s)];
    if (p.block == nullptr) {
        // coherent: the device's stores reach host memory while the kernel runs, not only when it has ended
        hipError_t e = hipHostMalloc(&p.block, 256, hipHostMallocCoherent);
        if (e != hipSuccess) { p.block = nullptr; throwHip("pinned scalar slot", e); }
        std::memset(p.block, 0, 256);
    }
    return p;
}
}  // namespace

namespace {
struct FlatSlots {
    void *block = nullptr;  // kFlatSlotBytes of slots, then kFlatCounterBytes of block counters, then kFlatStateBytes of row states
    unsigned ticket = 0;
};
const size_t kFlatSlotBytes = 2u << 20;      // 2048 blocks x 16 accumulator words x 8 bytes for a whole-array reduction; the
                                             // rest so that a cooperative softmax over a few thousand rows is one launch
const size_t kFlatCounterBytes = 16u << 10;  // 65 counters, 128 bytes apart
const size_t kFlatStateBytes = 256u << 10;   // 2048 row (or row group) states, 128 bytes apart
std::map<std::pair<int, hipStream_t>, FlatSlots> gFlatSlots;
}  // namespace

// Tickets tag the slot words and row states of one launch; the cooperative softmax kernels keep 30 bits of them.  Slots
// are never cleared between launches, so a word left behind 2^30 tickets ago would pass for a fresh one: shortly before
// the counter crosses a multiple of 2^30 (a call takes a handful of tickets) the slots and states are cleared on the
// stream - behind everything that still uses them - and the counter is moved past the boundary.
const unsigned kTicketPeriod = 1u << 30, kTicketMargin = 256;

void addFlatSlots(Workspace &w, hipStream_t s) {
    // A stream that is being captured into a graph gets no slots: the tickets that keep one launch's partial results apart
    // from the next one's are drawn here, on the host, and a graph would replay the one it was captured with.  Without
    // slots every caller takes its path of two launches (partial results in the workspace, merged by a second kernel),
    // which replays like any other pair of kernels.
    if (streamIsCapturing(s)) return;
    int dev = 0;
    (void)hipGetDevice(&dev);
    std::lock_guard<std::mutex> lock(gMutex);
    FlatSlots &f = gFlatSlots[std::make_pair(dev, s)];
    if (f.block == nullptr) {
        hipError_t e = hipMalloc(&f.block, kFlatSlotBytes + kFlatCounterBytes + kFlatStateBytes);
        if (e != hipSuccess) { f.block = nullptr; throwHip("reduction slots allocation", e); }
        e = hipMemset(f.block, 0, kFlatSlotBytes + kFlatCounterBytes + kFlatStateBytes);
        if (e != hipSuccess) throwHip("reduction slots clearing", e);
    }
    if ((f.ticket & (kTicketPeriod - 1)) >= kTicketPeriod - kTicketMargin) {
        launchFill(s, f.block, kFlatSlotBytes);
        launchFill(s, reinterpret_cast<char *>(f.block) + kFlatSlotBytes + kFlatCounterBytes, kFlatStateBytes);
        f.ticket = (f.ticket | (kTicketPeriod - 1)) + 1;  // the next ticket is this + 1 (zero is skipped by nextSlotTicket)
    }
    w.fault = reinterpret_cast<unsigned *>(reinterpret_cast<char *>(pinnedSlotLocked(s).block) + kPinnedFaultOffset);
    w.slots = reinterpret_cast<unsigned long long *>(f.block);
    w.slotBytes = kFlatSlotBytes;
    w.counter = reinterpret_cast<unsigned *>(reinterpret_cast<char *>(f.block) + kFlatSlotBytes);
    w.rowStates = reinterpret_cast<unsigned *>(reinterpret_cast<char *>(f.block) + kFlatSlotBytes + kFlatCounterBytes);
    w.rowStateCount = kFlatStateBytes / sizeof(unsigned);
    w.slotTicketSource = &f.ticket;  // map nodes stay where they are
}

static unsigned *faultWordIfAny(hipStream_t s) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    std::lock_guard<std::mutex> lock(gMutex);
    auto it = gPinnedSlots.find(std::make_pair(dev, s));
    if (it == gPinnedSlots.end() || it->second.block == nullptr) return nullptr;
    return reinterpret_cast<unsigned *>(reinterpret_cast<char *>(it->second.block) + kPinnedFaultOffset);
}

void *pinnedScalarFor(hipStream_t s) {
    std::lock_guard<std::mutex> lock(gMutex);
    return pinnedSlotLocked(s).block;
}

ScalarSignal nextScalarSignal(hipStream_t s) {
    std::lock_guard<std::mutex> lock(gMutex);
    PinnedSlot &p = pinnedSlotLocked(s);
    ScalarSignal sig;
    sig.words = reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(p.block) + 128);
    sig.plain = p.block;
    sig.fault = reinterpret_cast<unsigned *>(reinterpret_cast<char *>(p.block) + kPinnedFaultOffset);
    sig.ticket = ++p.ticket;
    if (sig.ticket == 0) sig.ticket = ++p.ticket;  // zero is what a fresh slot holds
    return sig;
}

void takeScalar(const ScalarSignal &sig, hipStream_t s, const char *what, void *value, size_t bytes) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) throwHip(what, e);
    const int words = (int)((bytes + 3) / 4);
    const volatile unsigned long long *tagged = sig.words;
    auto arrived = [&]() {
        for (int i = 0; i < words; i++)
            if ((unsigned)(tagged[i] >> 32) != sig.ticket) return false;
        return true;
    };
    bool have = false;
    if (sig.words == nullptr || environment().debug.load()) {
        e = hipStreamSynchronize(s);
        if (e != hipSuccess) throwHip(what, e);
    } else {
        // Spin on the words alone at first (asking the runtime about the stream costs microseconds and delays the answer);
        // a launch that failed or wrote nothing never tags them, so from 50 us on the stream is asked as well.
        const auto start = std::chrono::steady_clock::now();
        auto nextQuery = start + std::chrono::microseconds(50);
        for (unsigned spins = 1; !(have = arrived()); spins++) {
#if defined(__x86_64__)
            __builtin_ia32_pause();  // leaves the core's shared resources to a sibling thread while this one spins
#endif
            if ((spins & 0xff) != 0) continue;
            const auto now = std::chrono::steady_clock::now();
            if (now < nextQuery) continue;
            if (now - start > std::chrono::microseconds(300)) {
                // a long kernel: wait the runtime's way (which may yield the core) rather than spin on
                e = hipStreamSynchronize(s);
                if (e != hipSuccess) throwHip(what, e);
                break;
            }
            e = hipStreamQuery(s);
            if (e == hipSuccess) break;
            if (e != hipErrorNotReady) throwHip(what, e);
            nextQuery = now + std::chrono::microseconds(20);
        }
    }
    std::atomic_thread_fence(std::memory_order_acquire);
    if (!have && sig.words != nullptr) have = arrived();  // the stream has drained: the words are there if they were written
    throwOnFault(sig.fault, what);
    if (have) {
        unsigned w[4] = {0, 0, 0, 0};
        for (int i = 0; i < words && i < 4; i++) w[i] = (unsigned)tagged[i];
        std::memcpy(value, w, bytes);
    } else if (sig.plain != nullptr) {
        // no kernel of this call tagged the words: take the plain copy at the start of the block
        std::memcpy(value, sig.plain, bytes);
    } else {
        throw std::runtime_error(std::string(what) + ": no scalar slot to read the result from");
    }
}

void releaseStreamResources(hipStream_t s) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    const auto key = std::make_pair(dev, s);
    Workspace w;
    w.ptr = nullptr;
    void *slots = nullptr, *pinned = nullptr;
    {
        std::lock_guard<std::mutex> lock(gMutex);
        auto wi = gWorkspaces.find(key);
        if (wi != gWorkspaces.end()) { w = wi->second; gWorkspaces.erase(wi); }
        auto fi = gFlatSlots.find(key);
        if (fi != gFlatSlots.end()) { slots = fi->second.block; gFlatSlots.erase(fi); }
        auto pi = gPinnedSlots.find(key);
        if (pi != gPinnedSlots.end()) { pinned = pi->second.block; gPinnedSlots.erase(pi); }
    }
    if (w.ptr == nullptr && slots == nullptr && pinned == nullptr) return;
    hipError_t e = hipStreamSynchronize(s);  // what is queued on the stream may still use them
    if (e != hipSuccess) throwHip("releaseStreamResources", e);
    if (w.ptr != nullptr) (void)hipFree(w.ptr);
    if (slots != nullptr) (void)hipFree(slots);
    if (pinned != nullptr) (void)hipHostFree(pinned);
}

void setSlotTicketForTesting(hipStream_t s, unsigned value) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    std::lock_guard<std::mutex> lock(gMutex);
    gFlatSlots[std::make_pair(dev, s)].ticket = value;
}

bool resolveTad(Nd4jPointer *extra, int hostSlot, int offsetSlot, const Long *hostXInfo, const int *dimension,
                int dimLen, ResolvedTad &out, hipStream_t s) {
    const Long *hostTad = reinterpret_cast<const Long *>(slotOf(extra, hostSlot));
    const Long *devOff = reinterpret_cast<const Long *>(slotOf(extra, offsetSlot));
    if (hostTad != nullptr && devOff != nullptr) {
        out.hostInfo = hostTad;
        out.devOffsets = devOff;
        out.tadLength = siNumel(hostTad);
        out.numTads = out.tadLength > 0 ? siNumel(hostXInfo) / out.tadLength : 0;
        return true;
    }
    std::vector<int> dims;
    if (!hostInts(dimension, dimLen, dims, s)) return false;
    int rank = siRank(hostXInfo);
    for (int &d : dims) {
        if (d < 0) d += rank;
        if (d < 0 || d >= rank) return false;
    }
    std::vector<Long> key(hostXInfo, hostXInfo + siLength(rank));
    key.push_back(-777);
    for (int d : dims) key.push_back(d);
    int dev = 0;
    (void)hipGetDevice(&dev);
    key.push_back(dev);  // the offsets live in this device's memory

    std::map<std::vector<Long>, std::shared_ptr<CachedTad> > dropped;  // destroyed after the lock below is gone
    std::unique_lock<std::mutex> lock(gMutex);
    auto it = gTadCache.find(key);
    std::shared_ptr<CachedTad> c;
    if (it != gTadCache.end()) {
        c = it->second;
    } else {
        if (gTadCache.size() >= kTadCacheLimitEntries || gTadCacheBytes >= kTadCacheLimitBytes) takeTadCacheLocked(dropped);
        c = std::make_shared<CachedTad>();
        computeTad(hostXInfo, dims.data(), dimLen, c->pack, true);
        c->tadLength = tadLengthOf(hostXInfo, dims.data(), dimLen);
        size_t bytes = c->pack.offsets.size() * sizeof(Long);
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&c->devOffsets), bytes ? bytes : sizeof(Long));
        if (e != hipSuccess) { c->devOffsets = nullptr; throwHip("TAD offsets allocation", e); }
        if (bytes) {
            e = hipMemcpy(c->devOffsets, c->pack.offsets.data(), bytes, hipMemcpyHostToDevice);
            if (e != hipSuccess) throwHip("TAD offsets upload", e);
        }
        gTadCache[key] = c;
        gTadCacheBytes += bytes + c->pack.shapeInfo.size() * sizeof(Long) + key.size() * sizeof(Long);
    }
    out.keep = c;
    out.hostInfo = c->pack.shapeInfo.data();
    out.devOffsets = c->devOffsets;
    out.numTads = c->pack.numTads;
    out.tadLength = c->tadLength;
    lock.unlock();
    dropped.clear();
    return true;
}

}  // namespace nd4j_amd
