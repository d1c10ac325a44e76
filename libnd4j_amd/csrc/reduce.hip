// Reduce family: acc = update(acc, op(x, extra)); result = postProcess(acc, n, extra).
// Reference loops: include/loops/cpu/reduce.cpp:14-64 (scalar), 91-193 (per TAD), 206-323 (strided scalar);
// functors: include/ops/ops.h:1534-2560 and include/ops/special_accumulation_ops.h:16-45; opNum table:
// include/loops/legacy_ops.h:195-221.  Partial accumulators are merged with `update`, never `merge`,
// exactly as both reference back ends do (cpu/reduce.cpp:258-260).
#include <mutex>
#include <stdexcept>
#include <string>

#include "launch.h"
#include "reduce_engine.cuh"

namespace nd4j_amd {

// Scratch of the whole-array reduction that allocates nothing (launchReduceScalarNoAlloc below): the first 256 bytes
// hold the maximum that LogSumExp's first pass leaves for its second, the rest the per-block partial accumulators.
// Every GPU the library runs on holds its own copy of this array until the process ends.  Host code never uses the
// array's name as an address: it asks for the array's address on the current device once, and passes that on.
static constexpr size_t kNoAllocScratchBytes = 64 * 1024;
static constexpr size_t kNoAllocPartialsOffset = 256;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

enum StartKind { START_ZERO, START_ONE, START_FIRST };

template <int OP> struct ReduceOp { static constexpr bool valid = false; };

#define ND4J_REDUCE(OP, NAME, START, OPBODY, UPDBODY, POSTBODY)                                                   \
    template <> struct ReduceOp<OP> {                                                                             \
        static constexpr bool valid = true;                                                                       \
        static constexpr StartKind start = START;                                                                 \
        template <typename C, typename P> static __device__ __forceinline__ C op(C d1, P p, C shift) { OPBODY }   \
        template <typename C> static __device__ __forceinline__ C update(C old, C v) { UPDBODY }                  \
        template <typename C, typename P> static __device__ __forceinline__ C post(C r, Long n, P p, C shift) {   \
            POSTBODY                                                                                              \
        }                                                                                                         \
    };
#define ND4J_SUM_UPD return v + old;

ND4J_REDUCE(0, Mean, START_ZERO, return d1;, ND4J_SUM_UPD, return r / (C)(int)n;)
ND4J_REDUCE(1, Sum, START_ZERO, return d1;, ND4J_SUM_UPD, return r;)
ND4J_REDUCE(3, Max, START_FIRST, return d1;, return m::max_(v, old);, return r;)
ND4J_REDUCE(4, Min, START_FIRST, return d1;, return m::min_(v, old);, return r;)
ND4J_REDUCE(5, Norm1, START_ZERO, return m::abs_(d1);, ND4J_SUM_UPD, return r;)
ND4J_REDUCE(6, Norm2, START_ZERO, return d1 * d1;, ND4J_SUM_UPD, return m::sqrt_(r);)
ND4J_REDUCE(7, NormMax, START_ZERO, return d1;, return m::max_(m::abs_(old), m::abs_(v));, return m::abs_(r);)
ND4J_REDUCE(8, Prod, START_ONE, return d1;, return v * old;, return r;)
// Variance / StandardDeviation as reduce ops expect the mean in extra[0] and a bias term in extra[1]
// (ops.h:2500-2560)
ND4J_REDUCE(9, StandardDeviation, START_ZERO, {
    C d = d1 - p[0];
    return d * d;
}, return old + v;, {
    C bias = p[1];
    C var = (r - (m::pow_(bias, (C)2) / (C)(int)n)) / (C)(n - 1);
    return m::sqrt_(var);
})
ND4J_REDUCE(10, Variance, START_ZERO, {
    C d = d1 - p[0];
    return d * d;
}, return old + v;, {
    C bias = p[1];
    return (r - (m::pow_(bias, (C)2) / (C)(int)n)) / (C)(n - 1);
})
ND4J_REDUCE(11, ASum, START_ZERO, return m::abs_(d1);, return m::abs_(v) + m::abs_(old);, return m::abs_(r);)
ND4J_REDUCE(12, MatchCondition, START_ZERO, return matchConditionOp<C>(d1, p);, return old + v;, return r;)
ND4J_REDUCE(13, AMax, START_FIRST, return m::abs_(d1);, return m::max_(m::abs_(v), m::abs_(old));, return m::abs_(r);)
ND4J_REDUCE(14, AMin, START_FIRST, return m::abs_(d1);, return m::min_(m::abs_(v), m::abs_(old));, return m::abs_(r);)
ND4J_REDUCE(15, AMean, START_ZERO, return m::abs_(d1);, return m::abs_(v) + m::abs_(old);, return m::abs_(r) / (C)(int)n;)
ND4J_REDUCE(16, Entropy, START_ZERO, return d1 * m::log_(d1);, ND4J_SUM_UPD, return r;)
ND4J_REDUCE(17, LogEntropy, START_ZERO, return m::log_(m::pow_(d1, (C)2));, ND4J_SUM_UPD, return r;)
ND4J_REDUCE(18, ShannonEntropy, START_ZERO, return m::pow_(d1, (C)2) * m::log_(m::pow_(d1, (C)2));, ND4J_SUM_UPD, return -r;)
// LogSumExp: `shift` is the maximum computed by the pre-pass (blas/cpu/NativeOpExcutioner.cpp:122-147)
ND4J_REDUCE(19, LogSumExp, START_ZERO, return m::exp_(d1 - shift);, ND4J_SUM_UPD, return shift + m::log_(r);)
ND4J_REDUCE(20, Any, START_ZERO, return d1;, ND4J_SUM_UPD, return r > (C)0 ? (C)1 : (C)0;)
ND4J_REDUCE(21, All, START_ONE, return d1;, return v * old;, return r > (C)0 ? (C)1 : (C)0;)
ND4J_REDUCE(22, CountNonZero, START_ZERO, return d1 == (C)0 ? (C)0 : (C)1;, ND4J_SUM_UPD, return r;)
ND4J_REDUCE(23, NormFrobenius, START_ZERO, {
    C a = m::abs_(d1);
    return a * a;
}, ND4J_SUM_UPD, return m::sqrt_(r);)
ND4J_REDUCE(24, NormP, START_ZERO, return m::pow_(m::abs_(d1), (C)p[0]);, ND4J_SUM_UPD, return m::pow_(r, (C)1 / (C)p[0]);)
ND4J_REDUCE(25, SquaredNorm, START_ZERO, return d1 * d1;, ND4J_SUM_UPD, return r;)
ND4J_REDUCE(26, CountZero, START_ZERO, return d1 == (C)0 ? (C)1 : (C)0;, ND4J_SUM_UPD, return r;)
#undef ND4J_REDUCE
#undef ND4J_SUM_UPD

static constexpr int kReduceOpCount = 27;

template <typename TT, int OP> struct ReducePol {
    typedef TT T;
    typedef typename Compute<TT>::type C;
    typedef C Acc;
    // ops whose functor or post-processing evaluates exp / log / pow (variance and standard deviation square their
    // bias term with pow); 20-23 have no functor
    static constexpr bool tables = OP == 9 || OP == 10 || (OP >= 16 && OP <= 24);
    static constexpr int kChains = 4;  // accumulators of one lane may be kept apart and combined (combine is the update)
    static constexpr int kFlatBlocks = 512;  // blocks of the whole-array kernel: two per compute unit (see runFlatReduce)
    static constexpr int kColBlocks = 512;   // and of the strided vector kernel (see runTadReduce)
    Params<TT> p;
    const TT *shiftSource;  // LogSumExp: per-TAD (TAD calls) or single (scalar calls) maximum; else null
    int shiftPerTad;
    C shift;

    __device__ __forceinline__ void setTad(Long r, const TT *) {
        if (OP == 19) shift = toCompute(shiftSource[shiftPerTad ? r : 0]);
    }
    __device__ __forceinline__ Acc init(const TT *first) const {
        if (ReduceOp<OP>::start == START_FIRST) return toCompute(first[0]);
        return ReduceOp<OP>::start == START_ONE ? (C)1 : (C)0;
    }
    __device__ __forceinline__ void accumulate(Acc &a, C v, Long) const {
        a = ReduceOp<OP>::template update<C>(a, ReduceOp<OP>::template op<C>(v, p, shift));
    }
    __device__ __forceinline__ void checkpoint(Acc &) const {}
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return ReduceOp<OP>::template update<C>(a, b); }
    __device__ __forceinline__ TT finalize(Acc a, Long n) const {
        return fromCompute<TT>(ReduceOp<OP>::template post<C>(a, n, p, shift));
    }
};

template <typename T> struct ReduceTadBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const T *x, const T *extra, T *z, const TadPlan &pl, Workspace ws) {
            if constexpr (ReduceOp<OP>::valid) {
                ReducePol<T, OP> pol;
                pol.p.p = extra;
                pol.shiftSource = z;  // LogSumExp: z already holds the per-TAD maxima
                pol.shiftPerTad = 1;
                pol.shift = 0;
                runTadReduce(s, pol, x, z, pl, ws);
                return true;
            } else {
                return false;
            }
        }
    };
};
template <typename T> struct ReduceFlatBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const T *x, const T *extra, T *z, const FlatPlan &pl, Workspace ws) {
            if constexpr (ReduceOp<OP>::valid) {
                ReducePol<T, OP> pol;
                pol.p.p = extra;
                pol.shiftSource = extra;  // LogSumExp: the caller passes the device scalar holding the maximum
                pol.shiftPerTad = 0;
                pol.shift = 0;
                runFlatReduce(s, pol, x, z, pl, ws);
                return true;
            } else {
                return false;
            }
        }
    };
};

template <typename T>
bool launchReduceTad(hipStream_t s, int opNum, const T *x, const T *extra, T *z, const TadPlan &plan, Workspace ws) {
    return dispatchSeq<ReduceTadBody<T>::template Run>(opNum, std::make_integer_sequence<int, kReduceOpCount>{}, s, x,
                                                       extra, z, plan, ws);
}
template <typename T>
bool launchReduceScalar(hipStream_t s, int opNum, const T *x, const T *extra, T *z, const FlatPlan &plan, Workspace ws) {
    return dispatchSeq<ReduceFlatBody<T>::template Run>(opNum, std::make_integer_sequence<int, kReduceOpCount>{}, s, x,
                                                        extra, z, plan, ws);
}

// Row maximum and row sum of exp(x - maximum) in ONE pass, for the softmax family over rows too long for registers:
// the running sum is rescaled whenever the running maximum rises, so each element costs one exp.  Not an op of the
// reference (its loops take the maximum first, special_ops.h:1488-1518); the sums differ from a two-pass sum by the
// roundings of the few rescalings.  The maximum is the stored result, the sum goes to a second per-row array.
template <typename TT> struct SoftmaxStatsPol {
    typedef TT T;
    typedef typename Compute<TT>::type C;
    struct Acc { C m, s; };
    static constexpr bool tables = false;  // its exp runs on the hardware's exp2
    C *sums;  // in the compute type: a row sum of a half array may exceed the range of half
    Long row;

    __device__ __forceinline__ void setTad(Long r, const TT *) { row = r; }
    __device__ __forceinline__ Acc init(const TT *first) const {
        Acc a;
        a.m = toCompute(first[0]);
        a.s = (C)0;
        return a;
    }
    __device__ __forceinline__ void accumulate(Acc &a, C v, Long) const {
        const C d = v - a.m;
        const C e = m::expSoft_(-m::abs_(d));
        const bool rises = d > (C)0;
        a.s = rises ? a.s * e + (C)1 : a.s + e;
        a.m = rises ? v : a.m;
    }
    __device__ __forceinline__ void checkpoint(Acc &) const {}
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const {
        Acc r;
        r.m = m::max_(a.m, b.m);
        // an accumulator that has seen nothing yet holds s == 0 and the row's first element as m
        r.s = a.s * m::expSoft_(a.m - r.m) + b.s * m::expSoft_(b.m - r.m);
        return r;
    }
    __device__ __forceinline__ TT finalize(Acc a, Long) const {
        sums[row] = a.s;
        return fromCompute<TT>(a.m);
    }
};

template <typename T>
bool launchSoftmaxStats(hipStream_t s, const T *x, T *maxima, typename Compute<T>::type *sums, const TadPlan &plan, Workspace ws) {
    SoftmaxStatsPol<T> pol;
    pol.sums = sums;
    pol.row = 0;
    runTadReduce(s, pol, x, maxima, plan, ws);
    return true;
}

// ---- the whole-array reduction over the static scratch ---------------------------------------------------
namespace {
constexpr int kScratchDevices = 64;
std::mutex gScratchMutex;
void *gScratchAddress[kScratchDevices] = {};

// Address of `scratch` on the current device, looked up once per device.
void *scratchOnCurrentDevice() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) throw std::runtime_error(std::string("hipGetDevice: ") + hipGetErrorString(e));
    if (dev < 0 || dev >= kScratchDevices) throw std::runtime_error("device index beyond the no-allocation scratch table");
    std::lock_guard<std::mutex> lock(gScratchMutex);
    if (gScratchAddress[dev] == nullptr) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            throw std::runtime_error(std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e));
        gScratchAddress[dev] = ptr;
    }
    return gScratchAddress[dev];
}
}  // namespace

void prepareNoAllocScratch() { (void)scratchOnCurrentDevice(); }

// The two-launch form this entry point takes (flatKernel into partials, flatFinish over them) and the one-launch form of
// execReduceFloat fold the same blocks in the same order only while every block's accumulator fits the scratch array:
// the "bit for bit" promise of the header rests on that.
static_assert((kNoAllocScratchBytes - kNoAllocPartialsOffset) / sizeof(float) >= kFlatMaxBlocks,
              "the no-allocation scratch must hold one float accumulator per block of the largest whole-array grid");

bool launchReduceScalarNoAlloc(hipStream_t s, int opNum, const float *x, const float *extra, float *z, const FlatPlan &plan) {
    char *base = reinterpret_cast<char *>(scratchOnCurrentDevice());
    Workspace ws;
    ws.ptr = base + kNoAllocPartialsOffset;
    ws.bytes = kNoAllocScratchBytes - kNoAllocPartialsOffset;
    if (opNum == 19) {
        // LogSumExp: the maximum first, then exp(x - maximum) summed (blas/cpu/NativeOpExcutioner.cpp:138-141)
        float *maxSlot = reinterpret_cast<float *>(base);
        if (!launchReduceScalar<float>(s, 3, x, extra, maxSlot, plan, ws)) return false;
        return launchReduceScalar<float>(s, 19, x, maxSlot, z, plan, ws);
    }
    return launchReduceScalar<float>(s, opNum, x, extra, z, plan, ws);
}

#define INST(T)                                                                                                    \
    template bool launchReduceTad<T>(hipStream_t, int, const T *, const T *, T *, const TadPlan &, Workspace);     \
    template bool launchReduceScalar<T>(hipStream_t, int, const T *, const T *, T *, const FlatPlan &, Workspace); \
    template bool launchSoftmaxStats<T>(hipStream_t, const T *, T *, Compute<T>::type *, const TadPlan &, Workspace);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
