// Index-reduce family: (value, index) reductions; the winning index is stored in the data type.
// Reference loops: include/loops/cpu/indexreduce.cpp:36-129 (scalar), 131-228 (per TAD); functors:
// include/ops/ops.h:2992-3466; opNum table: include/loops/legacy_ops.h:287-293.
// Ties resolve to the lowest index (the reference's device rule, ops.h:3256-3259), which is also what the
// reference's sequential CPU scans produce.
#include "launch.h"
#include "reduce_engine.cuh"

namespace nd4j_amd {

template <typename C> struct IndexAcc;
template <> struct IndexAcc<float> { Long index; float value; float pad; };
template <> struct IndexAcc<double> { Long index; double value; };

// MAX_FLOAT / MIN_FLOAT of ops.h:21-22
template <typename C> __device__ __forceinline__ C bigValue() { return (C)1e37; }
template <typename C> __device__ __forceinline__ C tinyValue() { return (C)1e-37; }

template <typename TT, int OP> struct IndexPol {
    typedef TT T;
    typedef typename Compute<TT>::type C;
    typedef IndexAcc<C> Acc;
    static constexpr bool tables = false;  // no exp / log / pow in these accumulators
    static constexpr int kChains = 4;      // accumulators of one lane may be kept apart and combined (ties go to the lower index)
    static constexpr int kSlotWords = 2 + sizeof(C) / 4;  // index and value; the float accumulator's padding word stays behind
    static constexpr int kFlatBlocks = 768;   // blocks of the whole-array kernel: three per compute unit (see runFlatReduce)
    Params<TT> p;

    __device__ __forceinline__ void setTad(Long, const TT *) {}
    __device__ __forceinline__ Acc init(const TT *) const {
        Acc a;
        a.index = (OP == 4 || OP == 5) ? -1 : 0;
        if (OP == 0) a.value = -bigValue<C>();            // IndexMax
        else if (OP == 1 || OP == 3) a.value = bigValue<C>();  // IndexMin, IndexAbsoluteMin
        else if (OP == 2) a.value = tinyValue<C>();       // IndexAbsoluteMax
        else a.value = -bigValue<C>();                    // FirstIndex / LastIndex
        if (sizeof(Acc) > sizeof(Long) + sizeof(C)) zeroPad(a);
        return a;
    }
    static __device__ __forceinline__ void zeroPad(IndexAcc<float> &a) { a.pad = 0.0f; }
    static __device__ __forceinline__ void zeroPad(IndexAcc<double> &) {}

    // true when candidate (v, i) replaces (a.value, a.index)
    __device__ __forceinline__ bool better(C v, Long i, C av, Long ai) const {
        if (OP == 0 || OP == 2) return v > av || (v == av && i < ai);
        return v < av || (v == av && i < ai);
    }
    __device__ __forceinline__ void accumulate(Acc &a, C v, Long i) const {
        if (OP <= 3) {
            C c = (OP == 2 || OP == 3) ? m::abs_(v) : v;
            if (better(c, i, a.value, a.index)) { a.value = c; a.index = i; }
        } else {
            // FirstIndex / LastIndex: the element qualifies when MatchCondition::op(value, extra) != 0
            if (matchConditionOp<C>(v, p) != (C)0) {
                if (a.index < 0 || (OP == 4 ? i < a.index : i > a.index)) { a.index = i; a.value = v; }
            }
        }
    }
    // the same for an element that lies behind everything the accumulator has seen: a tie never replaces
    static constexpr bool hasAscending = true;
    __device__ __forceinline__ void accumulateAscending(Acc &a, C v, Long i) const {
        if (OP <= 3) {
            C c = (OP == 2 || OP == 3) ? m::abs_(v) : v;
            const bool wins = (OP == 0 || OP == 2) ? c > a.value : c < a.value;
            a.value = wins ? c : a.value;
            a.index = wins ? i : a.index;
        } else if (matchConditionOp<C>(v, p) != (C)0) {
            if (OP == 5 || a.index < 0) { a.index = i; a.value = v; }
        }
    }
    __device__ __forceinline__ void checkpoint(Acc &) const {}
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const {
        if (OP <= 3) {
            return better(b.value, b.index, a.value, a.index) ? b : a;
        }
        if (b.index < 0) return a;
        if (a.index < 0) return b;
        if (OP == 4) return b.index < a.index ? b : a;
        return b.index > a.index ? b : a;
    }
    __device__ __forceinline__ TT finalize(Acc a, Long) const { return fromCompute<TT>((C)a.index); }
};

static constexpr int kIndexReduceOpCount = 6;

template <typename T> struct IndexTadBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const T *x, const T *extra, T *z, const TadPlan &pl, Workspace ws) {
            IndexPol<T, OP> pol;
            pol.p.p = extra;
            runTadReduce(s, pol, x, z, pl, ws);
            return true;
        }
    };
};
template <typename T> struct IndexFlatBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, const T *x, const T *extra, T *z, const FlatPlan &pl, Workspace ws) {
            IndexPol<T, OP> pol;
            pol.p.p = extra;
            runFlatReduce(s, pol, x, z, pl, ws);
            return true;
        }
    };
};

template <typename T>
bool launchIndexReduceTad(hipStream_t s, int opNum, const T *x, const T *extra, T *z, const TadPlan &plan, Workspace ws) {
    return dispatchSeq<IndexTadBody<T>::template Run>(opNum, std::make_integer_sequence<int, kIndexReduceOpCount>{}, s, x,
                                                      extra, z, plan, ws);
}
template <typename T>
bool launchIndexReduceScalar(hipStream_t s, int opNum, const T *x, const T *extra, T *z, const FlatPlan &plan,
                             Workspace ws) {
    return dispatchSeq<IndexFlatBody<T>::template Run>(opNum, std::make_integer_sequence<int, kIndexReduceOpCount>{}, s, x,
                                                       extra, z, plan, ws);
}

#define INST(T)                                                                                                       \
    template bool launchIndexReduceTad<T>(hipStream_t, int, const T *, const T *, T *, const TadPlan &, Workspace);   \
    template bool launchIndexReduceScalar<T>(hipStream_t, int, const T *, const T *, T *, const FlatPlan &, Workspace);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
