// Summary-stats family: variance / standard deviation from moments accumulated in double.
// Reference: include/loops/cpu/summarystatsreduce.cpp:24-196; moment merge
// include/loops/summarystatsreduce.h:221-257 (Chan et al. parallel update); getValue include/ops/ops.h:3471-3509.
//
// Each lane gathers short runs of samples as shifted sums (count, sum(x-c), sum((x-c)^2) around the run's
// first sample c), turns a full run into (n, mean, M2) and merges it with the pairwise formula the
// reference applies sample by sample.  Only n, mean and M2 are carried: min/max/M3/M4 never reach
// variance or standard deviation.
#include "launch.h"
#include "reduce_engine.cuh"

namespace nd4j_amd {

struct StatsAcc {
    double n, mean, m2;      // merged so far
    double cn, cs1, cs2, cp; // current run: count, shifted sums, shift
};

static constexpr double kStatsRun = 128.0;

__device__ __forceinline__ void statsMerge(double &n, double &mean, double &m2, double nb, double meanb, double m2b) {
    if (nb == 0.0) return;
    if (n == 0.0) { n = nb; mean = meanb; m2 = m2b; return; }
    double tot = n + nb;
    double delta = meanb - mean;
    mean = mean + delta * nb / tot;
    m2 = m2 + m2b + delta * delta * n * nb / tot;
    n = tot;
}
__device__ __forceinline__ void statsFlush(StatsAcc &a) {
    if (a.cn == 0.0) return;
    double meanb = a.cp + a.cs1 / a.cn;
    double m2b = a.cs2 - a.cs1 * a.cs1 / a.cn;
    if (m2b < 0.0) m2b = 0.0;
    statsMerge(a.n, a.mean, a.m2, a.cn, meanb, m2b);
    a.cn = 0.0; a.cs1 = 0.0; a.cs2 = 0.0;
}

template <typename TT, int OP> struct StatsPol {
    typedef TT T;
    typedef typename Compute<TT>::type C;
    typedef StatsAcc Acc;
    static constexpr bool tables = false;  // no exp / log / pow in these accumulators
    int biasCorrected;
    int phantomZero;  // the reference's single-dimension non-EWS branch starts from a zero sample

    __device__ __forceinline__ void setTad(Long, const TT *) {}
    // Every lane's first run is shifted by the same value, the first sample of the TAD (of the array): lanes that have
    // not closed a run yet then merge by adding their three sums (combine), which is what the merge tree of a short
    // TAD consists of.  A run opened after a merge is shifted by its own first sample, as before.
    __device__ __forceinline__ Acc init(const TT *first) const {
        Acc a;
        a.n = a.mean = a.m2 = 0.0;
        a.cn = a.cs1 = a.cs2 = 0.0;
        a.cp = (double)toCompute(first[0]);
        return a;
    }
    __device__ __forceinline__ void accumulate(Acc &a, C v, Long) const {
        double d = (double)v;
        if (a.cn == 0.0 && a.n != 0.0) a.cp = d;
        double e = d - a.cp;
        a.cs1 += e;
        a.cs2 += e * e;
        a.cn += 1.0;
    }
    // closes the current run once it holds kStatsRun samples or more (kept out of accumulate() so that the
    // per-sample code is straight-line)
    __device__ __forceinline__ void checkpoint(Acc &a) const {
        if (a.cn >= kStatsRun) statsFlush(a);
    }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const {
        if (a.n == 0.0 && b.n == 0.0 && a.cp == b.cp) {  // two open first runs around the common shift: no divisions
            a.cn += b.cn;
            a.cs1 += b.cs1;
            a.cs2 += b.cs2;
            return a;
        }
        statsFlush(a);
        statsFlush(b);
        statsMerge(a.n, a.mean, a.m2, b.n, b.mean, b.m2);
        return a;
    }
    // While no lane of the wave has closed a run, every lane holds three sums around the TAD's common shift: those are
    // all that has to travel (6 words per step instead of 14), and they merge by addition.
    static constexpr bool ownWaveMerge = true;
    template <int WIDTH> __device__ __forceinline__ Acc waveMergeOwn(Acc a) const {
        if (__all(a.n == 0.0)) {
#pragma unroll
            for (int d = WIDTH / 2; d >= 1; d >>= 1) {
                // (lanes of one segment work on one TAD and share its shift; what arrives from beyond the segment's end
                // lands in lanes whose result is not used)
                a.cn += shflDownAny(a.cn, d);
                a.cs1 += shflDownAny(a.cs1, d);
                a.cs2 += shflDownAny(a.cs2, d);
            }
            return a;
        }
#pragma unroll
        for (int d = WIDTH / 2; d >= 1; d >>= 1) a = combine(a, shflDownAny(a, d));
        return a;
    }
    __device__ __forceinline__ TT finalize(Acc a, Long) const {
        statsFlush(a);
        if (phantomZero) {
            double n = 1.0, mean = 0.0, m2 = 0.0;
            statsMerge(n, mean, m2, a.n, a.mean, a.m2);
            a.n = n; a.mean = mean; a.m2 = m2;
        }
        // SummaryStatsData::variance / varianceBiasCorrected (summarystatsreduce.h:94-113)
        double var = a.n <= 1.0 ? 0.0 : a.m2 / a.n;
        double vb = a.n <= 1.0 ? 0.0 : a.m2 / (a.n - 1.0);
        // getValue (ops.h:3477-3509): the bias-corrected value is tested, and for the standard deviation
        // also square-rooted, after its cast to the data type
        C result;
        if (biasCorrected) {
            C r = (C)vb;
            if (OP == 0) result = r < (C)0 ? (C)var : r;
            else result = r < (C)0 ? (C)::sqrt(var) : m::sqrt_(r);
        } else {
            result = (OP == 0) ? (C)var : (C)::sqrt(var);
        }
        return fromCompute<TT>(result);
    }
};

template <typename T> struct StatsTadBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, bool bias, int phantom, const T *x, T *z, const TadPlan &pl, Workspace ws) {
            StatsPol<T, OP> pol;
            pol.biasCorrected = bias ? 1 : 0;
            pol.phantomZero = phantom;
            runTadReduce(s, pol, x, z, pl, ws);
            return true;
        }
    };
};
template <typename T> struct StatsFlatBody {
    template <int OP> struct Run {
        static bool run(hipStream_t s, bool bias, const T *x, T *z, const FlatPlan &pl, Workspace ws) {
            StatsPol<T, OP> pol;
            pol.biasCorrected = bias ? 1 : 0;
            pol.phantomZero = 0;
            runFlatReduce(s, pol, x, z, pl, ws);
            return true;
        }
    };
};

template <typename T>
bool launchSummaryStatsTad(hipStream_t s, int opNum, bool biasCorrected, bool phantomZero, const T *x, T *z,
                           const TadPlan &plan, Workspace ws) {
    return dispatchSeq<StatsTadBody<T>::template Run>(opNum, std::make_integer_sequence<int, 2>{}, s, biasCorrected,
                                                      phantomZero ? 1 : 0, x, z, plan, ws);
}
template <typename T>
bool launchSummaryStatsScalar(hipStream_t s, int opNum, bool biasCorrected, const T *x, T *z, const FlatPlan &plan,
                              Workspace ws) {
    return dispatchSeq<StatsFlatBody<T>::template Run>(opNum, std::make_integer_sequence<int, 2>{}, s, biasCorrected, x, z,
                                                       plan, ws);
}

#define INST(T)                                                                                                     \
    template bool launchSummaryStatsTad<T>(hipStream_t, int, bool, bool, const T *, T *, const TadPlan &, Workspace); \
    template bool launchSummaryStatsScalar<T>(hipStream_t, int, bool, const T *, T *, const FlatPlan &, Workspace);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
