// Summary-stats family: variance / standard deviation from moments accumulated in double.
// Reference: include/loops/cpu/summarystatsreduce.cpp:24-196; moment merge
// include/loops/summarystatsreduce.h:221-257 (Chan et al. parallel update); getValue include/ops/ops.h:3471-3509.
//
// Each lane gathers runs of samples as shifted sums (count, sum(x-c), sum((x-c)^2) around a shift c), turns a closed
// run into (n, mean, M2) and merges it with the pairwise formula the reference applies sample by sample.  Only n,
// mean and M2 are carried: min/max/M3/M4 never reach variance or standard deviation.
//
// The shift is a sample of the same TAD (its first one) until a lane closes a run, the merged mean afterwards.  With
// M2 = sum(e^2) - (sum e)^2 / n the cancellation is 1 + (mean(e) / sigma)^2, at worst the run length + 1 (every sample
// equal but the one that became the shift): runs of up to kStatsRun samples lose at most 2^17 of double precision's
// 2^53.  So a lane rarely closes a run before the merge, and lanes that have not merge by adding their sums.
#include "launch.h"
#include "reduce_engine.cuh"

namespace nd4j_amd {

struct StatsAcc {
    double n, mean, m2;  // merged so far
    double cs1, cs2;     // current run: sum(x - cp), sum((x - cp)^2)
    double cp;           // current shift (a value the data type holds exactly)
    int cn, pad;         // current run: count
};

static constexpr int kStatsRun = 65536;

__device__ __forceinline__ void statsMerge(double &n, double &mean, double &m2, double nb, double meanb, double m2b) {
    if (nb == 0.0) return;
    if (n == 0.0) { n = nb; mean = meanb; m2 = m2b; return; }
    double tot = n + nb;
    double delta = meanb - mean;
    mean = mean + delta * nb / tot;
    m2 = m2 + m2b + delta * delta * n * nb / tot;
    n = tot;
}
// closes the current run; the next one is shifted by the merged mean, rounded to what the data type holds
template <typename C> __device__ __forceinline__ void statsFlush(StatsAcc &a) {
    if (a.cn == 0) return;
    const double cn = (double)a.cn;
    double meanb = a.cp + a.cs1 / cn;
    double m2b = a.cs2 - a.cs1 * a.cs1 / cn;
    if (m2b < 0.0) m2b = 0.0;
    statsMerge(a.n, a.mean, a.m2, cn, meanb, m2b);
    a.cn = 0; a.cs1 = 0.0; a.cs2 = 0.0;
    a.cp = (double)(C)a.mean;
}

template <typename TT, int OP> struct StatsPol {
    typedef TT T;
    typedef typename Compute<TT>::type C;
    typedef StatsAcc Acc;
    static constexpr bool tables = false;  // no exp / log / pow in these accumulators
    static constexpr int kColBlocks = 1024;  // blocks of the strided vector kernel (see runTadReduce)
    int biasCorrected;
    int phantomZero;  // the reference's single-dimension non-EWS branch starts from a zero sample

    __device__ __forceinline__ void setTad(Long, const TT *) {}
    // Every lane's first run is shifted by the same value, the first sample of the TAD (of the array): lanes that have
    // not closed a run yet then merge by adding their sums (combine), which is what the merge tree consists of.
    __device__ __forceinline__ Acc init(const TT *first) const {
        Acc a;
        a.n = a.mean = a.m2 = 0.0;
        a.cs1 = a.cs2 = 0.0;
        a.cn = a.pad = 0;
        a.cp = (double)toCompute(first[0]);
        return a;
    }
    // The difference to the shift is taken in the compute type: shift and sample are both values of that type, and where
    // the difference matters (samples close to the shift) it is exact; sums and squares are kept in double.
    __device__ __forceinline__ void accumulate(Acc &a, C v, Long) const {
        const double e = (double)(v - (C)a.cp);
        a.cs1 += e;
        a.cs2 = __builtin_fma(e, e, a.cs2);
        a.cn += 1;
    }
    // closes the current run once it holds kStatsRun samples or more (kept out of accumulate() so that the
    // per-sample code is straight-line)
    __device__ __forceinline__ void checkpoint(Acc &a) const {
        if (a.cn >= kStatsRun) statsFlush<C>(a);
    }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const {
        // two open first runs around the common shift: no divisions (the count is a 32-bit integer: longer runs are closed)
        if (a.n == 0.0 && b.n == 0.0 && a.cp == b.cp && a.cn <= (1 << 29) && b.cn <= (1 << 29)) {
            a.cn += b.cn;
            a.cs1 += b.cs1;
            a.cs2 += b.cs2;
            return a;
        }
        statsFlush<C>(a);
        statsFlush<C>(b);
        statsMerge(a.n, a.mean, a.m2, b.n, b.mean, b.m2);
        return a;
    }
    // While no lane of the wave has closed a run, every lane holds two sums and a count around the TAD's common shift:
    // those are all that has to travel (5 words per step instead of 16), and they merge by addition.
    static constexpr bool ownWaveMerge = true;
    template <int WIDTH> __device__ __forceinline__ Acc waveMergeOwn(Acc a) const {
        if (__all(a.n == 0.0 && a.cn <= (1 << 24))) {
#pragma unroll
            for (int d = WIDTH / 2; d >= 1; d >>= 1) {
                // (lanes of one segment work on one TAD and share its shift; what arrives from beyond the segment's end
                // lands in lanes whose result is not used)
                a.cn += __shfl_down(a.cn, d, kWave);
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
        statsFlush<C>(a);
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
