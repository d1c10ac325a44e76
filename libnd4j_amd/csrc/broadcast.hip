// Broadcast family: z[tad][f] = op(x[tad][f], y[f]).  Reference loop: include/loops/cpu/broadcasting.cpp:42-156.
#include "elementwise.cuh"
#include "launch.h"

namespace nd4j_amd {

template <typename T> struct BroadcastBody {
    template <int KIND> struct Run {
        static bool run(hipStream_t s, const T *x, const T *y, T *z, const BroadcastPlan &pl) {
            typedef Broadcast2F<KIND> F;
            if (pl.numTads <= 0 || pl.tadLength <= 0) return true;
            if (pl.kind == BroadcastPlan::ROW && pl.consecutive && pl.tadLength % Pack<T>::N == 0 &&
                pl.tadLength / Pack<T>::N < 0xffffffffLL && (((uintptr_t)x | (uintptr_t)y | (uintptr_t)z) & 15) == 0) {
                const Long nvec = pl.numTads * (pl.tadLength / Pack<T>::N);
                // (blocks of 128 threads, as for two-operand element-wise calls: a row added to [65536, 1024] floats 85.7 -> 83 us;
                // the functors with lookup tables keep the 256 threads their staging is written for)
                const int blk = F::tables ? kBlock : kBlock / 2;
                ND4J_LAUNCH((bcFlatKernel<T, F>), dim3(gridFor(nvec, blk * 2, F::tables ? kGridCap : kMaxGrid)), dim3(blk), 0,
                                   s, x, y, z, nvec, (unsigned)(pl.tadLength / Pack<T>::N), Params<T>{nullptr});
            } else if (pl.kind == BroadcastPlan::ROW && pl.consecutive && pl.tadLength >= Pack<T>::N && pl.tadLength < 0xffffffffLL &&
                       (((uintptr_t)x | (uintptr_t)z) & 15) == 0) {
                // gap-free rows whose length is not a multiple of the vector width
                const Long n = pl.numTads * pl.tadLength;
                ND4J_LAUNCH((bcFlatAnyKernel<T, F>), dim3(gridFor(n / Pack<T>::N + 1, kBlock, F::tables ? kGridCap : kMaxGrid)),
                                   dim3(kBlock), 0, s, x, y, z, n, pl.tadLength, Params<T>{nullptr});
            } else if (pl.wholeRun >= (unsigned)Pack<T>::N && runUnits<T>(1, pl.wholeN, pl.wholeRun) <= kMaxRunUnits) {
                // contiguous TADs with gaps whose places follow from x's own strides: the call is an element-wise walk over x,
                // y repeating along the dimensions that are not the TAD's; no offset tables (add a row to [65536, 1024] with
                // a pitch of 1032: 69.5 % of the HBM peak with two units per thread, 62 % with one or four, 66.5 % through
                // bcRowKernel; TADs over several dimensions are better off with their tables: 71 % against 64 %)
                launchRuns<T, F, false, 2>(s, x, pl.wx, y, pl.wy, z, pl.wz, nullptr, nullptr, Params<T>{nullptr}, 1, pl.wholeN,
                                           pl.wholeRun, false);
            } else if (pl.kind == BroadcastPlan::ROW) {
                constexpr int VEC = Pack<T>::N;
                Long vecsPerTad = (pl.tadLength + VEC - 1) / VEC;
                int colShift = 0;
                while ((1 << colShift) < kBlock && (1LL << colShift) < vecsPerTad) colShift++;
                const int colThreads = 1 << colShift, rowsPerBlock = kBlock >> colShift;
                Long gy = (vecsPerTad + colThreads - 1) / colThreads;
                if (gy > 65535) gy = 65535;
                // four passes per block (the y vector is loaded once per block) while that leaves >= 4096 blocks
                Long perBlock = (Long)rowsPerBlock * kBcRows;
                if ((pl.numTads / (perBlock * 4)) * gy >= 4096) perBlock *= 4;
                int gx = gridFor(pl.numTads, perBlock, kMaxGrid);
                int aligned = (((uintptr_t)x | (uintptr_t)z) & 15) == 0 ? 1 : 0;
                ND4J_LAUNCH((bcRowKernel<T, F, false>), dim3(gx, (unsigned)gy), dim3(kBlock), 0, s, x, y, z, pl.xOffsets,
                                   pl.zOffsets, pl.tadLength, pl.numTads, aligned, colShift, Params<T>{nullptr});
            } else if (pl.kind == BroadcastPlan::COL && pl.denseAlike && pl.tadEws >= 1 && pl.tadEws < 0xffffffffLL &&
                       pl.tadLength < 0xffffffffLL && (((uintptr_t)x | (uintptr_t)z) & 15) == 0) {
                // any single dimension of a dense array: runs of tadEws consecutive elements share one y
                const Long n = pl.numTads * pl.tadLength;
                ND4J_LAUNCH((bcFlatInnerKernel<T, F>), dim3(gridFor(n / Pack<T>::N + 1, kBlock, F::tables ? kGridCap : kMaxGrid)),
                                   dim3(kBlock), 0, s, x, y, z, n, pl.tadEws, pl.tadLength, Params<T>{nullptr});
            } else if (pl.kind == BroadcastPlan::COL) {
                int gx = (int)((pl.numTads + kBlock - 1) / kBlock);
                Long gy = (Long)kGridCap / gx;
                if (gy < 1) gy = 1;
                if (gy > pl.tadLength) gy = pl.tadLength;
                if (gy > 65535) gy = 65535;
                ND4J_LAUNCH((bcColKernel<T, F, false>), dim3(gx, (unsigned)gy), dim3(kBlock), 0, s, x, y, z, pl.xOffsets,
                                   pl.zOffsets, pl.tadLength, pl.numTads, pl.tadEws, pl.yEws, pl.zEws, Params<T>{nullptr});
            } else if (pl.slabInner >= (unsigned)Pack<T>::N && pl.slabInner % Pack<T>::N == 0 &&
                       (((uintptr_t)x | (uintptr_t)y | (uintptr_t)z) & 15) == 0) {
                // ([256, 1024, 256] floats along {0, 2}: 79.5 % of the HBM peak, 79.0 / 78.3 on blocks of 128 / 64 threads; 70.6 as
                // runs with offset tables)
                const Long nvec = pl.numTads * pl.tadLength / Pack<T>::N;  // (the host sends arrays of up to 2^31 - 1 elements here)
                ND4J_LAUNCH((bcFlatSlabKernel<T, F>), dim3(gridFor(nvec, kBlock * 2, F::tables ? kGridCap : kMaxGrid)), dim3(kBlock), 0,
                            s, x, y, z, (unsigned)nvec, FastDiv(pl.slabInner / Pack<T>::N), FastDiv(pl.slabMid), Params<T>{nullptr});
            } else if (pl.runLength > 0 && runUnits<T>(pl.numTads, pl.tadLength, pl.runLength) <= kMaxRunUnits) {
                // TADs over several dimensions whose innermost one is contiguous in x, y and z
                launchRuns<T, F, true>(s, x, pl.xm, y, pl.ym, z, pl.zm, pl.xOffsets, pl.zOffsets, Params<T>{nullptr}, pl.numTads,
                                 pl.tadLength, pl.runLength, pl.runMajor);
            } else if (pl.numTads >= 64) {
                // several dimensions, no contiguous runs: a lane per TAD, so that neighbouring TADs coalesce
                int gx = (int)((pl.numTads + kBlock - 1) / kBlock);
                Long gy = (Long)kGridCap / gx;
                if (gy < 1) gy = 1;
                if (gy > pl.tadLength) gy = pl.tadLength;
                if (gy > 65535) gy = 65535;
                ND4J_LAUNCH((bcColKernel<T, F, false, true>), dim3(gx, (unsigned)gy), dim3(kBlock), 0, s, x, y, z, pl.xOffsets,
                                   pl.zOffsets, pl.tadLength, pl.numTads, (Long)0, (Long)0, (Long)0, Params<T>{nullptr}, pl.xm, pl.ym,
                                   pl.zm);
            } else {
                int grid = gridFor(pl.numTads, 1, kGridCap);
                ND4J_LAUNCH((bcGeneralKernel<T, F>), dim3(grid), dim3(kBlock), 0, s, x, pl.xm, y, pl.ym, z, pl.zm,
                                   pl.xOffsets, pl.zOffsets, pl.tadLength, pl.numTads);
            }
            return true;
        }
    };
};

template <typename T>
bool launchBroadcast(hipStream_t s, int opNum, const T *x, const T *y, T *z, const BroadcastPlan &plan) {
    int kind = broadcastKind(opNum);
    if (kind == B_Invalid) return false;
    // only kinds that appear in the broadcast table are instantiated (B_Add .. B_TruncateDiv)
    return dispatchSeq<BroadcastBody<T>::template Run>(kind, std::make_integer_sequence<int, B_TruncateDiv + 1>{}, s, x, y,
                                                       z, plan);
}

#define INST(T) template bool launchBroadcast<T>(hipStream_t, int, const T *, const T *, T *, const BroadcastPlan &);
INST(float)
INST(float16)
INST(double)
#undef INST

}  // namespace nd4j_amd
