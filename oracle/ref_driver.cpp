// TEST INFRASTRUCTURE ONLY.
//
// C-ABI driver around the reference's own CPU loop templates (functions::*), compiled against the
// reference headers where they lie (never copied).  It is linked with the reference's loop
// translation units into oracle/_ref/libnd4j_ref.so by oracle/Makefile.  The exported names and
// signatures are identical to those of oracle/nd4j_oracle.cpp (the restatement), so a test can
// load either library behind the same ctypes wrapper.
//
// Entry points follow what blas/cpu/NativeOps.cpp does for the same call: e.g. execReduceFloat
// (NativeOps.cpp:952-973) forwards to NativeOpExcutioner::execReduce (NativeOpExcutioner.cpp:122-128),
// which runs a Max pass first for opNum 19 and then ReduceFunction<T>::exec.

#include <cstdint>
#include <cstring>
#include <omp.h>
#include <pointercast.h>
#include <types/float16.h>
#include <Environment.h>
#include <helpers/shape.h>
#include <helpers/TAD.h>
#include <loops/transform.h>
#include <loops/pairwise_transform.h>
#include <loops/broadcasting.h>
#include <loops/reduce.h>
#include <loops/indexreduce.h>
#include <loops/summarystatsreduce.h>
#include <loops/random.h>
#include <loops/reduce3.h>
#include <loops/scalar.h>

using functions::transform::Transform;
using functions::pairwise_transforms::PairWiseTransform;
using functions::broadcast::Broadcast;
using functions::reduce::ReduceFunction;
using functions::indexreduce::IndexReduce;
using functions::summarystats::SummaryStatsReduce;
using functions::random::RandomFunction;
using functions::scalar::ScalarTransform;
using functions::reduce3::Reduce3;

// Data-movement specials.  flatten / pullRows / tear / shuffle are function templates defined and explicitly
// instantiated in blas/cpu/NativeOps.cpp (1529-1664, 2044-2160, 2265-2325, instantiations 3574-3588); that file is
// compiled where it lies with hidden visibility and per-function sections, and the link drops everything these
// wrappers do not reach.  concat is nd4j::SpecialMethods<T>::concatCpuGeneric of include/ops/impl/specials.cpp,
// the conversions go through NativeOps::convertTypes itself (include/loops/type_conversions.h:696-850, a
// host loop in both of the reference's back ends).
#include <ops/specials.h>
template <typename T>
void flattenGeneric(Nd4jPointer *extraPointers, int offset, char order, T *result, Nd4jLong *resultShapeInfo, T *input,
                    Nd4jLong *inputShapeInfo);
template <typename T>
void pullRowsGeneric(T *x, Nd4jLong *xShapeInfo, T *z, Nd4jLong *zShapeInfo, const int n, Nd4jLong *indexes,
                     Nd4jLong *tadShapeInfo, Nd4jLong *tadOffsets, Nd4jLong *zTadShapeInfo, Nd4jLong *zTadOffsets);
template <typename T>
void tearGeneric(T *x, Nd4jLong *xShapeInfo, Nd4jPointer *targets, Nd4jLong *zShapeInfo, Nd4jLong *tadShapeInfo,
                 Nd4jLong *tadOffsets);
template <typename T>
void shuffleGeneric(T **dX, Nd4jLong **xShapeInfo, T **dZ, Nd4jLong **zShapeInfo, int N, int *shuffleMap,
                    Nd4jLong **tadOnlyShapeInfo, Nd4jLong **tadOffsets);
#include <NativeOps.h>

namespace {

template <typename T>
void reduceWithPrepass(int opNum, T *x, Nd4jLong *xSI, T *extra, T *z, Nd4jLong *zSI, int *dim, int dimLen) {
    if (opNum == 19)
        ReduceFunction<T>::exec(3, x, xSI, extra, z, zSI, dim, dimLen, nullptr, nullptr);
    ReduceFunction<T>::exec(opNum, x, xSI, extra, z, zSI, dim, dimLen, nullptr, nullptr);
}

template <typename T>
T reduceScalarWithPrepass(int opNum, T *x, Nd4jLong *xSI, T *extra) {
    if (opNum == 19) {
        T mx = ReduceFunction<T>::execScalar(3, x, xSI, extra);
        return ReduceFunction<T>::execScalar(opNum, x, xSI, &mx);
    }
    return ReduceFunction<T>::execScalar(opNum, x, xSI, extra);
}

}  // namespace

// per-TAD scalars: the caller of ScalarTransform::transform supplies the TAD tables (blas/cpu/NativeOps.cpp:2453-2481)
template <typename T>
void scalarAlongDimension(int opNum, T *x, Nd4jLong *xSI, T *z, Nd4jLong *zSI, T *scalars, T *extra, int *dim, int dimLen) {
    shape::TAD tad;
    tad.init(xSI, dim, dimLen);
    tad.createTadOnlyShapeInfo();
    tad.createOffsets();
    ScalarTransform<T>::transform(opNum, x, xSI, extra, z, zSI, scalars, dim, dimLen, tad.tadOnlyShapeInfo, tad.tadOffsets,
                                  nullptr, nullptr);
}

// reduce3 with the caller's TAD tables ("going tad-way", blas/cpu/NativeOps.cpp:1100-1108) and all pairs of TADs
// (1144-1161): the tables are built here with the reference's own shape::TAD
template <typename T>
void reduce3TadWay(int opNum, T *x, Nd4jLong *xSI, T *extra, T *y, Nd4jLong *ySI, T *z, Nd4jLong *zSI, int *dim, int dimLen) {
    shape::TAD tad;
    tad.init(xSI, dim, dimLen);
    tad.createTadOnlyShapeInfo();
    tad.createOffsets();
    Reduce3<T>::exec(opNum, x, xSI, extra, y, ySI, z, zSI, dim, dimLen, tad.tadOnlyShapeInfo, tad.tadOffsets);
}
template <typename T>
void reduce3AllPairs(int opNum, T *x, Nd4jLong *xSI, T *extra, T *y, Nd4jLong *ySI, T *z, Nd4jLong *zSI, int *dim, int dimLen) {
    shape::TAD tx, ty;
    tx.init(xSI, dim, dimLen);
    tx.createTadOnlyShapeInfo();
    tx.createOffsets();
    ty.init(ySI, dim, dimLen);
    ty.createTadOnlyShapeInfo();
    ty.createOffsets();
    Reduce3<T>::execAll(opNum, x, xSI, extra, y, ySI, z, zSI, dim, dimLen, tx.tadOnlyShapeInfo, tx.tadOffsets,
                        ty.tadOnlyShapeInfo, ty.tadOffsets);
}

#define ND4J_CPU_FAMILY(SUF, T)                                                                              \
    void nd4j_cpu_reduce3_scalar_##SUF(int op, void *x, Nd4jLong *xSI, void *extra, void *y, Nd4jLong *ySI,  \
                                       void *out) {                                                          \
        *(T *)out = Reduce3<T>::execScalar(op, (T *)x, xSI, (T *)extra, (T *)y, ySI);                       \
    }                                                                                                        \
    void nd4j_cpu_reduce3_##SUF(int op, void *x, Nd4jLong *xSI, void *extra, void *y, Nd4jLong *ySI,         \
                                void *z, Nd4jLong *zSI, int *dim, int dimLen) {                              \
        Reduce3<T>::exec(op, (T *)x, xSI, (T *)extra, (T *)y, ySI, (T *)z, zSI, dim, dimLen);               \
    }                                                                                                        \
    void nd4j_cpu_reduce3_tad_##SUF(int op, void *x, Nd4jLong *xSI, void *extra, void *y, Nd4jLong *ySI,     \
                                    void *z, Nd4jLong *zSI, int *dim, int dimLen) {                          \
        reduce3TadWay<T>(op, (T *)x, xSI, (T *)extra, (T *)y, ySI, (T *)z, zSI, dim, dimLen);               \
    }                                                                                                        \
    void nd4j_cpu_reduce3_all_##SUF(int op, void *x, Nd4jLong *xSI, void *extra, void *y, Nd4jLong *ySI,     \
                                    void *z, Nd4jLong *zSI, int *dim, int dimLen) {                          \
        reduce3AllPairs<T>(op, (T *)x, xSI, (T *)extra, (T *)y, ySI, (T *)z, zSI, dim, dimLen);             \
    }                                                                                                        \
    void nd4j_cpu_scalar_##SUF(int op, void *x, Nd4jLong *xSI, void *z, Nd4jLong *zSI, double scalar,        \
                               void *extra) {                                                                \
        ScalarTransform<T>::transform(op, (T *)x, xSI, (T *)z, zSI, sizeof(T) < 8 ? (T)(float)scalar : (T)scalar, \
                                      (T *)extra);                                                           \
    }                                                                                                        \
    void nd4j_cpu_scalar_strided_##SUF(int op, void *x, Nd4jLong xs, void *z, Nd4jLong zs, double scalar,    \
                                       void *extra, Nd4jLong n) {                                            \
        ScalarTransform<T>::transform(op, (T *)x, xs, (T *)z, zs, sizeof(T) < 8 ? (T)(float)scalar : (T)scalar, \
                                      (T *)extra, n);                                                        \
    }                                                                                                        \
    void nd4j_cpu_scalar_tad_##SUF(int op, void *x, Nd4jLong *xSI, void *z, Nd4jLong *zSI, void *scalars,    \
                                   void *extra, int *dim, int dimLen) {                                      \
        scalarAlongDimension<T>(op, (T *)x, xSI, (T *)z, zSI, (T *)scalars, (T *)extra, dim, dimLen);        \
    }                                                                                                        \
    void nd4j_cpu_transform_##SUF(int op, void *x, Nd4jLong *xSI, void *z, Nd4jLong *zSI, void *extra) {     \
        Transform<T>::exec(op, (T *)x, xSI, (T *)z, zSI, (T *)extra, nullptr, nullptr);                     \
    }                                                                                                        \
    void nd4j_cpu_transform_strided_##SUF(int op, void *x, Nd4jLong xs, void *z, Nd4jLong zs, void *extra,   \
                                          Nd4jLong n) {                                                      \
        Transform<T>::exec(op, (T *)x, xs, (T *)z, zs, (T *)extra, n);                                      \
    }                                                                                                        \
    void nd4j_cpu_pairwise_##SUF(int op, void *x, Nd4jLong *xSI, void *y, Nd4jLong *ySI, void *z,            \
                                 Nd4jLong *zSI, void *extra) {                                               \
        PairWiseTransform<T>::exec(op, (T *)x, xSI, (T *)y, ySI, (T *)z, zSI, (T *)extra);                  \
    }                                                                                                        \
    void nd4j_cpu_pairwise_strided_##SUF(int op, void *x, Nd4jLong xs, void *y, Nd4jLong ys, void *z,        \
                                         Nd4jLong zs, void *extra, Nd4jLong n) {                             \
        PairWiseTransform<T>::exec(op, (T *)x, xs, (T *)y, ys, (T *)z, zs, (T *)extra, n);                  \
    }                                                                                                        \
    void nd4j_cpu_broadcast_##SUF(int op, void *x, Nd4jLong *xSI, void *y, Nd4jLong *ySI, void *z,           \
                                  Nd4jLong *zSI, int *dim, int dimLen) {                                     \
        Broadcast<T>::exec(op, (T *)x, xSI, (T *)y, ySI, (T *)z, zSI, dim, dimLen, nullptr, nullptr,        \
                           nullptr, nullptr);                                                                \
    }                                                                                                        \
    void nd4j_cpu_reduce_##SUF(int op, void *x, Nd4jLong *xSI, void *extra, void *z, Nd4jLong *zSI,          \
                               int *dim, int dimLen) {                                                       \
        reduceWithPrepass<T>(op, (T *)x, xSI, (T *)extra, (T *)z, zSI, dim, dimLen);                        \
    }                                                                                                        \
    void nd4j_cpu_reduce_scalar_##SUF(int op, void *x, Nd4jLong *xSI, void *extra, void *out) {              \
        *(T *)out = reduceScalarWithPrepass<T>(op, (T *)x, xSI, (T *)extra);                                \
    }                                                                                                        \
    void nd4j_cpu_indexreduce_##SUF(int op, void *x, Nd4jLong *xSI, void *extra, void *z, Nd4jLong *zSI,     \
                                    int *dim, int dimLen) {                                                  \
        IndexReduce<T>::exec(op, (T *)x, xSI, (T *)extra, (T *)z, zSI, dim, dimLen, nullptr, nullptr);      \
    }                                                                                                        \
    void nd4j_cpu_indexreduce_scalar_##SUF(int op, void *x, Nd4jLong *xSI, void *extra, void *out) {         \
        *(T *)out = IndexReduce<T>::execScalar(op, (T *)x, xSI, (T *)extra);                                \
    }                                                                                                        \
    void nd4j_cpu_summarystats_##SUF(int op, int biasCorrected, void *x, Nd4jLong *xSI, void *extra,         \
                                     void *z, Nd4jLong *zSI, int *dim, int dimLen) {                         \
        SummaryStatsReduce<T>::exec(op, biasCorrected != 0, (T *)x, xSI, (T *)extra, (T *)z, zSI, dim,      \
                                    dimLen);                                                                 \
    }                                                                                                        \
    void nd4j_cpu_summarystats_scalar_##SUF(int op, int biasCorrected, void *x, Nd4jLong *xSI, void *extra,  \
                                            void *out) {                                                     \
        *(T *)out = SummaryStatsReduce<T>::execScalar(op, biasCorrected != 0, (T *)x, xSI, (T *)extra);     \
    }                                                                                                        \
    void nd4j_cpu_random_z_##SUF(int op, void *state, void *z, Nd4jLong *zSI, void *args) {                  \
        RandomFunction<T>::execTransform(op, state, (T *)z, zSI, (T *)args);                                \
    }                                                                                                        \
    void nd4j_cpu_random_xz_##SUF(int op, void *state, void *x, Nd4jLong *xSI, void *z, Nd4jLong *zSI,       \
                                  void *args) {                                                              \
        RandomFunction<T>::execTransform(op, state, (T *)x, xSI, (T *)z, zSI, (T *)args);                   \
    }                                                                                                        \
    void nd4j_cpu_random_xyz_##SUF(int op, void *state, void *x, Nd4jLong *xSI, void *y, Nd4jLong *ySI,      \
                                   void *z, Nd4jLong *zSI, void *args) {                                     \
        RandomFunction<T>::execTransform(op, state, (T *)x, xSI, (T *)y, ySI, (T *)z, zSI, (T *)args);      \
    }

#define ND4J_CPU_SPECIALS(SUF, T)                                                                                  \
    void nd4j_cpu_flatten_##SUF(int offset, int order, void *z, Nd4jLong *zSI, void *x, Nd4jLong *xSI) {           \
        flattenGeneric<T>(nullptr, offset, (char)order, (T *)z, zSI, (T *)x, xSI);                                 \
    }                                                                                                              \
    void nd4j_cpu_concat_##SUF(int dim, int n, void **data, Nd4jLong **infos, void *z, Nd4jLong *zSI) {            \
        nd4j::SpecialMethods<T>::concatCpuGeneric(dim, n, data, (Nd4jPointer *)infos, (T *)z, zSI);                \
    }                                                                                                              \
    void nd4j_cpu_pullrows_##SUF(void *x, Nd4jLong *xSI, void *z, Nd4jLong *zSI, long long n, Nd4jLong *idx,       \
                                 Nd4jLong *tadSI, Nd4jLong *tadOff, Nd4jLong *zTadSI, Nd4jLong *zTadOff) {         \
        pullRowsGeneric<T>((T *)x, xSI, (T *)z, zSI, (int)n, idx, tadSI, tadOff, zTadSI, zTadOff);                 \
    }                                                                                                              \
    void nd4j_cpu_tear_##SUF(void *x, Nd4jLong *xSI, void **targets, Nd4jLong *zSI, Nd4jLong *tadSI,               \
                             Nd4jLong *tadOff) {                                                                   \
        tearGeneric<T>((T *)x, xSI, targets, zSI, tadSI, tadOff);                                                  \
    }                                                                                                              \
    void nd4j_cpu_shuffle_##SUF(void **x, Nd4jLong **xSI, int N, int *map, Nd4jLong **tadSI, Nd4jLong **tadOff) {  \
        shuffleGeneric<T>((T **)x, xSI, (T **)x, xSI, N, map, tadSI, tadOff);                                      \
    }                                                                                                              \
    /* the CPU loops of specials.cpp: average adds x[k] / n term by term; accumulate adds into z, which is zeroed  \
       here first so that the result is the plain sum the device kernel of the same name produces */               \
    void nd4j_cpu_average_##SUF(void **x, void *z, int n, long long length, int propagate) {                       \
        nd4j::SpecialMethods<T>::averageGeneric((T **)x, (T *)z, n, length, propagate != 0);                       \
    }                                                                                                              \
    void nd4j_cpu_accumulate_##SUF(void **x, void *z, int n, long long length) {                                   \
        std::memset(z, 0, (size_t)length * sizeof(T));                                                             \
        nd4j::SpecialMethods<T>::accumulateGeneric((T **)x, (T *)z, n, length);                                    \
    }

extern "C" {

const char *nd4j_cpu_kind() { return "reference"; }

ND4J_CPU_SPECIALS(f32, float)
ND4J_CPU_SPECIALS(f16, float16)
ND4J_CPU_SPECIALS(f64, double)

int nd4j_cpu_convert(int srcType, void *x, long long n, int dstType, void *z) {
    const bool known = (srcType == 3 || srcType == 6 || srcType == 7) && (dstType == 3 || dstType == 6 || dstType == 7);
    if (!known || srcType == dstType) return 0;
    NativeOps ops;
    ops.convertTypes(nullptr, srcType, x, n, dstType, z);
    return 1;
}

ND4J_CPU_FAMILY(f32, float)
ND4J_CPU_FAMILY(f16, float16)
ND4J_CPU_FAMILY(f64, double)

// ---- RNG lifecycle: blas/cpu/NativeOps.cpp:2877-2906 ------------------------------------------------
void *nd4j_cpu_rng_init(long long seed, long long size, uint64_t *buffer) {
    auto rb = new nd4j::random::RandomBuffer(seed, size, buffer);
    nd4j::random::Xoroshiro128 gen(rb);
    gen.refreshBuffer();
    return rb;
}
void nd4j_cpu_rng_refresh(void *state, long long seed) {
    auto rb = reinterpret_cast<nd4j::random::RandomBuffer *>(state);
    rb->setSeed(seed);
    rb->setOffset(0);
    nd4j::random::Xoroshiro128 gen(rb);
    gen.refreshBuffer();
}
void nd4j_cpu_rng_reseed(void *state, long long seed) {
    reinterpret_cast<nd4j::random::RandomBuffer *>(state)->reSeed(seed);
}
void nd4j_cpu_rng_destroy(void *state) { delete reinterpret_cast<nd4j::random::RandomBuffer *>(state); }
void nd4j_cpu_rng_rewind(void *state, long long n) {
    reinterpret_cast<nd4j::random::RandomBuffer *>(state)->rewindH(n);
}
void nd4j_cpu_rng_set_offset(void *state, long long off) {
    reinterpret_cast<nd4j::random::RandomBuffer *>(state)->setOffset(off);
}
// out[0..4] = size, offset (currentPosition), seed, generation, amplifier.  The last two are private in
// the reference class, so they are read at their x86-64 layout positions (8-byte fields 7 and 9).
void nd4j_cpu_rng_state(void *state, long long *out) {
    auto rb = reinterpret_cast<nd4j::random::RandomBuffer *>(state);
    auto raw = reinterpret_cast<long long *>(state);
    out[0] = rb->getSize();
    out[1] = rb->getOffset();
    out[2] = rb->getSeed();
    out[3] = raw[7];
    out[4] = raw[9];
}
int nd4j_cpu_rng_sizeof() { return (int)sizeof(nd4j::random::RandomBuffer); }
void nd4j_cpu_rng_elements(void *state, long long start, long long n, uint64_t *out) {
    auto rb = reinterpret_cast<nd4j::random::RandomBuffer *>(state);
    for (long long i = 0; i < n; i++) out[i] = rb->relativeUInt(start + i);
}
void nd4j_cpu_rng_uniform_f32(void *state, long long start, long long n, float *out) {
    auto rb = reinterpret_cast<nd4j::random::RandomBuffer *>(state);
    for (long long i = 0; i < n; i++) out[i] = rb->relativeT<float>(start + i);
}

// ---- shape / TAD helpers --------------------------------------------------------------------------
// blas/cpu/NativeOps.cpp:2022-2032; returns the number of TADs.  target needs 2*rank+4 longs.
long long nd4j_cpu_tad_only_shape_info(Nd4jLong *xSI, int *dim, int dimLen, Nd4jLong *target, Nd4jLong *offsets) {
    shape::TAD tad;
    tad.init(xSI, dim, dimLen);
    tad.createTadOnlyShapeInfo();
    tad.createOffsets();
    std::memcpy(target, tad.tadOnlyShapeInfo, shape::shapeInfoByteLength(tad.tadOnlyShapeInfo));
    if (offsets != nullptr) std::memcpy(offsets, tad.tadOffsets, tad.numTads * sizeof(Nd4jLong));
    return tad.numTads;
}
long long nd4j_cpu_tad_count(Nd4jLong *xSI, int *dim, int dimLen) {
    shape::TAD tad;
    tad.init(xSI, dim, dimLen);
    return tad.numTads;
}
// shape::shapeBuffer / shape::shapeBufferFortran (shape.h:1640-1710)
void nd4j_cpu_shape_buffer(int rank, Nd4jLong *shp, int order, Nd4jLong *out) {
    if (order == 'f')
        shape::shapeBufferFortran(rank, shp, out);
    else
        shape::shapeBuffer(rank, shp, out);
}
int nd4j_cpu_compute_ews(int rank, Nd4jLong *shp, Nd4jLong *stride, int isFOrder) {
    return shape::computeElementWiseStride(rank, shp, stride, isFOrder);
}
int nd4j_cpu_get_order(int rank, Nd4jLong *shp, Nd4jLong *stride, int elementStride) {
    return shape::getOrder(rank, shp, stride, elementStride);
}
void nd4j_cpu_ind2sub(int order, int rank, Nd4jLong *shp, long long index, Nd4jLong *out) {
    if (order == 'c')
        shape::ind2subC(rank, shp, (int)index, out);
    else
        shape::ind2sub(rank, shp, (int)index, out);
}

// ---- environment ----------------------------------------------------------------------------------
void nd4j_cpu_set_thresholds(int elementThreshold, int tadThreshold) {
    nd4j::Environment::getInstance()->setElementwiseThreshold(elementThreshold);
    nd4j::Environment::getInstance()->setTadThreshold(tadThreshold);
}
void nd4j_cpu_set_threads(int n) { omp_set_num_threads(n); }
int nd4j_cpu_get_threads() { return omp_get_max_threads(); }

}  // extern "C"
