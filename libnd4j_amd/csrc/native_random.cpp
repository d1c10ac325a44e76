// NativeOps boundary, part 3: generator lifecycle and the random family.
// Reference: blas/cuda/NativeOps.cu:5312-5451 (entry points), include/loops/cpu/random.cpp:11-199 (branch
// selection and the rewind after every op), include/ops/special_random_ops.h (special ops, which only the
// (x, y, z) overload runs: cpu/random.cpp:15-18).
#include <cstring>
#include <stdexcept>

#include "../../include/NativeOps.h"
#include "rng.h"
#include "runtime.h"

using namespace nd4j_amd;

namespace {

// Fortran-order coordinate map of one operand (cpu/random.cpp:62-66 uses shape::ind2sub for x, y and z)
void fLinearMap(const Long *info, DimMap &out) {
    int rank = siRank(info);
    Long rs[kMaxRank], rt[kMaxRank];
    for (int i = 0; i < rank; i++) { rs[i] = siShape(info)[rank - 1 - i]; rt[i] = siStride(info)[rank - 1 - i]; }
    ownCanon(rank, rs, rt, out);
}

template <typename T>
void randomExec(Nd4jPointer *extra, int opNum, Nd4jPointer state, T *x, Long *xInfo, T *y, Long *yInfo, T *z, Long *zInfo,
                T *args, int operands) {
    hipStream_t s = streamOf(extra);
    RandomBuffer *rb = reinterpret_cast<RandomBuffer *>(state);
    if (rb == nullptr) return;
    std::vector<Long> sx, sy, sz;
    // The reference's device code decodes the shapeInfos itself and keeps the generator's position on the device, so
    // its host side needs none of them; here the host advances the generator and sizes the launch.  nd4j passes the
    // host copy of z's shapeInfo in extraPointers[0] on these calls: it is used when it is there and looks like one.
    // Operands that share one shapeInfo buffer (x == z in place, x = y = z for the distributions) are read once.
    const Long *hz = nullptr;
    if (const Long *h0 = reinterpret_cast<const Long *>(slotOf(extra, X_HOST_X_SHAPE))) {
        if (!isDeviceMemory(h0) && h0[0] >= 1 && h0[0] <= kMaxRank && (siOrder(h0) == 'c' || siOrder(h0) == 'f')) hz = h0;
    }
    if (hz == nullptr) hz = hostShapeInfo(nullptr, 0, zInfo, sz, s);
    const Long *hx = operands >= 2 ? (xInfo == zInfo ? hz : hostShapeInfo(nullptr, 0, xInfo, sx, s)) : nullptr;
    const Long *hy = operands >= 3 ? (yInfo == zInfo ? hz : (yInfo == xInfo ? hx : hostShapeInfo(nullptr, 0, yInfo, sy, s))) : nullptr;
    if (hz == nullptr || (operands >= 2 && hx == nullptr) || (operands >= 3 && hy == nullptr)) return;

    RandomPlan pl;
    pl.n = siNumel(hz);
    pl.xEws = hx ? siEws(hx) : 1;
    pl.yEws = hy ? siEws(hy) : 1;
    pl.zEws = siEws(hz);
    pl.yLength = hy ? siNumel(hy) : 0;
    pl.xm.rank = pl.ym.rank = pl.zm.rank = 0;
    pl.strided = pl.xEws >= 1 && pl.yEws >= 1 && pl.zEws >= 1;
    const bool special = opNum == 5 || opNum == 6 || (opNum >= 8 && opNum <= 11);
    if (!pl.strided) {
        if (special && operands == 3 && opNum != 5) {
            // Gaussian / Binomial / TruncatedNormal / LogNormal address y and z through their EWS only
            printf("[ERROR] random op %d needs element-wise strides on y and z\n", opNum);
            return;
        }
        if (opNum == 5 && operands == 3 && pl.n > pl.yLength) {
            // Without element-wise strides the reference's Choice indexes the probabilities with the RESULT's index
            // (special_random_ops.h:214): defined (and followed here) while there are no more results than
            // probabilities, a read beyond the probabilities otherwise - which a device must not replay
            throw std::invalid_argument("Choice without element-wise strides needs length(z) <= length(y): the reference "
                                        "reads outside the probabilities there");
        }
        fLinearMap(hz, pl.zm);
        if (hx) fLinearMap(hx, pl.xm);
        if (hy) fLinearMap(hy, pl.ym);
    }
    if (!launchRandom<T>(s, opNum, rb->deviceState(), x, y, z, args, pl, operands, y == z)) {
        reportUnknownOp("random", opNum);
        return;
    }
    checkLaunch("execRandom", s);
    // update rng state (cpu/random.cpp:79,136,183; Binomial rewinds length * trials and only when
    // trials > 0: special_random_ops.h:514-516)
    if (special && operands == 3 && (opNum == 8 || opNum == 9)) {
        T a0;
        std::memset(&a0, 0, sizeof(T));
        if (isDeviceMemory(args)) {
            (void)hipMemcpyAsync(&a0, args, sizeof(T), hipMemcpyDeviceToHost, s);
            syncAndCheck("execRandom(binomial trials)", s);
        } else {
            a0 = args[0];
        }
        double tv;
        if (sizeof(T) == 2) {
            unsigned short h;
            std::memcpy(&h, &a0, 2);
            // small integers only: decode the half by hand
            unsigned e = (h >> 10) & 0x1f, mnt = h & 0x3ff;
            tv = e == 0 ? mnt * 5.9604644775390625e-08 : (1024 + mnt) * (e >= 25 ? (double)(1u << (e - 25)) : 1.0 / (double)(1u << (25 - e)));
            if (h & 0x8000) tv = -tv;
        } else if (sizeof(T) == 4) {
            float f;
            std::memcpy(&f, &a0, 4);
            tv = f;
        } else {
            std::memcpy(&tv, &a0, 8);
        }
        int trials = (int)tv;
        if (trials > 0) rb->rewind(pl.n * trials);
    } else {
        rb->rewind(pl.n);
    }
}

}  // namespace

#define ND4J_RANDOM_MEMBERS(SUFFIX, T)                                                                             \
    void NativeOps::execRandom##SUFFIX(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *z,             \
                                       Nd4jLong *zShapeBuffer, T *extraArguments) {                                \
        randomExec<T>(extraPointers, opNum, state, nullptr, nullptr, nullptr, nullptr, z, zShapeBuffer,            \
                      extraArguments, 1);                                                                          \
    }                                                                                                              \
    void NativeOps::execRandom##SUFFIX(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *x,             \
                                       Nd4jLong *xShapeBuffer, T *y, Nd4jLong *yShapeBuffer, T *z,                 \
                                       Nd4jLong *zShapeBuffer, T *extraArguments) {                                \
        randomExec<T>(extraPointers, opNum, state, x, xShapeBuffer, y, yShapeBuffer, z, zShapeBuffer,              \
                      extraArguments, 3);                                                                          \
    }                                                                                                              \
    void NativeOps::execRandom##SUFFIX(Nd4jPointer *extraPointers, int opNum, Nd4jPointer state, T *x,             \
                                       Nd4jLong *xShapeBuffer, T *z, Nd4jLong *zShapeBuffer, T *extraArguments) {  \
        randomExec<T>(extraPointers, opNum, state, x, xShapeBuffer, nullptr, nullptr, z, zShapeBuffer,             \
                      extraArguments, 2);                                                                          \
    }

ND4J_RANDOM_MEMBERS(Float, float)
ND4J_RANDOM_MEMBERS(Half, float16)
ND4J_RANDOM_MEMBERS(Double, double)

// extraPointers[0] = host buffer of bufferSize u64 words, ptrToBuffer = device buffer of the same size
// (blas/cuda/NativeOps.cu:5384-5407).  The sequence is generated on the host and copied over on the stream.
Nd4jPointer NativeOps::initRandom(Nd4jPointer *extraPointers, long seed, long bufferSize, Nd4jPointer ptrToBuffer) {
    hipStream_t s = streamOf(extraPointers);
    RandomBuffer *rb = new RandomBuffer();
    rb->size = bufferSize;
    rb->devBuffer = reinterpret_cast<uint64_t *>(ptrToBuffer);
    rb->hostBuffer = reinterpret_cast<uint64_t *>(slotOf(extraPointers, 0));
    if (rb->hostBuffer == nullptr) {
        rb->hostBuffer = new uint64_t[bufferSize > 0 ? bufferSize : 1];
        rb->ownsHostBuffer = true;
    }
    rb->seed = seed;
    rb->amplifier = seed;
    rb->generation = 1;
    rb->currentPosition = 0;
    rb->fillHost();
    hipError_t e = hipMemcpyAsync(rb->devBuffer, rb->hostBuffer, (size_t)bufferSize * 8, hipMemcpyHostToDevice, s);
    if (e != hipSuccess) {
        if (rb->ownsHostBuffer) delete[] rb->hostBuffer;
        delete rb;
        throw std::runtime_error(std::string("initRandom: ") + hipGetErrorString(e));
    }
    // the host buffer may be pageable: make sure the copy has consumed it before returning
    syncAndCheck("initRandom", s);
    return rb;
}

void NativeOps::refreshBuffer(Nd4jPointer *extraPointers, long seed, Nd4jPointer ptrRandom) {
    hipStream_t s = streamOf(extraPointers);
    RandomBuffer *rb = reinterpret_cast<RandomBuffer *>(ptrRandom);
    // kernels of earlier ops may still read the device buffer
    syncAndCheck("refreshBuffer", s);
    rb->setSeed(seed);
    rb->currentPosition = 0;
    rb->fillHost();
    hipError_t e = hipMemcpyAsync(rb->devBuffer, rb->hostBuffer, (size_t)rb->size * 8, hipMemcpyHostToDevice, s);
    if (e != hipSuccess) throw std::runtime_error(std::string("refreshBuffer: ") + hipGetErrorString(e));
    syncAndCheck("refreshBuffer", s);
}

void NativeOps::reSeedBuffer(Nd4jPointer *, long seed, Nd4jPointer ptrRandom) {
    // CPU semantics (blas/cpu/NativeOps.cpp:2896-2900): only the amplifier changes.  The reference's CUDA
    // back end additionally resets the offset (blas/cuda/NativeOps.cu:5439-5450); parity is checked
    // against the CPU stream, so the offset is kept.
    RandomBuffer *rb = reinterpret_cast<RandomBuffer *>(ptrRandom);
    rb->amplifier = seed;
}

void NativeOps::destroyRandom(Nd4jPointer ptrRandom) {
    RandomBuffer *rb = reinterpret_cast<RandomBuffer *>(ptrRandom);
    if (rb == nullptr) return;
    (void)hipDeviceSynchronize();  // as the reference does: the streams that used the generator are unknown here
    if (rb->ownsHostBuffer) delete[] rb->hostBuffer;
    delete rb;
}
