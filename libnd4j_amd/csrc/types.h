// Plain data types shared by host and device code.
//
// Nd4jPointer / Nd4jLong follow the reference's include/pointercast.h:9-11.  `float16` is the 2-byte
// storage struct of include/types/float16.h:201-205: entry points only ever receive pointers to it.
#pragma once

#include <cstdint>

#include "../../include/nd4j_types.h"

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>

namespace nd4j_amd {

// Storage <-> compute conversions.  fp16 follows the reference's software conversion
// (include/types/float16.h:102-195): IEEE round-to-nearest-even, and every NaN is stored as 0x7fff.
template <typename T> struct Compute;
template <> struct Compute<float> { typedef float type; };
template <> struct Compute<double> { typedef double type; };
template <> struct Compute<float16> { typedef float type; };

__device__ __forceinline__ float toCompute(float v) { return v; }
__device__ __forceinline__ double toCompute(double v) { return v; }
__device__ __forceinline__ float halfBitsToFloat(unsigned short b) {
    return (float)__builtin_bit_cast(_Float16, b);
}
__device__ __forceinline__ unsigned short floatToHalfBits(float f) {
    if (f != f) return (unsigned short)0x7fffu;
    return __builtin_bit_cast(unsigned short, (_Float16)f);
}
__device__ __forceinline__ float toCompute(float16 v) { return halfBitsToFloat(v.x); }

template <typename T> __device__ __forceinline__ T fromCompute(typename Compute<T>::type v);
template <> __device__ __forceinline__ float fromCompute<float>(float v) { return v; }
template <> __device__ __forceinline__ double fromCompute<double>(double v) { return v; }
template <> __device__ __forceinline__ float16 fromCompute<float16>(float v) {
    float16 h;
    h.x = floatToHalfBits(v);
    return h;
}

// extraParams is a device pointer in the caller's storage type; ops read it lazily through this view,
// so a null pointer is fine for ops that take no parameters.
template <typename T> struct Params {
    const T *p;
    // the scalar operand of the scalar family, handed over by value (unused elsewhere)
    typename Compute<T>::type scalar = 0;
    __device__ __forceinline__ typename Compute<T>::type operator[](int i) const { return toCompute(p[i]); }
    // the scalar as the storage type holds it (the reference converts it to T before the loop)
    __device__ __forceinline__ typename Compute<T>::type scalarValue() const { return toCompute(fromCompute<T>(scalar)); }
};

}  // namespace nd4j_amd
#endif
