// Plain argument types of the NativeOps boundary.
// Reference: include/pointercast.h:9-11 (Nd4jPointer, Nd4jLong) and include/types/float16.h:201-205
// (float16 is a 2-byte storage struct; entry points only ever take pointers to it).
#pragma once

#include <stdint.h>

typedef void *Nd4jPointer;
typedef long long Nd4jLong;
typedef int Nd4jStatus; /* include/pointercast.h:12 */

#ifdef __cplusplus
struct float16 {
    unsigned short x;
};
#else
typedef struct float16 {
    unsigned short x;
} float16;
#endif
