// The Log transform's routine (libnd4j_amd/csrc/log_poly.h), built for the host from the very lines the device compiles,
// against the C library's logf (what the reference's nd4j_log<float> calls: include/templatemath.h) and against double
// log rounded to float.
//   log_host_check <stride>     every stride-th positive float bit pattern up to infinity; stride 1 = all of them
// Prints the histograms of ULP distances and exits 0 when none exceeds 1, and zero, negative, infinite and NaN arguments
// give what logf gives.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../libnd4j_amd/csrc/log_poly.h"

static int32_t bitsOf(float f) { int32_t i; std::memcpy(&i, &f, 4); return i; }

int main(int argc, char **argv) {
    const uint32_t stride = argc > 1 ? (uint32_t)std::strtoul(argv[1], nullptr, 10) : 127;
    long toLibrary[3] = {0, 0, 0}, toExact[3] = {0, 0, 0};
    for (uint32_t b = 1; b < 0x7f800000u; b += stride) {
        float x;
        std::memcpy(&x, &b, 4);
        const float mine = nd4j_amd::logNear(x), theirs = ::logf(x), exact = (float)::log((double)x);
        const bool sameSign = ((bitsOf(mine) ^ bitsOf(theirs)) >> 31) == 0 || (mine == 0.0f && theirs == 0.0f);
        int dl = sameSign ? std::abs(bitsOf(mine) - bitsOf(theirs)) : 2, de = std::abs(bitsOf(mine) - bitsOf(exact));
        toLibrary[dl > 2 ? 2 : dl]++;
        toExact[de > 2 ? 2 : de]++;
    }
    const float inf = __builtin_inff();
    const bool specials = nd4j_amd::logNear(0.0f) == -inf && nd4j_amd::logNear(-0.0f) == -inf && nd4j_amd::logNear(inf) == inf &&
                          std::isnan(nd4j_amd::logNear(-1.0f)) && std::isnan(nd4j_amd::logNear(-inf)) &&
                          std::isnan(nd4j_amd::logNear(std::nanf(""))) && bitsOf(nd4j_amd::logNear(1.0f)) == 0;
    std::printf("ulp to logf:  0:%ld 1:%ld more:%ld\n", toLibrary[0], toLibrary[1], toLibrary[2]);
    std::printf("ulp to exact: 0:%ld 1:%ld more:%ld\n", toExact[0], toExact[1], toExact[2]);
    std::printf("specials:%d\n", (int)specials);
    const bool ok = toLibrary[2] == 0 && toExact[2] == 0 && specials;
    std::printf(ok ? "log host check: ok\n" : "log host check: FAILED\n");
    return ok ? 0 : 1;
}
