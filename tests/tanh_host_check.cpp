// The Tanh transform's polynomial for arguments below 1 (libnd4j_amd/csrc/tanh_poly.h), built for the host from the
// very lines the device compiles, against the C library's tanhf (what the reference's nd4j_tanh<float> calls:
// include/templatemath.h:847) and against double tanh rounded to float.
//   tanh_host_check <stride>     every stride-th float bit pattern in (0, 1), both signs; stride 1 = all of them
// Prints the histograms of ULP distances and exits 0 when none exceeds 2 (library) and 1 (correctly rounded).
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../libnd4j_amd/csrc/tanh_poly.h"

static int32_t bitsOf(float f) { int32_t i; std::memcpy(&i, &f, 4); return i; }

int main(int argc, char **argv) {
    const uint32_t stride = argc > 1 ? (uint32_t)std::strtoul(argv[1], nullptr, 10) : 61;
    long toLibrary[4] = {0, 0, 0, 0}, toExact[4] = {0, 0, 0, 0};
    bool odd = true;
    for (uint32_t b = 1; b < 0x3f800000u; b += stride) {
        float x;
        std::memcpy(&x, &b, 4);
        const float mine = nd4j_amd::tanhBelowOne(x), theirs = ::tanhf(x), exact = (float)::tanh((double)x);
        int dl = std::abs(bitsOf(mine) - bitsOf(theirs)), de = std::abs(bitsOf(mine) - bitsOf(exact));
        toLibrary[dl > 3 ? 3 : dl]++;
        toExact[de > 3 ? 3 : de]++;
        if (bitsOf(nd4j_amd::tanhBelowOne(-x)) != (int32_t)(bitsOf(mine) ^ 0x80000000)) odd = false;
    }
    const float nan = std::nanf("");
    const bool nanStays = std::isnan(nd4j_amd::tanhBelowOne(nan));
    const bool zeros = bitsOf(nd4j_amd::tanhBelowOne(0.0f)) == 0 && (uint32_t)bitsOf(nd4j_amd::tanhBelowOne(-0.0f)) == 0x80000000u;
    std::printf("ulp to tanhf: 0:%ld 1:%ld 2:%ld more:%ld\n", toLibrary[0], toLibrary[1], toLibrary[2], toLibrary[3]);
    std::printf("ulp to exact: 0:%ld 1:%ld 2:%ld more:%ld\n", toExact[0], toExact[1], toExact[2], toExact[3]);
    std::printf("odd:%d nan:%d zeros:%d\n", (int)odd, (int)nanStays, (int)zeros);
    const bool ok = toLibrary[3] == 0 && toExact[2] == 0 && toExact[3] == 0 && odd && nanStays && zeros;
    std::printf(ok ? "tanh host check: ok\n" : "tanh host check: FAILED\n");
    return ok ? 0 : 1;
}
