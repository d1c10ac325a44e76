// Host-side generator state behind initRandom / execRandom*.
//
// Field meaning follows nd4j::random::RandomBuffer (reference: include/helpers/helper_generator.h:61-74):
// a buffer of `size` 64-bit words filled by xoroshiro128+ seeded through splitmix64
// (Xoroshiro128::refreshBuffer, 612-621), plus (currentPosition, generation, amplifier) that getElement
// (185-220) folds into every draw.  The state lives on the host and is handed to kernels by value; after
// an op the host applies rewindH(length) (322-334), so ops on one generator are ordered by the caller
// exactly as on the reference (one op at a time per generator).
#pragma once

#include <cstdint>

#include "launch.h"

namespace nd4j_amd {

struct RandomBuffer {
    Long size = 0;
    uint64_t *hostBuffer = nullptr;
    uint64_t *devBuffer = nullptr;
    bool ownsHostBuffer = false;
    Long seed = 0;
    Long generation = 1;
    Long currentPosition = 0;
    Long amplifier = 0;

    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    // splitmix64 finaliser (helper_generator.h:569-575)
    static uint64_t seedConv(Long s) {
        uint64_t x = (uint64_t)s;
        uint64_t z = (x += 0x9E3779B97F4A7C15ULL);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
        return z ^ (z >> 31);
    }
    // xoroshiro128+ stream with the reference's seeding: s0 = seedConv(seed), s1 = seedConv(seed*119+3)
    void fillHost() {
        uint64_t s0 = seedConv(seed);
        uint64_t s1 = seedConv(seed * 119 + 3);
        for (Long i = 0; i < size; i++) {
            hostBuffer[i] = s0 + s1;
            s1 ^= s0;
            s0 = rotl(s0, 55) ^ s1 ^ (s1 << 14);
            s1 = rotl(s1, 36);
        }
    }
    void setSeed(Long s) { seed = s; amplifier = s; generation = 1; }
    void rewind(Long n) {
        Long newPos = currentPosition + n;
        if (newPos > size) {
            generation += newPos / size;
            newPos = newPos % size;
        } else if (newPos == size) {
            generation++;
            newPos = 0;
        }
        currentPosition = newPos;
    }
    RngState deviceState() const {
        RngState st;
        st.buffer = reinterpret_cast<const unsigned long long *>(devBuffer);
        st.size = size;
        st.position = currentPosition;
        st.generation = generation;
        st.seed = seed;
        st.amplifier = amplifier;
        st.rSize = size > 0 ? 1.0 / (double)size : 0.0;
        st.mGeneration = generation > 0 ? ~0ULL / (unsigned long long)generation : 0ULL;
        st.mAmplifier = amplifier > 0 ? ~0ULL / (unsigned long long)amplifier : 0ULL;
        return st;
    }
};

}  // namespace nd4j_amd
