// Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11): a counter-based
// generator -- four 32-bit words that are a pure function of a 128-bit counter and a 64-bit key, so that the kernel
// that drops elements and the one that regenerates the mask for the backward pass agree by construction.
#pragma once
#include <cstdint>

namespace hstu {

struct PhiloxWords {
    uint32_t w[4];
};

__host__ __device__ inline PhiloxWords philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        c1 = (uint32_t)p1;
        c3 = (uint32_t)p0;
        c0 = n0;
        c2 = n2;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return PhiloxWords{{c0, c1, c2, c3}};
}

// Dropout of the output step: element (row r, column c) of the [rows, width] matrix `joined` is kept when word c % 4 of
// philox(counter = (group, offset), key = seed), group = (r * width + c) / 4, is at least `thresh` = floor(p * 2^32).
// `width` is the logical width (a multiple of 8), not a stride: the mask does not depend on how the matrix is stored.
struct DropoutParams {
    uint64_t seed, offset;
    uint32_t thresh;  // 0: nothing is dropped
    float scale;      // 1 / (1 - p), applied to the survivors in fp32 before they are rounded
};

// The words for the four elements of group `group`.
__host__ __device__ inline PhiloxWords dropout_words(const DropoutParams& d, uint64_t group) {
    return philox4x32_10((uint32_t)group, (uint32_t)(group >> 32), (uint32_t)d.offset, (uint32_t)(d.offset >> 32), (uint32_t)d.seed,
                         (uint32_t)(d.seed >> 32));
}

}  // namespace hstu
