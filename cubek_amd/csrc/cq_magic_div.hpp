// Division by a launch-invariant divisor as a multiplication and a shift, for the wave-uniform
// row arithmetic of the kernels (a scalar unit has no integer division).  Plain C++: the host
// computes the constants, host tests check them, the kernels apply them.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define CQ_MAGIC_FN __host__ __device__ inline
#else
#define CQ_MAGIC_FN inline
#endif

namespace cq {

// For d >= 1 and any n < 2^31: with s = ceil(log2 d) and magic = floor(2^(31+s) / d) + 1
// (which fits 32 bits), n / d == (n * magic) >> (31 + s).
CQ_MAGIC_FN void magic_of(uint32_t d, uint32_t* magic, uint32_t* shift) {
    uint32_t s = 0;
    while ((1ull << s) < d) s++;
    *magic = static_cast<uint32_t>((1ull << (31 + s)) / d + 1);
    *shift = 31 + s;
}
CQ_MAGIC_FN uint32_t magic_div(uint32_t n, uint32_t magic, uint32_t shift) {
    return static_cast<uint32_t>((static_cast<uint64_t>(n) * magic) >> shift);
}

}  // namespace cq
