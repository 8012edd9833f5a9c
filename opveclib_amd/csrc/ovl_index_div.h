// Division of a 32-bit index by a divisor that is fixed per launch: one multiply-high, one subtraction, one addition
// and two shifts instead of the integer division sequence (Granlund & Montgomery, "Division by invariant integers
// using multiplication").  Exact for every 32-bit dividend and every divisor from 1 to 2^32 - 1
// (tests/test_index_div_host.py).  Compiles for the host and for the device.
#ifndef OVL_INDEX_DIV_H_
#define OVL_INDEX_DIV_H_

#include <stdint.h>

#if defined(__HIPCC__)
#define OVL_INDEX_DIV_HD __host__ __device__ __forceinline__
#else
#define OVL_INDEX_DIV_HD inline
#endif

struct index_divisor {
    uint32_t divisor, magic, shift1, shift2;
};

OVL_INDEX_DIV_HD uint32_t divide(uint32_t n, const index_divisor& d) {
    const uint32_t t = (uint32_t)(((uint64_t)d.magic * n) >> 32);
    return (t + ((n - t) >> d.shift1)) >> d.shift2;
}

inline index_divisor make_divisor(uint32_t divisor) {
    uint32_t log2_ceil = 0;
    while ((1ull << log2_ceil) < divisor) ++log2_ceil;
    index_divisor d;
    d.divisor = divisor;
    d.magic = (uint32_t)(((1ull << 32) * ((1ull << log2_ceil) - divisor)) / divisor + 1);
    d.shift1 = log2_ceil < 1 ? log2_ceil : 1;
    d.shift2 = log2_ceil > 1 ? log2_ceil - 1 : 0;
    return d;
}

#endif  // OVL_INDEX_DIV_H_
