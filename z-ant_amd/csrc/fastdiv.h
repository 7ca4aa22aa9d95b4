// Division by a launch-time constant as a multiply-high and a shift; usable from host code (no HIP headers needed) and,
// under hipcc, from kernels.
#pragma once
#include <cstdint>

// Division by a divisor fixed at launch time: q = x / n for every x < 2^31, as one multiply-high and a shift
// (m = floor(2^(31+l) / n) + 1 with l = ceil(log2 n): the excess of m over 2^(31+l) / n is at most n / n, which x < 2^31
// cannot grow into a whole quotient step).  A runtime 32-bit division is some twenty VALU instructions.
struct FastDiv {
    unsigned m;
    int s;  // q = mulhi(x, m) >> s; s < 0: n == 1
};
static inline FastDiv make_fastdiv(unsigned n) {
    FastDiv d = {0u, -1};
    if (n <= 1) return d;
    int l = 0;
    while ((uint64_t(1) << l) < n) ++l;
    d.m = unsigned((uint64_t(1) << (31 + l)) / n + 1);
    d.s = l - 1;
    return d;
}
#if defined(__HIPCC__)
__device__ __forceinline__ unsigned fastdiv(unsigned x, FastDiv d) { return d.s < 0 ? x : __umulhi(x, d.m) >> d.s; }
#endif
