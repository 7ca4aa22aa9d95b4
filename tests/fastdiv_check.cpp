// CPU check of the fixed-divisor division the kernels use for index decoding (csrc/fastdiv.h): the multiplier and
// shift make_fastdiv() returns must give x / n for every dividend below 2^31.  The kernel-side fastdiv() is the same
// two operations (__umulhi, shift), restated here with 64-bit host arithmetic.
#include <cstdio>
#include <cstdlib>

#include "fastdiv.h"

static unsigned apply(unsigned x, FastDiv d) { return d.s < 0 ? x : unsigned((uint64_t(x) * d.m) >> 32) >> d.s; }

int main() {
    unsigned long long bad = 0, checked = 0;
    const unsigned top = 0x7fffffffu;
    const unsigned ns[] = {1, 2, 3, 4, 5, 6, 7, 9, 10, 13, 14, 16, 17, 25, 28, 56, 64, 100, 169, 255, 256, 257, 1000, 4095, 4096,
                           4097, 65535, 65536, 65537, 1u << 20, (1u << 20) + 1, 1u << 30, (1u << 30) + 1, top - 1, top};
    srand(1);
    for (unsigned n : ns) {
        const FastDiv d = make_fastdiv(n);
        const uint64_t steps = top / n;
        for (uint64_t k = 0; k < 3000; ++k) {
            // both ends of quotient steps near the bottom and the top of the range, and random dividends
            const uint64_t q = steps - k % (steps + 1);
            const uint64_t xs[] = {k, k * n, k * n + n - 1, top - k, q * n, q * n + n - 1, uint64_t(rand()) * 2 + (rand() & 1)};
            for (uint64_t x : xs) {
                if (x > top) continue;
                ++checked;
                if (apply(unsigned(x), d) != unsigned(x) / n) ++bad;
            }
        }
    }
    // every divisor up to 5000 against the top of the dividend range (where a too-small multiplier fails first) and the bottom
    for (unsigned n = 1; n <= 5000; ++n) {
        const FastDiv d = make_fastdiv(n);
        for (unsigned x = top - 20000; x <= top && x >= top - 20000; ++x) { ++checked; if (apply(x, d) != x / n) ++bad; }
        for (unsigned x = 0; x < 20000; ++x) { ++checked; if (apply(x, d) != x / n) ++bad; }
    }
    printf("checked %llu bad %llu\n", checked, bad);
    return bad != 0;
}
