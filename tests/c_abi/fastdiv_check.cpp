// Host check of the index divider the kernels use (autograd_amd/csrc/fastdiv.hpp) against
// the machine's own division: a stride through all 32-bit dividends for a list of divisors
// (the ones launches really use, powers of two and their neighbours, the extremes), the
// dividends at every multiple's edge, and random pairs.  Exit status 0 = no difference.
#include <cstdio>
#include <cstdlib>
#include "fastdiv.hpp"

int main() {
    unsigned long long bad = 0;
    const uint32_t ds[] = {1, 2, 3, 5, 6, 7, 8, 12, 16, 24, 32, 48, 64, 96, 127, 128, 129, 192, 384, 768, 1000, 1023, 1024,
                           1025, 1536, 1792, 2048, 4096, 14336, 65535, 65536, 65537, 1000003, 0x7fffffffu, 0x80000000u,
                           0x80000001u, 0xfffffffeu, 0xffffffffu};
    for (uint32_t d : ds) {
        const agrad::FastDiv f(d);
        for (uint64_t x = 0; x < (1ull << 32); x += 9973) {
            uint32_t rem;
            if (f.divmod((uint32_t)x, rem) != (uint32_t)x / d || rem != (uint32_t)x % d) ++bad;
        }
        const uint32_t xs[] = {0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 0xffffffffu, 0xfffffffeu, 0x80000000u, 0x7fffffffu};
        for (uint32_t x : xs)
            if (f.div(x) != x / d) ++bad;
    }
    srand(1);
    for (int i = 0; i < 3000000; ++i) {
        uint32_t d = ((uint32_t)rand() << 1) ^ (uint32_t)rand();
        if (i % 3 == 0) d &= 0xffffu;
        if (i % 7 == 0) d &= 0xffu;
        if (d == 0) d = 1;
        const uint32_t x = ((uint32_t)rand() << 16) ^ (uint32_t)rand();
        if (agrad::FastDiv(d).div(x) != x / d) ++bad;
    }
    if (bad) std::printf("fastdiv: %llu differences\n", bad);
    return bad != 0;
}
