// Exact division of a 32-bit index by a divisor the host knows at launch: one multiply-high,
// a subtract, an add and two shifts (Granlund & Montgomery's round-up method: with
// L = ceil(log2 d) and m = floor(2^32 (2^L - d) / d) + 1, x / d = (t + ((x - t) >> min(L, 1)))
// >> max(L - 1, 0) where t = mulhi(m, x), for every 32-bit x and every d >= 1).  The
// compiler's own sequence for a divisor it does not know is a float reciprocal with two
// corrections, about 25 instructions in front of a thread's first load.
//
// Plain C++: the device code includes it through common.hpp, and a host-compiled test
// checks it against the machine's division.
#pragma once
#include <cstdint>

#if defined(__HIPCC__)
#define AGRAD_FASTDIV_FN __host__ __device__ __forceinline__
#else
#define AGRAD_FASTDIV_FN inline
#endif

namespace agrad {

struct FastDiv {
    uint32_t d, m, sh1, sh2;
    FastDiv() = default;
    explicit FastDiv(uint32_t divisor) {
        d = divisor ? divisor : 1u;
        uint32_t L = 0;
        while (L < 32 && (1ull << L) < d) ++L;
        m = (uint32_t)((((1ull << L) - d) << 32) / d) + 1u;
        sh1 = L < 1 ? L : 1u;
        sh2 = L > 0 ? L - 1 : 0u;
    }
    AGRAD_FASTDIV_FN uint32_t div(uint32_t x) const {
        const uint32_t t = (uint32_t)(((uint64_t)m * x) >> 32);
        return (t + ((x - t) >> sh1)) >> sh2;
    }
    // x / d, and the remainder
    AGRAD_FASTDIV_FN uint32_t divmod(uint32_t x, uint32_t& rem) const {
        const uint32_t q = div(x);
        rem = x - q * d;
        return q;
    }
};

}  // namespace agrad
