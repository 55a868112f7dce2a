// Division by a launch-constant divisor without an integer divide in the kernel.
// For 0 <= n < 2^31 and 1 <= d < 2^31:  n / d == (n * M) >> s  with
// l = ceil(log2 d), s = 31 + l, M = ceil(2^s / d)  (M < 2^32).
// (Granlund & Montgomery, "Division by invariant integers using multiplication",
// with a 31-bit dividend so that the multiplier fits 32 bits.)
#pragma once
#include <cstdint>

#if defined(__HIP__)
#define MHIP_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define MHIP_HD inline
#endif

namespace mhip {

struct FastDiv32 {
    uint32_t d = 1;
    uint32_t mul = 0x80000000u;
    uint32_t shift = 31;

    FastDiv32() = default;
    explicit FastDiv32(uint32_t divisor) {
        d = divisor ? divisor : 1;
        uint32_t l = 0;
        while ((1ull << l) < d) ++l;
        shift = 31 + l;
        const unsigned __int128 one = 1;
        mul = (uint32_t)(((one << shift) + d - 1) / d);
    }
    MHIP_HD uint32_t div(uint32_t n) const { return (uint32_t)(((uint64_t)n * mul) >> shift); }
    MHIP_HD void divmod(uint32_t n, uint32_t& q, uint32_t& r) const {
        q = div(n);
        r = n - q * d;
    }
};

constexpr uint32_t kFastDivLimit = 0x7fffffffu;  // dividends and divisors must stay below 2^31

}  // namespace mhip
