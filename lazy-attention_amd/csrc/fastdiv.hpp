// Exact division by a divisor fixed at launch time, without a division instruction.  Plain C++: usable on the host
// (where the multiplier is formed, and where the unit test runs) and in device code.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define LAZYATTN_HD __host__ __device__ __forceinline__
#else
#define LAZYATTN_HD inline
#endif

namespace lazyattn {

// Division of a 32-bit unsigned number by a divisor known at launch: the host forms a multiplier and two shifts
// (the round-up method: exact for every 32-bit numerator) and the kernel spends a multiply-high, a subtraction, an
// addition and two shifts -- on the scalar unit for wave-uniform values -- where the general division is some forty
// instructions.  The work-item decode and the split ranges at the head of the kernel divide seven times, on every
// wave's way to its first memory request.
struct FastDiv {
    uint32_t mul, sh1, sh2, div;
    static LAZYATTN_HD uint32_t mulhi(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }
    LAZYATTN_HD explicit FastDiv(uint32_t d = 1) : mul(0), sh1(0), sh2(0), div(d) {
        if (d <= 1) return;                                      // n / 1: (0 + (n >> 0)) >> 0
        uint32_t s = 0;
        while ((1ull << s) < d) ++s;                             // ceil(log2 d)
        mul = (uint32_t)(((1ull << 32) * ((1ull << s) - d)) / d + 1);
        sh1 = 1;
        sh2 = s - 1;
    }
    LAZYATTN_HD uint32_t quot(uint32_t n) const {
        const uint32_t t = mulhi(n, mul);
        return (t + ((n - t) >> sh1)) >> sh2;
    }
    LAZYATTN_HD uint32_t rem(uint32_t n, uint32_t q) const { return n - q * div; }
};

}  // namespace lazyattn
