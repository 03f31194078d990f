// Division by a launch-constant divisor (host side; no device headers, so host tests can include it).
#pragma once

#include <cstdint>

namespace kth {

// Division by a launch-constant divisor d for numerators below 2^31:
// q = (mulhi(n, mul) + n) >> shift with shift = ceil(log2 d), mul = floor(2^32 (2^shift - d) / d) + 1.
struct FastDiv { uint32_t mul, shift; };

// d == 0 (a dim of an empty tensor: nothing is launched over it) gives a divider that is never used
// rather than a host division by zero.
inline FastDiv make_div(uint32_t d) {
    FastDiv f{0, 0};
    if (d == 0) return f;
    uint32_t shift = 0;
    while ((1ull << shift) < d) shift++;
    f.shift = shift;
    f.mul = static_cast<uint32_t>((((1ull << shift) - d) << 32) / d + 1);
    return f;
}

// The quotient as the kernels compute it (__umulhi on the device).
inline uint32_t fast_div(uint32_t n, FastDiv f) {
    return static_cast<uint32_t>(((static_cast<uint64_t>(n) * f.mul) >> 32) + n) >> f.shift;
}

}  // namespace kth
