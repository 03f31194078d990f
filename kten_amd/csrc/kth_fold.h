// Folding of constant (op) constant on the host (no device code here: the header is also built into a host test).
#pragma once

#include <cstdint>
#include <cstring>

#include "../../include/kten_hip.h"

namespace kth {

// op(x, y) of two constants on the host, for the result of a scalar operation on a store that is one
// owed constant: the store of the result is then owed the outcome and nothing is launched. Done only
// where the host's arithmetic cannot differ from the kernel's: finite-or-infinite operands that are not
// subnormal, a result that is neither NaN nor subnormal. The value is formed in double and rounded once
// more to float; for + - x / of floats that second rounding changes nothing (53 >= 2 * 24 + 2).
inline bool fold_constants(int op, float x, float y, float* out) {
    auto plain = [](float v) {
        uint32_t b; memcpy(&b, &v, 4);
        const uint32_t e = (b >> 23) & 0xffu;
        return (e != 0u || (b & 0x7fffffu) == 0u) && !(e == 0xffu && (b & 0x7fffffu) != 0u);   // not subnormal, not NaN
    };
    if (!plain(x) || !plain(y)) return false;
    const double dx = x, dy = y;
    double r;
    switch (op) {
    case KTH_PLUS:  r = dx + dy; break;
    case KTH_MINUS: r = dx - dy; break;
    case KTH_TIMES: r = dx * dy; break;
    case KTH_DIV:   r = dx / dy; break;
    default: return false;
    }
    if (r != r) return false;
    if (r != 0.0 && (r < 0 ? -r : r) < 1.17549435082228750797e-38) return false;
    *out = static_cast<float>(r);
    return true;
}


}  // namespace kth
