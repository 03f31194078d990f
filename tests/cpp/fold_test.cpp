// Host test of the constant folding of kten_amd/csrc/kth_fold.h: whenever fold_constants accepts a pair, its
// result must be the bits of the float operation itself (the host's single-precision + - * / are IEEE, correctly
// rounded), and it must decline subnormal or NaN operands and results.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "kth_fold.h"

static uint32_t bits(float v) { uint32_t b; std::memcpy(&b, &v, 4); return b; }
static float from_bits(uint32_t b) { float v; std::memcpy(&v, &b, 4); return v; }

int main() {
    uint64_t state = 0x243f6a8885a308d3ull;
    auto next = [&]() { state = state * 6364136223846793005ull + 1442695040888963407ull; return static_cast<uint32_t>(state >> 32); };
    const float edge[] = {0.0f, -0.0f, 1.0f, -1.0f, 2.0f, 0.5f, 3.0f, 1.0f / 3.0f, 1.17549435e-38f, 1.17549449e-38f, 3.4028235e38f, -3.4028235e38f,
                          1e-45f, 1e-40f, 16777216.0f, 16777217.0f, 1e30f, 1e-30f, 1e20f, 1e-20f, INFINITY, -INFINITY, NAN};
    const int n_edge = sizeof(edge) / sizeof(edge[0]);
    const int ops[] = {KTH_PLUS, KTH_MINUS, KTH_TIMES, KTH_DIV};
    unsigned long long folded = 0, declined = 0;
    for (long round = 0; round < 4000000; round++) {
        float x, y;
        if (round < n_edge * n_edge) { x = edge[round / n_edge]; y = edge[round % n_edge]; }
        else {
            x = from_bits(next()); y = from_bits(next());
            if (round % 3 == 0) y = from_bits(bits(x) + (next() % 64) - 32);           // near x: cancellation, quotients near 1
            if (round % 7 == 0) { x = from_bits((next() & 0x807fffffu) | ((1u + next() % 40) << 23)); }   // tiny magnitudes: products underflow
        }
        for (int op : ops) {
            volatile float vx = x, vy = y;
            volatile float direct = op == KTH_PLUS ? vx + vy : op == KTH_MINUS ? vx - vy : op == KTH_TIMES ? vx * vy : vx / vy;
            float got = 0.0f;
            const bool ok = kth::fold_constants(op, x, y, &got);
            const float want = direct;
            const bool sub = std::fpclassify(want) == FP_SUBNORMAL || std::fpclassify(x) == FP_SUBNORMAL || std::fpclassify(y) == FP_SUBNORMAL;
            const bool nan = std::isnan(want) || std::isnan(x) || std::isnan(y);
            if (ok) {
                folded++;
                if (sub || nan) { std::printf("op %d of %a and %a was folded to %a\n", op, x, y, got); return 1; }
                if (bits(got) != bits(want)) { std::printf("op %d of %a and %a: folded %a, the float operation gives %a\n", op, x, y, got, want); return 1; }
            } else {
                declined++;
                // declining is always safe; it is expected only for subnormal or NaN operands and results and for results
                // that round up to the smallest normal float
                if (!sub && !nan && std::fabs(want) > 1.17549435e-38f) {
                    std::printf("op %d of %a and %a (= %a) was declined\n", op, x, y, want); return 1;
                }
            }
        }
    }
    if (kth::fold_constants(KTH_POW, 2.0f, 3.0f, nullptr)) { std::printf("pow must not be folded\n"); return 1; }
    std::printf("fold ok: %llu folded, %llu declined\n", folded, declined);
    return 0;
}
