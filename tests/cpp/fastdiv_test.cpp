// Host test of the launch-constant divider (kten_amd/csrc/kth_fastdiv.h): a zero divisor, which
// the plan builders meet for a dim of an empty tensor, must not divide on the host, and every other
// divisor must give n / d for numerators below 2^31.
#include <cstdint>
#include <cstdio>

#include "kth_fastdiv.h"

int main() {
    const kth::FastDiv z = kth::make_div(0);
    if (z.mul != 0 || z.shift != 0) { std::printf("make_div(0) = {%u, %u}\n", z.mul, z.shift); return 1; }
    uint64_t state = 0x9e3779b97f4a7c15ull, checked = 0;
    auto next = [&]() { state = state * 6364136223846793005ull + 1442695040888963407ull; return static_cast<uint32_t>(state >> 33); };
    const uint32_t edge[] = {1u, 2u, 3u, 4u, 5u, 7u, 255u, 256u, 257u, 4095u, 4096u, 65535u, 65536u, 65537u,
                             0x3fffffffu, 0x40000000u, 0x40000001u, 0x7ffffffeu, 0x7fffffffu};
    for (int round = 0; round < 4000; round++) {
        const uint32_t d = round < 19 ? edge[round] : (next() >> (next() % 31)) | 1u;
        const kth::FastDiv f = kth::make_div(d);
        for (int k = 0; k < 500; k++) {
            uint32_t n = next() & 0x7fffffffu;
            if (k < 19) n = edge[k] & 0x7fffffffu;
            if (k == 19) n = 0;
            if (k >= 20 && k < 30) n = static_cast<uint32_t>((static_cast<uint64_t>(d) * (k - 19) - (k & 1)) & 0x7fffffffu);
            if (kth::fast_div(n, f) != n / d) { std::printf("%u / %u: got %u\n", n, d, kth::fast_div(n, f)); return 1; }
            checked++;
        }
    }
    std::printf("fastdiv ok: %llu quotients\n", static_cast<unsigned long long>(checked));
    return 0;
}
