// The fp32 routines of the math mode "within 2 ulp" (kten_amd/csrc/kth_f32math.h) on the host, against
// (float) libm_f64((double) x), the value kotlin.math's Float overloads return (JVMRawTensor.kt:144,395-425).
// The header uses IEEE operations only, so these are the bits the device computes.
//
//   f32math_test [stride]      every stride-th bit pattern of the 2^32 (default 509; 1 = all of them)
//
// Prints, per function, how many results lie 0, 1, 2 and more ulps from that float, and fails if any lies more than 2
// away. sin / cos / tan are checked for |x| <= 65536 (beyond, every mode takes the long f64 routine on the device).
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "../../kten_amd/csrc/kth_f32math.h"

using namespace kth::f32;

static int64_t ordered(float x) {                       // monotone map of the floats to integers; -0 and +0 one step apart
    uint32_t u; memcpy(&u, &x, 4);
    return (u & 0x80000000u) ? -static_cast<int64_t>(u & 0x7fffffffu) - 1 : static_cast<int64_t>(u);
}

static uint64_t ulp_distance(float got, float want) {
    if (got != got && want != want) return 0;
    if (got != got || want != want) return 1u << 30;
    const int64_t d = ordered(got) - ordered(want);
    return static_cast<uint64_t>(d < 0 ? -d : d);
}

struct Case {
    const char* name;
    float (*fast)(float);
    double (*exact)(double);
    float limit;                                        // |x| beyond it is not checked (0: everything)
};

int main(int argc, char** argv) {
    const uint64_t stride = argc > 1 ? strtoull(argv[1], nullptr, 10) : 509;
    const Case cases[] = {
        {"exp", exp_, exp, 0}, {"log", log_, log, 0},
        {"tanh", tanh_, tanh, 0}, {"sinh", sinh_, sinh, 0}, {"cosh", cosh_, cosh, 0},
        {"sin", sin_short, sin, kTrigLimit}, {"cos", cos_short, cos, kTrigLimit}, {"tan", tan_short, tan, kTrigLimit},
        {"asin", asin_, asin, 0}, {"acos", acos_, acos, 0}, {"atan", atan_, atan, 0},
    };
    const unsigned threads = std::max(1u, std::min(16u, std::thread::hardware_concurrency()));
    int failed = 0;
    printf("%-8s %12s %12s %10s %8s %6s   worst input\n", "function", "inputs", "0 ulp", "1 ulp", "2 ulp", "> 2");
    for (const Case& c : cases) {
        std::vector<uint64_t> hist(threads * 4, 0), worst(threads, 0);
        std::vector<uint32_t> worst_at(threads, 0);
        std::vector<std::thread> pool;
        for (unsigned t = 0; t < threads; t++) {
            pool.emplace_back([&, t] {
                // the strided patterns, then (thread 0) the special values whatever the stride
                static const uint32_t special[] = {0x00000000u, 0x80000000u, 0x7f800000u, 0xff800000u, 0x7fc00000u, 0xffc00001u,
                                                   0x00000001u, 0x80000001u, 0x007fffffu, 0x00800000u, 0x7f7fffffu, 0xff7fffffu,
                                                   0x3f800000u, 0xbf800000u, 0x3f7fffffu, 0x3f800001u, 0x3f000000u, 0xbf000000u,
                                                   0x47800000u, 0xc7800000u, 0x42b17218u, 0x42b2d4fcu, 0x42b2d4fdu, 0xc2cff1b5u};
                const uint64_t extra = t == 0 ? sizeof(special) / sizeof(special[0]) : 0;
                for (uint64_t b = t * stride, i = 0; b < (1ull << 32) || i < extra; b += threads * stride) {
                    const uint32_t u = b < (1ull << 32) ? static_cast<uint32_t>(b) : special[i++];
                    float x; memcpy(&x, &u, 4);
                    if (c.limit != 0 && !(fabsf(x) <= c.limit)) continue;
                    const float want = static_cast<float>(c.exact(static_cast<double>(x)));
                    const uint64_t d = ulp_distance(c.fast(x), want);
                    hist[t * 4 + (d > 3 ? 3 : d)]++;
                    if (d > worst[t]) { worst[t] = d; worst_at[t] = u; }
                }
            });
        }
        for (auto& th : pool) th.join();
        uint64_t h[4] = {0, 0, 0, 0}, w = 0; uint32_t at = 0;
        for (unsigned t = 0; t < threads; t++) {
            for (int i = 0; i < 4; i++) h[i] += hist[t * 4 + i];
            if (worst[t] > w) { w = worst[t]; at = worst_at[t]; }
        }
        float xw; memcpy(&xw, &at, 4);
        printf("%-8s %12llu %12llu %10llu %8llu %6llu   %llu ulp at %.9g (0x%08x)\n", c.name,
               (unsigned long long)(h[0] + h[1] + h[2] + h[3]), (unsigned long long)h[0], (unsigned long long)h[1],
               (unsigned long long)h[2], (unsigned long long)h[3], (unsigned long long)w, xw, at);
        if (h[3]) failed = 1;
    }
    return failed;
}
