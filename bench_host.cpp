// cfg1 of the benchmark (y = (x + b) * x; s = sum(y) on x[2048,1024], b[1024]) issued by a compiled host: the C++
// mirror of the raw-tensor contract (include/kten_hip.hpp) in place of bench.py's Python mirror. With 8 MB tensors a
// step is four launches of a few microseconds each, and how fast the host issues them decides the step time; the
// reference's host is compiled (Kotlin on a JVM), so this is the figure to read for that configuration.
// bench.py runs this program for config.other_configs.cfg1.compiled_host and prints its one JSON line there.
//
//   bench_host [steps] [warmup]
#include <chrono>
#include <cstdio>
#include <cstdlib>

#include "kten_hip.hpp"
#include "kten_hip_bench.h"

using namespace kten::hip;

int main(int argc, char** argv) {
    const int steps = argc > 1 ? std::atoi(argv[1]) : 100;
    const int warmup = argc > 2 ? std::atoi(argv[2]) : 20;
    if (steps < 1 || warmup < 0) { std::fprintf(stderr, "usage: bench_host [steps >= 1] [warmup >= 0]\n"); return 2; }
    try {
        HipTensorOperations ops(0);
        const int rows = 2048, cols = 1024;
        // values in (-1, 1) from a 64-bit mix of the element number: any data of that range times alike
        auto value = [](int i) {
            uint64_t z = (static_cast<uint64_t>(i) + 1) * 0x9E3779B97F4A7C15ull;
            z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull; z ^= z >> 27;
            return static_cast<float>(static_cast<double>(z >> 11) / 9007199254740992.0 * 2.0 - 1.0);
        };
        Raw x = ops.createRaw(Shape{rows, cols}, value);
        Raw b = ops.createRaw(Shape{cols}, value);
        auto step = [&]() {
            auto scope = ops.garbageCollector();        // releases y, its intermediate and s when the step ends
            Raw y = x->plus(b)->times(x);
            Raw s = y->sum();
        };
        for (int i = 0; i < warmup; i++) step();
        ops.sync();
        uint64_t launches0 = 0, launches1 = 0, dummy = 0, moved0 = 0, moved1 = 0;
        check(kth_metrics(&dummy, &dummy, &launches0, &moved0));
        const auto t0 = std::chrono::steady_clock::now();
        check(kth_timer_begin());
        for (int i = 0; i < steps; i++) step();
        const double issued_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        float total_ms = 0.0f;
        check(kth_timer_end(&total_ms));
        ops.sync();
        const double wall_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        check(kth_metrics(&dummy, &dummy, &launches1, &moved1));
        const double bytes = 4.0 * (6.0 * rows * cols + cols + 1);     // the op list of the step: x + b, * x, sum
        std::printf("{\"host\": \"C++ mirror of the contract (include/kten_hip.hpp)\", \"steps\": %d, \"warmup\": %d, "
                    "\"ms_per_step\": %.5f, \"wall_ms_per_step\": %.5f, \"host_issue_ms_per_step\": %.5f, "
                    "\"launches_per_step\": %.1f, \"algorithmic_bytes_per_step\": %.0f, \"GBps\": %.1f}\n",
                    steps, warmup, total_ms / steps, wall_ms / steps, issued_ms / steps,
                    static_cast<double>(launches1 - launches0) / steps, bytes, bytes / (total_ms / steps) / 1e6);
    } catch (const std::exception& e) {
        std::fprintf(stderr, "bench_host: %s\n", e.what());
        return 1;
    }
    return 0;
}
