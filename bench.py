#!/usr/bin/env python3
"""Benchmark of the kten-hip hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg5] [--cpu-baseline/--no-cpu-baseline]

A step is one pass of the chosen workload's raw-op sequence over device-resident
synthetic inputs (kten_amd/workloads.py). The default workload is cfg5: the autograd
forward + backward of loss = sum(((x*w)+b) pow 2) on x[16384,4096], which exercises
broadcast binary ops, tensor-scalar ops, the full sum and the reduce-to-shape axis sums.
Prints ONE JSON line on stdout; everything else goes to stderr.

Timing: HIP events on the library's own stream around the K timed steps (kth_timer_*),
with a host-side wall clock around the same region as a cross-check. Per-kernel
durations come from HIP event pairs the library records around every launch inside the
same timed region (kth_profile_*).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch), each
# scaled by what the same counter reads for the plain copy kernel unary_kernel<OpIdentity>
# of 262 144 KiB (FETCH_SIZE x 1.9999, WRITE_SIZE x 1.000). Source: profiles/*.md.
MEASURED_TRAFFIC_BYTES = {
    ("cfg5", "binary_same_kernel<OpTimes>"): int((262155 * (262144 / 131077) + 262144) * 1024),
}
METRIC = "achieved HBM GB/s (% of MI355X peak) for broadcast binary ops and axis sum"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_step(name, ops, inputs):
    """Returns a zero-argument callable running one pass of the workload on resident inputs."""
    from kten_amd.workloads import WORKLOADS, cfg5_setup, cfg5_step
    wl = WORKLOADS[name]
    if name == "cfg5":
        x, w, b = cfg5_setup(ops, inputs)
        for t in (x, w, b):
            t.incrementRef()          # inputs outlive every garbage-collector scope

        def step():
            return cfg5_step(x, w, b)          # backward() opens its own garbage-collector scope
        return step
    if name in ("max_backward", "softmax_ce"):
        # Leaves are created once; the step is graph + backward, gradients zeroed in between.
        first = "x" if name == "max_backward" else "logits"
        leaf = ops.create(list(inputs[first].shape), True, inputs[first])
        other = None if name == "max_backward" else ops.create(list(inputs["targets"].shape), False, inputs["targets"])

        def step():
            out = leaf.max(-1).sum() if other is None else leaf.softmaxCrossEntropy(other)
            out.backward()
            return out
        return step
    resident = {k: ops.createRaw(list(v.shape), v) for k, v in inputs.items()}
    for r in resident.values():
        r.incrementRef()

    class Resident:
        """Hands the workload tensors that are already on the device."""
        def __init__(self, ops):
            self.ops = ops
        def __getattr__(self, k):
            return getattr(self.ops, k)
        def create(self, shape, requiresGrad, init):
            from kten_amd.autograd import NoGradVariable
            for key, v in inputs.items():
                if v is init:
                    return NoGradVariable(self.ops, resident[key])
            raise KeyError("unknown input")

    proxy = Resident(ops)

    def step():
        with ops.garbageCollector():
            return wl.run(proxy, inputs)
    return step


def cpu_baseline(name, threads):
    """The CPU restatement of kten-jvm on a bounded sample of the same workload."""
    from kten_amd.workloads import WORKLOADS
    from oracle import jvm_oracle as jo
    wl = WORKLOADS[name]
    sample = {"cfg1": dict(wl.full_dims), "cfg2": dict(wl.full_dims), "cfg3": dict(wl.full_dims),
              "cfg4": dict(wl.full_dims), "cfg5": dict(wl.full_dims),
              "max_backward": dict(wl.full_dims), "softmax_ce": {"batch": 8192, "classes": 2048},
              "reduce_shapes": {"scale": 4}, "indexed_moves": {"rows": 4096, "cols": 4096}, "layout_shapes": {"scale": 8}, "unary_maps": {"n": 1 << 25}}.get(name, dict(wl.full_dims))
    inputs = wl.make_inputs(sample)
    jo.set_threads(threads)
    try:
        cpu = jo.JvmOracleOperations()
        t0 = time.perf_counter()
        wl.run(cpu, inputs)
        dt = time.perf_counter() - t0
    finally:
        jo.set_threads(1)
    nbytes = wl.algorithmic_bytes(sample)
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{name} at {sample} ({nbytes / 1e6:.0f} MB algorithmic, {dt:.2f} s): C restatement of kten-jvm "
                      "semantics, not kten-jvm itself; copy-producing ops and sum() single-threaded as in the "
                      f"reference, in-place ops and axis reductions on {threads} threads"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="cfg5",
                    choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "max_backward", "softmax_ce", "transpose", "permute",
                             "concat_mask", "batch_norm", "reduce_shapes", "indexed_moves", "layout_shapes", "unary_maps"])
    ap.add_argument("--cpu-baseline", dest="cpu", action="store_true", default=True)
    ap.add_argument("--no-cpu-baseline", dest="cpu", action="store_false")
    ap.add_argument("--no-kernel-events", dest="events", action="store_false", default=True,
                    help="do not bracket every launch with an event pair inside the timed region")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this backend drives one GPU; the hot path has no cross-GPU step. Run with --gpus 1.")
        sys.exit(2)

    import kten_amd
    from kten_amd.workloads import WORKLOADS
    wl = WORKLOADS[args.config]
    dims = wl.full_dims
    nbytes = wl.algorithmic_bytes(dims)
    ops = kten_amd.platform(0)
    log(f"platform {ops.platformKey}: {ops.computeUnits} CUs, wave {ops.waveSize}, {ops.availableMemory / 2**30:.0f} GiB")
    log(f"workload {wl.name}: {wl.description}; {nbytes} algorithmic bytes per step")
    t0 = time.perf_counter()
    inputs = wl.make_inputs(dims)
    log(f"inputs generated in {time.perf_counter() - t0:.1f} s")
    step = make_step(args.config, ops, inputs)

    for _ in range(args.warmup):
        step()
    ops.sync()
    m0 = ops.getMetrics()
    # Timed region: exactly K steps between two events on the library's stream, with a
    # host wall clock around the same region (stream drained on both sides).
    wall0 = time.perf_counter()
    ops.timerBegin()
    for _ in range(args.steps):
        last = step()
    total_ms = ops.timerEnd()
    ops.sync()
    wall_ms = (time.perf_counter() - wall0) * 1e3
    m = ops.getMetrics()
    counted = (m["bytesMoved"] - m0["bytesMoved"]) / args.steps
    launches = (m["launches"] - m0["launches"]) / args.steps
    ms_per_step = total_ms / args.steps
    gbps = nbytes / ms_per_step / 1e6
    log(f"{args.steps} steps: {total_ms:.3f} ms on the stream, {wall_ms:.3f} ms wall; {launches:.0f} launches/step; "
        f"library counted {counted:.0f} B/step (formula {nbytes})")

    # Per-kernel durations: the same K steps again, now with a HIP event pair around
    # every launch. Kept out of the region `value` is computed from, because the event
    # pairs themselves cost about a tenth of the step time.
    kernels = {}
    if args.events:
        ops.profileBegin()
        ops.timerBegin()
        for _ in range(args.steps):
            step()
        ev_ms = ops.timerEnd()
        kernels = ops.profileEnd()
        log(f"{args.steps} steps with per-launch events: {ev_ms:.3f} ms on the stream")

    roofline = None
    if kernels:
        log(f"{'kernel':48s} {'launches':>8s} {'avg us':>9s} {'GB/s':>9s} {'% time':>7s}")
        tot = sum(v[2] for v in kernels.values())
        for k, (n, b, ms) in sorted(kernels.items(), key=lambda kv: -kv[1][2]):
            log(f"{k:48s} {n:8d} {ms / n * 1e3:9.2f} {(b / ms / 1e6) if ms else 0:9.1f} {100 * ms / tot:7.1f}")
        dom, (n, b, ms) = max(kernels.items(), key=lambda kv: kv[1][2])
        achieved = b / ms / 1e6
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBPS, 4),
                    "traffic": MEASURED_TRAFFIC_BYTES.get((args.config, dom)),
                    "bytes_per_launch": b // n, "avg_launch_us": round(ms / n * 1e3, 3), "launches": n,
                    "kernel_time_share": round(ms / tot, 4)}

    line = {
        "metric": METRIC, "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{wl.name}: {wl.description}", "algorithmic_bytes_per_step": nbytes,
                   "launches_per_step": launches, "elements_per_s": round(sum(int(v.size) for v in inputs.values())
                                                                         / (ms_per_step / 1e3)),
                   "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "wall_ms_per_step": round(wall_ms / args.steps, 4),
                   "per_kernel_durations": "HIP event pair around every launch, over a second pass of the same K steps"
                   if args.events else None},
        "roofline": roofline,
    }
    if args.cpu:
        threads = min(16, os.cpu_count() or 1)
        log(f"timing the CPU restatement on {threads} threads ...")
        line["cpu_baseline"] = cpu_baseline(args.config, threads)
        log(f"cpu baseline: {line['cpu_baseline']['value']} GB/s")
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
