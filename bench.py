#!/usr/bin/env python3
"""Benchmark of the kten-hip hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg5] [--cpu-baseline/--no-cpu-baseline]
                  [--no-kernel-events] [--no-cold] [--no-copy-ceiling] [--no-other-configs] [--math-mode exact|within_2_ulp]

A step is one pass of the chosen workload's raw-op sequence over device-resident
synthetic inputs (kten_amd/host_mirror/workloads.py). The default workload is cfg5: the autograd
forward + backward of loss = sum(((x*w)+b) pow 2) on x[16384,4096], which exercises
broadcast binary ops, tensor-scalar ops, the full sum and the reduce-to-shape axis sums.
Prints ONE JSON line on stdout; everything else goes to stderr.

`value` = bytes per step / time per step, with the bytes taken as the smaller of two totals: the
op-at-a-time total of the reference's op list (operands at their un-broadcast size, every result
once) and what the library's launches of that step really read and wrote. The second is smaller
where a tensor that is one constant (a fresh zerosLike, the broadcast seed gradient) is never
written out and read back, and where a copy (pow with the exponent 1 in the backward pass of a
square, copy()) is never made because neither side is written while both are alive; bytes that did
not cross the memory bus are not counted as bandwidth.
`config` carries both totals.

Timing: W warm-up steps, then exactly K steps between two HIP events on the library's own stream
(kth_timer_begin / kth_timer_end): `value` and `ms_per_step` come from that region; a host-side wall
clock around it is the cross-check. Median and minimum come from a second pass of K steps with an
event after every step (kth_timer_lap; each such event costs the stream about 2 us, so the pass with
them is not the one `value` is taken from). Per-kernel durations come from the start and stop events
that every launch of a third pass over the same K steps carries itself (kth_profile_*: the dispatch's own duration).
With the default workload the other BASELINE configurations (cfg1-cfg4) are timed the same way after
it and reported under config.other_configs.

Two context figures are measured in the same run: the device-to-device copy rate of this GPU
(`roofline.copy_ceiling`, hipMemcpyAsync and the library's copy kernel on 1 GiB), and the
dominant kernel launched over a rotation of buffer sets that no recent launch has touched
(`roofline.achieved_cold`), to tell what the memory-side cache contributes to `achieved`, which
is measured inside the op-at-a-time chain where every kernel reads what the previous one wrote.
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

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc request counters: reads as
# 64 x TCC_EA0_RDREQ_64B + 128 x TCC_EA0_RDREQ_128B (no 32-byte requests), writes as 64 x TCC_EA0_WRREQ_64B.
# Transcribed from the profile named beside it; this run does not measure it.
MEASURED_TRAFFIC_BYTES = {
    ("cfg5", "binary_same_kernel<OpTimes>"): 147 * 64 + 4194304 * 128 + 4194304 * 64,
    ("cfg5", "binary_bcast_vec_kernel_vv<OpTimes>"): 315 * 64 + 2097830 * 128 + 4194304 * 64,
}
TRAFFIC_SOURCE = ("profiles/cfg5_autograd_kernels.md (rocprofv3 --pmc TCC_EA0_RDREQ_{32B,64B,128B}_sum, TCC_EA0_WRREQ_{,64B}_sum of an "
                  "earlier run: requests times their sizes; transcribed, not measured by this run)")
METRIC = "achieved HBM GB/s (% of MI355X peak) for broadcast binary ops and axis sum"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_step(name, ops, inputs):
    """Returns a zero-argument callable running one pass of the workload on resident inputs, and the
    resident tensors (to be released by the caller when the workload is done)."""
    from kten_amd.host_mirror.workloads import WORKLOADS, cfg5_setup, cfg5_step
    wl = WORKLOADS[name]
    if name == "cfg5":
        x, w, b = cfg5_setup(ops, inputs)
        for t in (x, w, b):
            t.incrementRef()          # inputs outlive every garbage-collector scope

        def step():
            return cfg5_step(x, w, b)          # backward() opens its own garbage-collector scope
        return step, [x, w, b]
    if name in ("max_backward", "softmax_ce"):
        # Leaves are created once; the step is graph + backward, gradients zeroed in between.
        first = "x" if name == "max_backward" else "logits"
        leaf = ops.create(list(inputs[first].shape), True, inputs[first])
        other = None if name == "max_backward" else ops.create(list(inputs["targets"].shape), False, inputs["targets"])

        def step():
            out = leaf.max(-1).sum() if other is None else leaf.softmaxCrossEntropy(other)
            out.backward()
            return out
        return step, [t for t in (leaf, other) if t is not None]
    resident = {k: ops.createRaw(list(v.shape), v) for k, v in inputs.items()}
    for r in resident.values():
        r.incrementRef()

    from kten_amd.host_mirror.autograd import NoGradVariable
    by_identity = {id(v): resident[k] for k, v in inputs.items()}

    class Resident:
        """Hands the workload tensors that are already on the device."""
        def __init__(self, ops):
            self.ops = ops
        def __getattr__(self, k):
            return getattr(self.ops, k)
        def create(self, shape, requiresGrad, init):
            return NoGradVariable(self.ops, by_identity[id(init)])      # (KeyError: not one of the workload's inputs)

    proxy = Resident(ops)

    def step():
        with ops.garbageCollector():
            return wl.run(proxy, inputs)
    return step, list(resident.values())


def cold_probe(ops, kernel, nbytes_per_launch, dims, sets=8, rounds=3):
    """Average microseconds of `kernel` when each launch works on a buffer set of its own, `sets` of them in
    rotation, so that nothing it reads or writes was touched by the launches just before it (the sets together
    are several times the 256 MB memory-side cache). None for kernels it has no recipe for."""
    import ctypes
    import numpy as np
    from kten_amd import abi
    from kten_amd.abi import Op, check
    family, _, op = kernel.partition("<")
    op = op.rstrip(">")
    lib = ops.lib
    binary = {"OpPlus": Op.PLUS, "OpMinus": Op.MINUS, "OpTimes": Op.TIMES, "OpDiv": Op.DIV}
    unary = {"OpNeg": Op.NEG, "OpAbs": Op.ABS, "OpExp": Op.EXP, "OpLog": Op.LOG, "OpSqrt": Op.SQRT, "OpTanh": Op.TANH,
             "OpSigmoid": Op.SIGMOID, "OpSinh": Op.SINH, "OpCosh": Op.COSH, "OpSin": Op.SIN, "OpCos": Op.COS, "OpTan": Op.TAN,
             "OpAsin": Op.ASIN, "OpAcos": Op.ACOS, "OpAtan": Op.ATAN}
    rng = np.random.default_rng(0)

    def tensor(n):
        chunk = rng.standard_normal(1 << 20).astype(np.float32)
        t = ops.createRaw([n])
        for off in range(0, n, chunk.size):
            m = min(chunk.size, n - off)
            check(lib.kth_upload(t.storeReference, off, chunk.ctypes.data_as(ctypes.c_void_p), m))
        return t

    if family == "binary_same_kernel" and op in binary:
        n = nbytes_per_launch // 12
        make = lambda: (tensor(n), tensor(n), ops.createRaw([n]))
        sh = abi.shape_array([n])
        run = lambda s: check(lib.kth_binary(binary[op], s[0].storeReference, sh, 1, s[1].storeReference, sh, 1, s[2].storeReference, sh, 1))
    elif family == "binary_bcast_vec_kernel_vv" and op in binary and "rows" in dims and "cols" in dims:
        rows, cols = dims["rows"], dims["cols"]                      # [rows, cols] (op) [cols]
        make = lambda: (tensor(rows * cols), tensor(cols), ops.createRaw([rows * cols]))
        sa, sb = abi.shape_array([rows, cols]), abi.shape_array([cols])
        run = lambda s: check(lib.kth_binary(binary[op], s[0].storeReference, sa, 2, s[1].storeReference, sb, 1, s[2].storeReference, sa, 2))
    elif family in ("unary_kernel", "unary_lds_kernel") and (op in unary or op in ("OpSquare", "OpIdentity")):
        n = nbytes_per_launch // 8
        make = lambda: (tensor(n), ops.createRaw([n]))
        if op in unary:
            run = lambda s: check(lib.kth_unary(unary[op], s[0].storeReference, s[1].storeReference, n))
        else:
            run = lambda s: check(lib.kth_scalar(Op.POW, s[0].storeReference, 2.0 if op == "OpSquare" else 1.0, 0, s[1].storeReference, n))
    elif family == "scalar_kernel" and op in binary:
        n = nbytes_per_launch // 8
        make = lambda: (tensor(n), ops.createRaw([n]))
        run = lambda s: check(lib.kth_scalar(binary[op], s[0].storeReference, 1.25, 0, s[1].storeReference, n))
    elif family == "reduce_cols_kernel" and op in ("RedSum", "RedMean") and "rows" in dims and "cols" in dims:
        rows, cols = dims["rows"], dims["cols"]
        make = lambda: (tensor(rows * cols), ops.createRaw([cols]))
        code = Op.SUM if op == "RedSum" else Op.MEAN
        run = lambda s: check(lib.kth_reduce_axis(code, s[0].storeReference, s[1].storeReference, 1, rows, cols))
    else:
        return None
    with ops.garbageCollector():
        group = [make() for _ in range(sets)]
        for s in group:
            run(s)
        ops.sync()
        ops.profileBegin()
        for _ in range(rounds):
            for s in group:
                run(s)
        prof = ops.profileEnd()
    launches, _, ms = prof.get(kernel, (0, 0, 0.0))
    return ms / launches * 1e3 if launches else None


def launch_floor(ops):
    """What one more tiny launch costs the stream when it is queued behind running work: the time of three full-size
    maps followed by k launches on 4096 floats, k = 0 and 16, divided out. No profiler and no event between the
    launches (an event pair or a tracer adds about 2.5 us to every back-to-back launch)."""
    import ctypes
    import numpy as np
    from kten_amd import abi
    from kten_amd.abi import Op, check
    lib = ops.lib
    n = 1 << 26
    with ops.garbageCollector():
        big, big2 = ops.createRaw([n]), ops.createRaw([n])
        check(lib.kth_fill(big.storeReference, 0, n, 1.5))
        a, b, c = (ops.createRaw([4096], np.full(4096, 0.25 * (i + 1), dtype=np.float32)) for i in range(3))
        sh = abi.shape_array([4096])
        best = {}
        for k in (0, 16, 0, 16, 0, 16):
            ops.sync()
            ops.timerBegin()
            for _ in range(3):
                check(lib.kth_unary(Op.NEG, big.storeReference, big2.storeReference, n))
            for _ in range(k):
                check(lib.kth_binary(Op.PLUS, a.storeReference, sh, 1, b.storeReference, sh, 1, c.storeReference, sh, 1))
            best[k] = min(best.get(k, 1e9), ops.timerEnd() * 1e3)
    return (best[16] - best[0]) / 16


def cpu_baseline(name, threads):
    """The CPU restatement of kten-jvm on a bounded sample of the same workload."""
    from kten_amd.host_mirror.workloads import WORKLOADS
    from oracle import jvm_oracle as jo
    wl = WORKLOADS[name]
    sample = {"cfg1": dict(wl.full_dims), "cfg2": dict(wl.full_dims), "cfg3": dict(wl.full_dims),
              "cfg4": dict(wl.full_dims), "cfg5": dict(wl.full_dims),
              "max_backward": dict(wl.full_dims), "softmax_ce": {"batch": 8192, "classes": 2048},
              "reduce_shapes": {"scale": 4}, "indexed_moves": {"rows": 4096, "cols": 4096},
              "indexed_skew": {"table": 50000, "width": 64, "k": 65536, "flat": 1 << 20, "rows": 1024, "cols": 8192, "short": 256}, "layout_shapes": {"scale": 8}, "unary_maps": {"n": 1 << 25}}.get(name, dict(wl.full_dims))
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
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": os.cpu_count() or 1, "threads": threads, "kind": "port",
            "sample": f"{name} at {sample} ({nbytes / 1e6:.0f} MB algorithmic, {dt:.2f} s): C restatement of kten-jvm "
                      "semantics, not kten-jvm itself; copy-producing ops and sum() single-threaded as in the "
                      f"reference, in-place ops and axis reductions on {threads} threads"}


def jvm_probe():
    """Whether the reference's own toolchain exists on this host: with it, kten-jvm itself could be timed beside the
    C restatement; without it the restatement is the only CPU baseline. Nothing is installed or run."""
    import shutil
    return {tool: shutil.which(tool) for tool in ("java", "kotlinc", "mvn")}


def time_steps(ops, step, steps, warmup):
    """W untimed steps, then exactly K steps between two HIP events on the library's stream, with a host wall clock
    around the same region and the stream drained on both sides: `ms_per_step` comes from that region alone. Median
    and minimum come from a second pass of K steps with an event after every step (an event costs the stream about
    2 us, which the first region therefore does not contain)."""
    for _ in range(warmup):
        step()
    ops.sync()
    m0 = ops.getMetrics()
    wall0 = time.perf_counter()
    ops.timerBegin()
    for _ in range(steps):
        step()
    issued_ms = (time.perf_counter() - wall0) * 1e3          # the host has issued everything; the stream may still be running
    total_ms = ops.timerEnd()                                # waits for the closing event
    ops.sync()
    wall_ms = (time.perf_counter() - wall0) * 1e3
    m = ops.getMetrics()
    ops.timerLap()
    for _ in range(steps):
        step()
        ops.timerLap()
    laps, _ = ops.timerLaps()
    ops.sync()
    laps.sort()
    median_ms = laps[len(laps) // 2] if len(laps) % 2 else 0.5 * (laps[len(laps) // 2 - 1] + laps[len(laps) // 2])
    return {"ms_per_step": total_ms / steps, "median_ms": median_ms, "min_ms": laps[0], "wall_ms": wall_ms / steps,
            "host_issue_ms": issued_ms / steps,
            "moved": (m["bytesMoved"] - m0["bytesMoved"]) / steps, "launches": (m["launches"] - m0["launches"]) / steps}


def kernel_events(ops, step, steps):
    """The same K steps again with every launch carrying its own start and stop events (the dispatch's own duration,
    as a kernel trace shows it): {kernel: (launches, bytes, ms)}. Kept out of the region `value` is computed from."""
    ops.profileBegin()
    ops.timerBegin()
    for _ in range(steps):
        step()
    ev_ms = ops.timerEnd()
    return ops.profileEnd(), ev_ms


def compiled_host_cfg1(steps, warmup):
    """cfg1 once more with the C++ mirror of the contract as the host (bench_host.cpp, built by __graft_entry__.build()):
    with four launches of a few microseconds per step, the Python mirror's issue rate is what bench.py's own cfg1 figure
    measures. Runs as a child process while this one is idle on the GPU; None (with the reason logged) when the program
    is not built."""
    import subprocess
    exe = os.path.join(ROOT, "bench_host")
    if not os.path.isfile(exe):
        log("bench_host is not built (python -c 'import __graft_entry__ as g; g.build()'): no compiled-host figure for cfg1")
        return None
    try:
        out = subprocess.run([exe, str(steps), str(warmup)], capture_output=True, text=True, timeout=120)
    except (OSError, subprocess.TimeoutExpired) as e:
        log(f"bench_host did not run: {e}")
        return None
    if out.returncode != 0:
        log(f"bench_host failed ({out.returncode}): {out.stderr.strip()[-300:]}")
        return None
    r = json.loads(out.stdout.strip().splitlines()[-1])
    r["frac_of_hbm_peak"] = round(r["GBps"] / HBM_PEAK_GBPS, 4)
    log(f"cfg1 with a compiled host: {r['ms_per_step']:.4f} ms/step, {r['GBps']:.0f} GB/s ({100 * r['frac_of_hbm_peak']:.1f} % of peak), "
        f"host issue {r['host_issue_ms_per_step']:.4f} ms/step")
    return r


def other_config(ops, name, steps, warmup):
    """One of the other BASELINE configurations for the same steps / warm-up: its step rate and its largest kernel."""
    from kten_amd.host_mirror.workloads import WORKLOADS
    wl = WORKLOADS[name]
    dims = wl.full_dims
    nbytes = wl.algorithmic_bytes(dims)
    inputs = wl.make_inputs(dims)
    step, resident = make_step(name, ops, inputs)
    r = time_steps(ops, step, steps, warmup)
    kernels, _ = kernel_events(ops, step, steps)
    for t in resident:
        t.release()
    ops.sync()
    counted = min(nbytes, r["moved"])
    gbps = counted / r["ms_per_step"] / 1e6
    dom, (n, b, ms) = max(kernels.items(), key=lambda kv: kv[1][2])
    log(f"{name}: {r['ms_per_step']:.4f} ms/step mean ({r['median_ms']:.4f} median, {r['min_ms']:.4f} min), {gbps:.0f} GB/s "
        f"({100 * gbps / HBM_PEAK_GBPS:.1f} % of peak), host issue {r['host_issue_ms']:.4f} ms/step; largest kernel {dom} {ms / n * 1e3:.1f} us")
    res = {"workload": wl.description, "algorithmic_bytes_per_step": nbytes, "moved_bytes_per_step": round(r["moved"]),
           "launches_per_step": r["launches"],
           "ms_per_step": round(r["ms_per_step"], 4), "ms_per_step_median": round(r["median_ms"], 4), "ms_per_step_min": round(r["min_ms"], 4),
           "host_issue_ms_per_step": round(r["host_issue_ms"], 4),
           "GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
           "dominant_kernel": dom, "dominant_avg_launch_us": round(ms / n * 1e3, 2), "dominant_GBps": round(b / ms / 1e6, 1),
           "dominant_frac": round(b / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    if name == "cfg1":
        res["compiled_host"] = compiled_host_cfg1(steps, warmup)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="cfg5",
                    choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "max_backward", "softmax_ce", "transpose", "permute",
                             "concat_mask", "broadcast_reuse", "broadcast_pairs", "sum0_alone", "batch_norm", "reduce_shapes", "indexed_moves", "indexed_skew", "layout_shapes", "unary_maps"])
    ap.add_argument("--cpu-baseline", dest="cpu", action="store_true", default=True)
    ap.add_argument("--no-cpu-baseline", dest="cpu", action="store_false")
    ap.add_argument("--no-kernel-events", dest="events", action="store_false", default=True,
                    help="skip the pass in which every launch carries its own start and stop events")
    ap.add_argument("--no-cold", dest="cold", action="store_false", default=True,
                    help="skip the dominant kernel's run over a rotation of untouched buffer sets")
    ap.add_argument("--no-copy-ceiling", dest="ceiling", action="store_false", default=True,
                    help="skip the device-to-device copy measurement")
    ap.add_argument("--math-mode", default="within_2_ulp", choices=["exact", "within_2_ulp"],
                    help="how the transcendental maps are evaluated (kth_set_math_mode); the library's default is within_2_ulp")
    ap.add_argument("--other-configs", dest="others", action="store_true", default=None,
                    help="after the headline workload, run cfg1-cfg4 for the same steps and warm-up and report them under "
                         "config.other_configs (the default when the headline is cfg5)")
    ap.add_argument("--no-other-configs", dest="others", action="store_false")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this backend drives one GPU; the hot path has no cross-GPU step. Run with --gpus 1.")
        sys.exit(2)
    if args.others is None:
        args.others = args.config == "cfg5"

    import kten_amd
    from kten_amd.host_mirror.workloads import WORKLOADS
    wl = WORKLOADS[args.config]
    dims = wl.full_dims
    nbytes = wl.algorithmic_bytes(dims)
    ops = kten_amd.platform(0)
    ops.setMathMode(args.math_mode)
    log(f"platform {ops.platformKey}: {ops.computeUnits} CUs, wave {ops.waveSize}, {ops.availableMemory / 2**30:.0f} GiB; math mode {args.math_mode}")
    log(f"workload {wl.name}: {wl.description}; {nbytes} algorithmic bytes per step")
    t0 = time.perf_counter()
    inputs = wl.make_inputs(dims)
    log(f"inputs generated in {time.perf_counter() - t0:.1f} s")
    step, resident = make_step(args.config, ops, inputs)

    r = time_steps(ops, step, args.steps, args.warmup)
    ms_per_step, median_ms, min_ms, wall_ms = r["ms_per_step"], r["median_ms"], r["min_ms"], r["wall_ms"]
    counted, launches = r["moved"], r["launches"]
    # `value` never counts bytes that were not moved: where the library folds a constant tensor into its
    # consumer (no fill written, no operand read) its launches move less than the reference's op list names,
    # and the rate is taken on what they moved. Where they move more (transposed copies), the op list stands.
    gbps = min(nbytes, counted) / ms_per_step / 1e6
    log(f"{args.steps} steps: {ms_per_step * args.steps:.3f} ms on the stream ({ms_per_step:.4f} ms/step mean, {median_ms:.4f} median, "
        f"{min_ms:.4f} min), {wall_ms:.4f} ms/step wall, host issue {r['host_issue_ms']:.4f} ms/step; {launches:.0f} launches/step; "
        f"library counted {counted:.0f} B/step (formula {nbytes})")

    kernels = {}
    if args.events:
        kernels, ev_ms = kernel_events(ops, step, args.steps)
        log(f"{args.steps} steps with per-launch events: {ev_ms:.3f} ms on the stream")

    roofline = None
    if kernels:
        log(f"{'kernel':48s} {'launches':>8s} {'avg us':>9s} {'GB/s':>9s} {'% time':>7s}")
        tot = sum(v[2] for v in kernels.values())
        for k, (n, b, ms) in sorted(kernels.items(), key=lambda kv: -kv[1][2]):
            log(f"{k:48s} {n:8d} {ms / n * 1e3:9.2f} {(b / ms / 1e6) if ms else 0:9.1f} {100 * ms / tot:7.1f}")
        dom, (n, b, ms) = max(kernels.items(), key=lambda kv: kv[1][2])
        achieved = b / ms / 1e6
        traffic = MEASURED_TRAFFIC_BYTES.get((args.config, dom))
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBPS, 4),
                    "traffic": traffic, "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
                    "bytes_per_launch": b // n, "avg_launch_us": round(ms / n * 1e3, 3), "launches": n,
                    "kernel_time_share": round(ms / tot, 4),
                    "achieved_context": "inside the op-at-a-time chain: the kernel reads what the previous launch wrote, part of "
                                        "which the 256 MB memory-side cache still holds"}
        if args.cold:
            cold_us = cold_probe(ops, dom, b // n, dims)
            if cold_us:
                roofline["achieved_cold"] = round((b // n) / cold_us / 1e3, 1)
                roofline["frac_cold"] = round((b // n) / cold_us / 1e3 / HBM_PEAK_GBPS, 4)
                roofline["cold_launch_us"] = round(cold_us, 3)
                roofline["cold_context"] = "8 buffer sets in rotation, 3 rounds: no operand was read or written by the 7 launches before"
                log(f"{dom} on untouched buffers: {cold_us:.2f} us ({roofline['achieved_cold']} GB/s) against {ms / n * 1e3:.2f} us in the chain")
            else:
                roofline["achieved_cold"] = None
    if roofline is not None and args.ceiling:
        floor_us = launch_floor(ops)
        roofline["launch_floor_us"] = round(floor_us, 2)
        roofline["launch_floor_means"] = ("stream time one more launch on 4096 floats adds when it is queued behind running kernels "
                                          "(slope of 3 full-size maps + k tiny launches, k = 0 and 16; no events between them)")
        log(f"one more tiny launch queued behind running work costs the stream {floor_us:.2f} us")
        d2d, own = ops.measureCopy(1 << 28, 10)
        roofline["copy_ceiling"] = {"hipMemcpyDtoD_GBps": round(d2d, 1), "copy_kernel_GBps": round(own, 1), "bytes_each_way": 1 << 30,
                                    "note": "read + written bytes over time, 10 copies of 1 GiB back to back on this GPU"}
        log(f"device-to-device copy of 1 GiB: hipMemcpyAsync {d2d:.0f} GB/s, the library's copy kernel {own:.0f} GB/s")

    line = {
        "metric": METRIC, "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "ms_per_step_median": round(median_ms, 4),
        "ms_per_step_min": round(min_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{wl.name}: {wl.description}", "algorithmic_bytes_per_step": nbytes,
                   "fused_lower_bound_bytes": wl.fused_lower_bound_bytes(dims) if wl.fused_lower_bound_bytes else None,
                   "launches_per_step": launches,
                   "math_mode": args.math_mode,
                   "fp32_elements_per_s": round(min(nbytes, counted) / 4 / (ms_per_step / 1e3)),
                   "fp32_elements_per_s_means": "the bytes of `value` / 4 per second: every fp32 value a launch reads or writes",
                   "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
                   "moved_bytes_per_step": round(counted),
                   "GBps_on_moved_bytes": round(counted / ms_per_step / 1e6, 1),
                   "value_means": "min(algorithmic_bytes_per_step, moved_bytes_per_step) / ms_per_step. moved_bytes_per_step is what "
                                  "the library's launches of one step read and wrote, summed from their own byte counts; "
                                  "algorithmic_bytes_per_step is the op-at-a-time total of the reference's op list. The two differ "
                                  "where the library does not write out a tensor that is one constant (a fresh zerosLike, the "
                                  "broadcast seed gradient) and hands the constant to the consumer's kernel, or does not make a copy "
                                  "that nobody writes to (pow 1 of a backward pass) (fewer bytes moved: "
                                  "the op-list total over time would count bytes that never crossed the memory bus and is not a "
                                  "bandwidth; ms_per_step shows the gain), and where it moves more than the op list names "
                                  "(transposed copies of a scatter along an outer axis)",
                   "wall_ms_per_step": round(wall_ms, 4),
                   "host_issue_ms_per_step": round(r["host_issue_ms"], 4),
                   "host_issue_means": "wall time the host took to issue the K timed steps (Python mirror of the autograd layer + "
                                       "ctypes), per step, before it waited for the stream: close to ms_per_step means that the "
                                       "stream was waiting for the host at times",
                   "median_and_min": "from a second pass of K steps with an event after every step",
                   "per_kernel_durations": "start and stop events carried by every launch (the dispatch's own duration), over a third pass of the same K steps"
                   if args.events else None},
        "roofline": roofline,
    }
    if args.config == "cfg1":
        ops.sync()
        line["config"]["compiled_host"] = compiled_host_cfg1(args.steps, args.warmup)
    if args.others:
        for t in resident:
            t.release()
        ops.sync()
        line["config"]["other_configs"] = {name: other_config(ops, name, args.steps, args.warmup)
                                           for name in ("cfg1", "cfg2", "cfg3", "cfg4") if name != args.config}
        line["config"]["other_configs_note"] = ("the other BASELINE configurations, same steps and warm-up, inputs resident: GBps = "
                                                "min(algorithmic, moved) bytes / ms_per_step; dominant_* from the start and stop events every "
                                                "launch of a further pass carries; no CPU baseline for them")
    if args.cpu:
        threads = min(16, os.cpu_count() or 1)
        log(f"timing the CPU restatement on {threads} threads of {os.cpu_count()} host cores ...")
        line["cpu_baseline"] = cpu_baseline(args.config, threads)
        line["cpu_baseline"]["jvm_available"] = jvm_probe()
        line["cpu_baseline"]["oracle_used"] = ("the C restatement (kind \"port\"): " + ("a JVM toolchain is on this host but the reference's Maven "
                                               "dependencies are not, so kten-jvm itself was not built or timed"
                                               if all(line["cpu_baseline"]["jvm_available"].values()) else
                                               "java / kotlinc / mvn are not all present on this host, kten-jvm itself cannot be built or timed here"))
        log(f"cpu baseline: {line['cpu_baseline']['value']} GB/s; jvm toolchain: {line['cpu_baseline']['jvm_available']}")
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
