"""The five benchmark configurations through the `Tensor` API on the HIP backend.

Scaled-down shapes are compared with the CPU checker running the very same graph.
Full benchmark shapes are checked through what does not need the serial CPU restatement
of every pass: numpy closed forms for single-rounding ops, float64 references for the
reductions (plus the checker's own error on the reductions, which it can do in seconds),
argmax against numpy on tie-free data."""
import numpy as np
import pytest

from kten_amd.host_mirror.workloads import WORKLOADS, layout_shapes_at, reduce_shapes_at
from oracle import jvm_oracle as jo
from parity import assert_bits_equal, assert_reduction_close, assert_ulp_close, ulp_distance

pytestmark = pytest.mark.gpu

SMALL = {"cfg1": {"rows": 96, "cols": 200}, "cfg2": {"n": 100003}, "cfg3": {"rows": 300, "cols": 520},
         "cfg4": {"n": 6, "c": 16, "h": 12, "w": 20}, "cfg5": {"rows": 512, "cols": 384}}


def run_both(name, dims, gc):
    wl = WORKLOADS[name]
    inputs = wl.make_inputs(dims)
    got = {k: v.toArray() for k, v in wl.run(gc, inputs).items()}
    want = {k: v.toArray() for k, v in wl.run(jo.JvmOracleOperations(), inputs).items()}
    return inputs, got, want


def test_cfg1_small(gc):
    inp, got, want = run_both("cfg1", SMALL["cfg1"], gc)
    assert_bits_equal(got["y"], want["y"], "y")
    assert_reduction_close(got["s"], [jo.sum_all_f64(want["y"])], want["s"], "s")


@pytest.mark.parametrize("mode", ["exact", "within_2_ulp"])
def test_cfg2_small(mode, gc):
    with gc.mathMode(mode):
        inp, got, want = run_both("cfg2", SMALL["cfg2"], gc)
    if mode == "exact":
        # exp and log return the checker's floats, so z = e + l is the checker's too
        assert_ulp_close(got["z"], want["z"], 0, "z")
        return
    # z = e + l with each addend within 2 ulp of the checker's (the per-op bars are checked in test_gpu_elementwise and
    # test_gpu_all_floats): z is within 2 ulp of each addend plus its own rounding of the checker's z, which where the
    # addends cancel is many ulps of z itself
    x = inp["x"]
    e = jo.unary("exp", (-(x * x)) + np.float32(0.0))
    l = jo.unary("log", np.abs(x) + np.float32(1e-3))
    bound = 2.0 * np.spacing(np.abs(e)).astype(np.float64) + 2.0 * np.spacing(np.abs(l)).astype(np.float64) \
        + np.spacing(np.abs(want["z"])).astype(np.float64)
    err = np.abs(got["z"].astype(np.float64) - want["z"].astype(np.float64))
    assert np.all(err <= bound), f"z: {np.count_nonzero(err > bound)} values outside the bound of 2 ulp per addend"


def test_cfg3_small(gc):
    inp, got, want = run_both("cfg3", SMALL["cfg3"], gc)
    x = inp["x"]
    for axis in (0, 1):
        ref, _ = jo.axis_sum_f64(x, axis)
        assert_reduction_close(got[f"sum{axis}"], ref, want[f"sum{axis}"], f"sum{axis}")
        assert_reduction_close(got[f"mean{axis}"], ref / x.shape[axis], want[f"mean{axis}"], f"mean{axis}")
    assert_bits_equal(got["max1"], want["max1"], "max1")
    assert_bits_equal(got["argmax1"], want["argmax1"], "argmax1")


def test_cfg4_small(gc):
    inp, got, want = run_both("cfg4", SMALL["cfg4"], gc)
    assert_bits_equal(got["out"], want["out"], "out")
    ref = want["out"].astype(np.float64).sum((0, 2, 3), keepdims=True)
    n = want["out"].size // want["out"].shape[1]
    assert got["sum"].shape == (1, SMALL["cfg4"]["c"], 1, 1)
    assert_reduction_close(got["sum"], ref, want["sum"], "sum(0,2,3)")
    assert_reduction_close(got["mean"], ref / n, want["mean"], "mean(0,2,3)")


def test_cfg5_small(gc):
    inp, got, want = run_both("cfg5", SMALL["cfg5"], gc)
    x, w, b = (inp[k].astype(np.float64) for k in ("x", "w", "b"))
    # the reference values follow the fp32 intermediates the graph really produces
    t32 = (inp["x"] * inp["w"]) + inp["b"]
    g32 = (np.float32(2.0) * np.ones_like(t32)) * t32
    assert_reduction_close(got["loss"], [(t32 * t32).astype(np.float64).sum()], want["loss"], "loss")
    assert_reduction_close(got["grad_w"], (g32 * inp["x"]).astype(np.float64).sum(0), want["grad_w"], "grad w")
    assert_reduction_close(got["grad_b"], [g32.astype(np.float64).sum()], want["grad_b"], "grad b")
    # and are close to the exact mathematics
    t = x * w + b
    np.testing.assert_allclose(got["loss"], [(t * t).sum()], rtol=1e-5)
    np.testing.assert_allclose(got["grad_w"], (2 * t * x).sum(0), rtol=1e-4, atol=1e-4)


def test_cfg5_raw_op_sequence_intermediates_bit_exact(gc):
    """The elementwise passes of the forward and backward graph, op by op (bit-exact)."""
    inp = WORKLOADS["cfg5"].make_inputs(SMALL["cfg5"])
    cpu = jo.JvmOracleOperations()
    outs = []
    for ops in (gc, cpu):
        x = ops.createRaw(list(inp["x"].shape), inp["x"]); w = ops.createRaw(list(inp["w"].shape), inp["w"])
        b = ops.createRaw([1], inp["b"])
        t1 = x * w; t2 = t1 + b; t3 = t2.pow(2.0)
        g = ops.createRaw([1], [1.0]).broadcastTo(t3.shape)
        ig = g * 2.0
        ig *= t2.pow(1.0)
        gw = ig * x; gx = ig * w
        outs.append([t.toArray() for t in (t1, t2, t3, g, ig, gw, gx)])
    for name, a, c in zip(("x*w", "+b", "pow 2", "broadcast", "*2 *= pow1", "g*x", "g*w"), *outs):
        assert_bits_equal(a, c, name)


def test_cfg5_gradient_accumulates_over_two_backward_passes(gc):
    from kten_amd.host_mirror.workloads import cfg5_setup, cfg5_step
    inp = WORKLOADS["cfg5"].make_inputs({"rows": 64, "cols": 128})
    x, w, b = cfg5_setup(gc, inp)
    cfg5_step(x, w, b)
    g1 = w.grad().toArray().copy()
    cfg5_step(x, w, b)
    np.testing.assert_allclose(w.grad().toArray(), 2 * g1, rtol=1e-6)
    w.zeroGrad()
    assert not w.grad().toArray().any()


# ---------------------------------------------------------------- full benchmark shapes

def test_cfg1_full(gc):
    wl = WORKLOADS["cfg1"]
    inp, got, want = run_both("cfg1", wl.full_dims, gc)
    assert_bits_equal(got["y"], want["y"], "y")
    assert_bits_equal(got["y"], (inp["x"] + inp["b"]) * inp["x"], "y vs numpy")
    ref = jo.sum_all_f64(want["y"])
    assert_reduction_close(got["s"], [ref], want["s"], "s")
    assert abs(float(got["s"][0]) - ref) <= 1e-5 * abs(ref)


def test_cfg2_full(gc):
    wl = WORKLOADS["cfg2"]
    inp = wl.make_inputs(wl.full_dims)
    x = inp["x"]
    xt = gc.create([x.size], False, x)
    sq = xt ** 2
    assert_bits_equal(sq.toArray(), x * x, "pow 2")
    neg = -sq
    assert_bits_equal(neg.toArray(), (-(x * x)) + np.float32(0.0), "-(x pow 2)")
    ab = xt.abs() + 1e-3
    assert_bits_equal(ab.toArray(), np.abs(x) + np.float32(1e-3), "abs + 1e-3")
    e, l = neg.exp(), ab.log()
    z = (e + l).toArray()
    ea, la = e.toArray(), l.toArray()
    assert_bits_equal(z, ea + la, "e + l")
    # exp / log against f64 numpy on the whole tensor (numpy's f64 routines agree with the
    # checker's libm to the last f64 bit or nearly so), and against the checker itself on a slice
    e_ref = np.exp((-(x * x)).astype(np.float64)).astype(np.float32)
    l_ref = np.log((np.abs(x) + np.float32(1e-3)).astype(np.float64)).astype(np.float32)
    assert ulp_distance(ea, e_ref).max() <= 2 and ulp_distance(la, l_ref).max() <= 2
    sl = slice(12345, 12345 + (1 << 20))
    assert_ulp_close(ea[sl], jo.unary("exp", (-(x[sl] * x[sl])) + np.float32(0.0)), 2, "exp slice")
    assert_ulp_close(la[sl], jo.unary("log", np.abs(x[sl]) + np.float32(1e-3)), 2, "log slice")


def test_cfg3_full(gc):
    wl = WORKLOADS["cfg3"]
    inp = wl.make_inputs(wl.full_dims)
    x = inp["x"]
    got = {k: v.toArray() for k, v in wl.run(gc, inp).items()}
    jo.set_threads(16)
    try:
        for axis in (0, 1):
            ref, _ = jo.axis_sum_f64(x, axis)
            jvm_sum = jo.aggregate("sum", x, axis); jvm_mean = jo.aggregate("mean", x, axis)
            e, je = assert_reduction_close(got[f"sum{axis}"], ref, jvm_sum, f"sum{axis}")
            print(f"sum axis {axis}: max |err| {e:.3e} (kten-jvm restatement {je:.3e})")
            assert_reduction_close(got[f"mean{axis}"], ref / x.shape[axis], jvm_mean, f"mean{axis}")
        assert_bits_equal(got["max1"], jo.aggregate("max", x, 1).reshape(-1), "max1")
        assert_bits_equal(got["argmax1"], jo.aggregate("arg_max", x, 1).reshape(-1), "argmax1")
    finally:
        jo.set_threads(1)
    assert_bits_equal(got["max1"], x.max(1), "max1 vs numpy")
    assert (got["argmax1"] == np.argmax(x, 1)).all()


def test_cfg4_full(gc):
    wl = WORKLOADS["cfg4"]
    inp = wl.make_inputs(wl.full_dims)
    got = {k: v.toArray() for k, v in wl.run(gc, inp).items()}
    out = inp["act"] * inp["scale"] + inp["bias"]            # numpy: one rounding per op, like the JVM
    assert_bits_equal(got["out"], out, "out")
    ref = out.astype(np.float64).sum((0, 2, 3), keepdims=True)
    cpu = jo.JvmOracleOperations()
    jo.set_threads(16)
    try:
        o = cpu.createRaw(list(out.shape), out)
        jvm_sum = o.sum(0, True).sum(2, True).sum(3, True).toArray()
        jvm_mean = o.mean(0, True).mean(2, True).mean(3, True).toArray()
    finally:
        jo.set_threads(1)
    assert got["sum"].shape == (1, 128, 1, 1)
    assert_reduction_close(got["sum"], ref, jvm_sum, "sum(0,2,3)")
    assert_reduction_close(got["mean"], ref / (64 * 56 * 56), jvm_mean, "mean(0,2,3)")


def test_cfg5_full(gc):
    wl = WORKLOADS["cfg5"]
    inp = wl.make_inputs(wl.full_dims)
    got = {k: v.toArray() for k, v in wl.run(gc, inp).items()}
    x32, w32, b32 = inp["x"], inp["w"], inp["b"]
    t32 = (x32 * w32) + b32                                    # fp32 intermediates as the graph makes them
    g32 = np.float32(2.0) * t32                                # (1 * 2f) * (t pow 1f)
    loss_ref = np.square(t32).astype(np.float64).sum()
    gw_ref = np.einsum("ij,ij->j", g32.astype(np.float64), x32.astype(np.float64))
    gb_ref = g32.astype(np.float64).sum()
    # kten-jvm's own serial-float results for the same reductions
    jo.set_threads(16)
    try:
        jvm_loss = jo.sum_all(np.square(t32))
        gx = g32 * x32
        jvm_gw = jo.aggregate("sum", gx, 0).reshape(-1)
        jvm_gb = jo.aggregate("sum", jo.aggregate("sum", g32, 0).reshape(-1), 0)
    finally:
        jo.set_threads(1)
    e, je = assert_reduction_close(got["loss"], [loss_ref], [jvm_loss], "loss")
    print(f"loss {got['loss'][0]!r}: |err| {e:.3e} (kten-jvm restatement {je:.3e})")
    assert_reduction_close(got["grad_w"], gw_ref, jvm_gw, "grad w")
    assert_reduction_close(got["grad_b"], [gb_ref], jvm_gb, "grad b")
    assert abs(float(got["loss"][0]) - loss_ref) <= 1e-5 * loss_ref


@pytest.mark.parametrize("dims", [{"n": 7, "t": 400, "h": 1020, "p": 6, "q": 3, "r": 4, "s": 40000}, None], ids=["small", "full"])
def test_broadcast_reuse(dims, gc):
    """Broadcast binary ops whose repeating operand is megabytes large (the tiles of the output are then ordered for
    reuse in L2): bit for bit against numpy's broadcasting."""
    wl = WORKLOADS["broadcast_reuse"]
    inp = wl.make_inputs(dims or wl.full_dims)
    gc.profileBegin()
    out = wl.run(gc, inp)
    launched = " ".join(gc.profileEnd().keys())
    assert "_chunked" in launched, launched
    assert_bits_equal(out["sum"].toArray(), inp["x"] + inp["y"], "x + y")
    assert_bits_equal(out["product"].toArray(), inp["a"] * inp["b"], "a * b")


def _check_reduce_shapes(inp, got, scale):
    for i, (shape, axis, op) in enumerate(reduce_shapes_at({"scale": scale})):
        x = inp[f"x{i}"]
        res = got[f"{op}{i}"]
        if op in ("sum", "mean"):
            ref, _ = jo.axis_sum_f64(x, axis)
            want = jo.aggregate(op, x, axis).reshape(-1)
            assert_reduction_close(res.reshape(-1), ref / (shape[axis] if op == "mean" else 1), want, f"{op} {shape}")
        else:
            code = {"max": "max", "argMax": "arg_max"}[op]
            assert_bits_equal(res.reshape(-1), jo.aggregate(code, x, axis).reshape(-1), f"{op} {shape}")


def test_reduce_shapes_small(gc):
    wl = WORKLOADS["reduce_shapes"]
    inp = wl.make_inputs({"scale": 64})
    got = {k: v.toArray() for k, v in wl.run(gc, inp).items()}
    _check_reduce_shapes(inp, got, 64)


def test_reduce_shapes_full(gc):
    """The five geometries at 2^26 elements each against the checker running on 16 threads."""
    wl = WORKLOADS["reduce_shapes"]
    inp = wl.make_inputs(wl.full_dims)
    got = {k: v.toArray() for k, v in wl.run(gc, inp).items()}
    jo.set_threads(16)
    try:
        _check_reduce_shapes(inp, got, 1)
    finally:
        jo.set_threads(1)


@pytest.mark.parametrize("dims", [{"rows": 300, "cols": 520}, {"rows": 16384, "cols": 4096}], ids=["small", "full"])
def test_indexed_moves(dims, gc):
    """Bit-exact against the checker, full size included: gather, assignment with the last entry
    winning, adds in index order, row selection and row accumulation."""
    wl = WORKLOADS["indexed_moves"]
    inp = wl.make_inputs(dims)
    got = {k: v.toArray() for k, v in wl.run(gc, inp).items()}
    want = {k: v.toArray() for k, v in wl.run(jo.JvmOracleOperations(), inp).items()}
    for k in ("gathered", "assigned", "added", "selected", "summed"):
        assert_bits_equal(got[k], want[k], k)
    assert_bits_equal(got["gathered"], np.take_along_axis(inp["x"], inp["along_cols"].astype(np.int64), 1), "gather vs numpy")
    assert_bits_equal(got["selected"], inp["x"][inp["row_list"].astype(np.int64)], "indexSelect vs numpy")


@pytest.mark.parametrize("dims", [{"table": 300, "width": 20, "k": 5000, "flat": 4096, "rows": 64, "cols": 9000, "short": 40},
                                  {"table": 50000, "width": 256, "k": 262144, "flat": 1 << 22, "rows": 8192, "cols": 8192, "short": 256}],
                         ids=["small", "full"])
def test_indexed_skew(dims, gc):
    """Bit-exact against the checker, full size included: rows and elements that a large share of the entries name (the adds
    into them in index order), a flat tensor with twice as many entries as elements, index rows far shorter than the target's."""
    wl = WORKLOADS["indexed_skew"]
    inp = wl.make_inputs(dims)
    got = {k: v.toArray() for k, v in wl.run(gc, inp).items()}
    jo.set_threads(16)
    try:
        want = {k: v.toArray() for k, v in wl.run(jo.JvmOracleOperations(), inp).items()}
    finally:
        jo.set_threads(1)
    for k in ("table_grad", "histogram", "latest", "row_sums", "placed"):
        assert_bits_equal(got[k], want[k], k)
    last = np.zeros(dims["flat"], np.float32)
    last[inp["bins"].astype(np.int64)] = inp["weights"]                  # numpy assigns in order: the last entry stays
    assert_bits_equal(got["latest"], last, "scatter on a flat tensor vs numpy")


@pytest.mark.parametrize("scale", [64, 1], ids=["small", "full"])
def test_layout_shapes(scale, gc):
    """Permutes and the range get against numpy (which the checker is pinned to for these moves), bit for bit."""
    wl = WORKLOADS["layout_shapes"]
    dims = {"scale": scale}
    inp = wl.make_inputs(dims)
    got = wl.run(gc, inp)
    shapes, _ = layout_shapes_at(dims)
    for i, (shape, perm) in enumerate(shapes):
        assert_bits_equal(got[f"permuted{i}"].toArray(), np.transpose(inp[f"x{i}"], perm), f"permute {shape} {perm}")
    assert_bits_equal(got["box"].toArray(), inp["boxed"][:, 1:inp["boxed"].shape[1] - 2], "range get")


@pytest.mark.parametrize("n", [70001, 1 << 26], ids=["small", "full"])
def test_unary_maps(n, gc):
    """The transcendental maps at the benchmark size: at most 2 ulp from the checker on a slice (or the whole
    small tensor), and on the whole tensor from numpy's float64 routines rounded once, which agree with the
    checker's libm to the last float64 bit or nearly so."""
    wl = WORKLOADS["unary_maps"]
    inp = wl.make_inputs({"n": n})
    got = wl.run(gc, inp)
    x, p = inp["x"], inp["p"]
    sl = slice(0, n) if n < (1 << 20) else slice(54321, 54321 + (1 << 20))
    f64 = {"tanh": np.tanh, "sinh": np.sinh, "cosh": np.cosh, "sin": np.sin, "cos": np.cos, "tan": np.tan,
           "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan, "sigmoid": lambda v: 1.0 / (1.0 + np.exp(-v))}
    for name, fn in f64.items():
        res = got[name].toArray()
        assert_ulp_close(res[sl], jo.unary(name, x[sl]), 2, name + " against the checker")
        assert ulp_distance(res, fn(x.astype(np.float64)).astype(np.float32)).max() <= 2, name + " against float64"
        gc.release(got[name])
    res = got["pow1.5"].toArray()
    assert_ulp_close(res[sl], jo.binary("pow", p[sl], np.float32(1.5)), 2, "pow against the checker")
    assert ulp_distance(res, np.power(p.astype(np.float64), 1.5).astype(np.float32)).max() <= 2, "pow against float64"
