"""The five benchmark / parity workloads, written against the `Tensor` API exactly as a
kten user would write them, so that the backend sees the raw-op sequences the reference's
autograd layer emits. Each workload has: its input shapes, the seeded inputs, the
computation, and the algorithmic bytes of the raw-op sequence (every operand counted once
at its un-broadcast size plus the output, 4 bytes each, op at a time; in-place targets
are counted as read + write).

`dims` lets tests run the same workload at a size a CPU checker finishes in seconds.
"""
from dataclasses import dataclass
from typing import Callable, Dict, List

import numpy as np

from .inputs import SplitMix64


@dataclass
class Workload:
    name: str
    description: str
    full_dims: Dict[str, int]
    make_inputs: Callable[[Dict[str, int]], Dict[str, np.ndarray]]
    run: Callable            # (ops, inputs) -> dict name -> Tensor
    algorithmic_bytes: Callable[[Dict[str, int]], int]
    # Bytes a single fused kernel would have to move for the same results (inputs once, outputs once): context
    # for the op-at-a-time figure, which is what the raw-tensor contract makes a backend do.
    fused_lower_bound_bytes: Callable[[Dict[str, int]], int] = None


# ---- 1: broadcast + full reduction ------------------------------------------------------

def _in1(d):
    g = SplitMix64(0)
    return {"x": g.uniform([d["rows"], d["cols"]], -1.0, 1.0), "b": g.uniform([d["cols"]], -1.0, 1.0)}


def _run1(ops, inp):
    x = ops.create(list(inp["x"].shape), False, inp["x"])
    b = ops.create(list(inp["b"].shape), False, inp["b"])
    y = (x + b) * x
    s = y.sum()
    return {"y": y, "s": s}


def _bytes1(d):
    n, k = d["rows"] * d["cols"], d["cols"]
    return 4 * (6 * n + k + 1)


# ---- 2: unary chain -----------------------------------------------------------------------

def _in2(d):
    return {"x": SplitMix64(1).normal([d["n"]])}


def _run2(ops, inp):
    x = ops.create(list(inp["x"].shape), False, inp["x"])
    z = (-(x ** 2)).exp() + (x.abs() + 1e-3).log()
    return {"z": z}


def _bytes2(d):
    return 4 * 17 * d["n"]


# ---- 3: axis reductions -------------------------------------------------------------------

def _in3(d):
    return {"x": SplitMix64(2).normal([d["rows"], d["cols"]])}


def _run3(ops, inp):
    x = ops.create(list(inp["x"].shape), False, inp["x"])
    return {"sum0": x.sum(0), "sum1": x.sum(1), "mean0": x.mean(0), "mean1": x.mean(1),
            "max1": x.max(1), "argmax1": x.argMax(1)}


def _bytes3(d):
    n = d["rows"] * d["cols"]
    return 4 * (2 * (n + d["cols"]) + 4 * (n + d["rows"]))


# ---- 4: channel broadcast + reduce over (0, 2, 3) ------------------------------------------

def _in4(d):
    g = SplitMix64(3)
    n, c, h, w = d["n"], d["c"], d["h"], d["w"]
    return {"act": g.uniform([n, c, h, w], -2.0, 2.0), "scale": g.uniform([1, c, 1, 1], 0.5, 1.5),
            "bias": g.uniform([1, c, 1, 1], -0.1, 0.1)}


def _run4(ops, inp):
    act = ops.create(list(inp["act"].shape), False, inp["act"])
    scale = ops.create(list(inp["scale"].shape), False, inp["scale"])
    bias = ops.create(list(inp["bias"].shape), False, inp["bias"])
    out = act * scale + bias
    # the axis order in which the reference reduces a gradient to a [1,C,1,1] operand
    s = out.sum(0, True).sum(2, True).sum(3, True)
    m = out.mean(0, True).mean(2, True).mean(3, True)
    return {"out": out, "sum": s, "mean": m}


def _bytes4(d):
    n, c, h, w = d["n"], d["c"], d["h"], d["w"]
    full = n * c * h * w
    chain = (full + c * h * w) + (c * h * w + c * w) + (c * w + c)
    return 4 * (4 * full + 2 * c + 2 * chain)


# ---- 5: autograd forward + backward --------------------------------------------------------

def _in5(d):
    g = SplitMix64(4)
    return {"x": g.normal([d["rows"], d["cols"]]), "w": g.uniform([d["cols"]], -0.05, 0.05),
            "b": g.uniform([1], -0.05, 0.05)}


def cfg5_setup(ops, inp):
    x = ops.create(list(inp["x"].shape), False, inp["x"])
    w = ops.create(list(inp["w"].shape), True, inp["w"])
    b = ops.create(list(inp["b"].shape), True, inp["b"])
    return x, w, b


def cfg5_step(x, w, b):
    loss = (((x * w) + b) ** 2).sum()
    loss.backward()
    return loss


def _run5(ops, inp):
    x, w, b = cfg5_setup(ops, inp)
    loss = cfg5_step(x, w, b)
    return {"loss": loss, "grad_w": w.grad(), "grad_b": b.grad()}


def _bytes5(d):
    m, c = d["rows"] * d["cols"], d["cols"]
    big = 22 * m                      # F1-F4, B1-B8: the passes over [rows, cols]
    small = (2 * c                    # w read by x*w and g*w
             + 1                      # b read by +b
             + 1 + 1 + 1              # sum() output, the [1] seed gradient written, then read by broadcastTo
             + c + (c + 1)            # sum(0) -> [cols] for b, then sum(0, keep) -> [1]
             + c                      # sum(0) -> [cols] for w
             + 3 * c + 3)             # gradient += g on w and b (read, read, write)
    return 4 * (big + small)


# ---- next rows: Max with its scatter backward, softmax cross entropy --------------------------

def _in_max(d):
    return {"x": SplitMix64(5).normal([d["rows"], d["cols"]])}


def _run_max(ops, inp):
    x = ops.create(list(inp["x"].shape), True, inp["x"])
    m = x.max(-1)
    m.sum().backward()
    return {"max": m, "grad_x": x.grad()}


def _bytes_max(d):
    n, r = d["rows"] * d["cols"], d["rows"]
    # max + argMax (2(N+R)), sum() (R+1), seed (1), broadcastTo (1+R), zerosLike (N), scatter (3R), gradient += (3N)
    return 4 * (6 * n + 7 * r + 3)


def _in_sce(d):
    g = SplitMix64(6)
    logits = g.normal([d["batch"], d["classes"]])
    labels = np.floor(g.uniform([d["batch"]], 0.0, 1.0) * np.float32(d["classes"])).clip(0, d["classes"] - 1)
    return {"logits": logits, "targets": labels.astype(np.float32)}


def _run_sce(ops, inp):
    logits = ops.create(list(inp["logits"].shape), True, inp["logits"])
    targets = ops.create(list(inp["targets"].shape), False, inp["targets"])
    loss = logits.softmaxCrossEntropy(targets)
    loss.backward()
    return {"loss": loss, "grad_logits": logits.grad()}


def _bytes_sce(d):
    n, b = d["batch"] * d["classes"], d["batch"]
    # 15N + 12B + 1 forward, 9N + 2B + 1 backward, 2B for the copy made by targets.unsqueeze(-1)
    return 4 * (24 * n + 16 * b + 2)


# ---- layout movers -------------------------------------------------------------------------

def _in_tr(d):
    return {"x": SplitMix64(7).uniform([d["rows"], d["cols"]], -1.0, 1.0)}


def _run_tr(ops, inp):
    x = ops.create(list(inp["x"].shape), False, inp["x"])
    return {"xt": x.transpose(0, 1)}


def _bytes_tr(d):
    return 4 * 2 * d["rows"] * d["cols"]


def _in_perm(d):
    return {"x": SplitMix64(8).uniform([d["n"], d["c"], d["h"], d["w"]], -1.0, 1.0)}


def _run_perm(ops, inp):
    x = ops.create(list(inp["x"].shape), False, inp["x"])
    nhwc = x.permute(0, 2, 3, 1)
    return {"nhwc": nhwc, "back": nhwc.permute(0, 3, 1, 2)}


def _bytes_perm(d):
    return 4 * 4 * d["n"] * d["c"] * d["h"] * d["w"]


def _in_cat(d):
    g = SplitMix64(9)
    return {"a": g.uniform([d["rows"], d["left"]], -1.0, 1.0), "b": g.uniform([d["rows"], d["right"]], -1.0, 1.0),
            "mask": (g.uniform([d["left"] + d["right"]], 0.0, 1.0) < 0.25).astype(np.float32)}


def _run_cat(ops, inp):
    from .autograd import concat
    from .shape_functions import ALL
    a = ops.create(list(inp["a"].shape), False, inp["a"])
    b = ops.create(list(inp["b"].shape), False, inp["b"])
    mask = ops.create(list(inp["mask"].shape), False, inp["mask"])
    cat = concat(a, b, axis=1)
    masked = cat.maskedFill(mask, 0.0)
    right = masked[ALL, (inp["a"].shape[1], -1)]
    masked[(0, -1), (0, inp["a"].shape[1] - 1)] = 1.0
    return {"cat": cat, "masked": masked, "right": right}


def _bytes_cat(d):
    n, la, lb = d["rows"] * (d["left"] + d["right"]), d["rows"] * d["left"], d["rows"] * d["right"]
    # concat: two range sets (2 la + 2 lb); maskedFill (2 n + mask); range get (2 lb); range fill (la)
    return 4 * (2 * n + 2 * n + (d["left"] + d["right"]) + 2 * lb + la)


# ---- broadcast of operands that repeat and are too large for one L2 -------------------------------

def _in_reuse(d):
    g = SplitMix64(16)
    return {"x": g.uniform([d["n"], d["t"], d["h"]], -1.0, 1.0), "y": g.uniform([1, d["t"], d["h"]], -1.0, 1.0),
            "a": g.uniform([1, d["q"], d["r"], d["s"]], -1.0, 1.0), "b": g.uniform([d["p"], 1, d["r"], d["s"]], -1.0, 1.0)}


def _run_reuse(ops, inp):
    t = {k: ops.create(list(v.shape), False, v) for k, v in inp.items()}
    return {"sum": t["x"] + t["y"], "product": t["a"] * t["b"]}


def _bytes_reuse(d):
    x, y = d["n"] * d["t"] * d["h"], d["t"] * d["h"]
    a, b, out = d["q"] * d["r"] * d["s"], d["p"] * d["r"] * d["s"], d["p"] * d["q"] * d["r"] * d["s"]
    return 4 * (2 * x + y + a + b + out)


# ---- two operands that are both smaller than the output, in four dims or with a dim both keep ----

# (a shape, b shape) at scale 1; the first dim of each pair's output is what `scale` divides for smaller runs
BROADCAST_PAIRS = [([1, 196, 1, 2], [4, 1, 20452, 1]), ([246, 1, 4, 1], [1, 206, 4, 165]),
                   ([111, 5496, 1], [111, 1, 55]), ([2481, 4, 1, 21], [1, 4, 161, 1])]


def broadcast_pairs_at(scale):
    def shrink(shape, lead):
        s = list(shape)
        if s[lead] > 1:
            s[lead] = max(2, s[lead] // scale)
        return s
    out = []
    for k, (sa, sb) in enumerate(BROADCAST_PAIRS):
        lead = {0: 2, 1: 0, 2: 1, 3: 0}[k]          # the long dim of the pair: 20452, 246, 5496, 2481
        out.append((shrink(sa, lead), shrink(sb, lead)))
    return out


def _in_pairs(d):
    g = SplitMix64(17)
    inp = {}
    for k, (sa, sb) in enumerate(broadcast_pairs_at(d["scale"])):
        inp[f"a{k}"] = g.uniform(sa, -1.0, 1.0); inp[f"b{k}"] = g.uniform(sb, 0.5, 1.5)
    return inp


def _run_pairs(ops, inp):
    t = {k: ops.create(list(v.shape), False, v) for k, v in inp.items()}
    return {"minus0": t["a0"] - t["b0"], "div1": t["a1"] / t["b1"], "times2": t["a2"] * t["b2"], "plus3": t["a3"] + t["b3"]}


def _bytes_pairs(d):
    total = 0
    for sa, sb in broadcast_pairs_at(d["scale"]):
        out = int(np.prod(np.broadcast_shapes(tuple(sa), tuple(sb))))
        total += int(np.prod(sa)) + int(np.prod(sb)) + out
    return 4 * total


# ---- the column reduction of cfg5 by itself -------------------------------------------------------

def _in_sum0(d):
    return {"x": SplitMix64(4).normal([d["rows"], d["cols"]])}


def _run_sum0(ops, inp):
    x = ops.create(list(inp["x"].shape), False, inp["x"])
    return {"sum0": x.sum(0)}


# ---- fused batch normalisation ------------------------------------------------------------------

def _in_bn(d):
    g = SplitMix64(10)
    n, c, h, w = d["n"], d["c"], d["h"], d["w"]
    return {"x": g.normal([n, c, h, w]) * np.float32(1.5) + np.float32(0.25), "grad_out": g.normal([n, c, h, w]),
            "gamma": g.uniform([c], 0.5, 1.5), "beta": g.uniform([c], -0.1, 0.1),
            "running_mean": np.zeros([c], dtype=np.float32), "running_var": np.ones([c], dtype=np.float32)}


def _run_bn(ops, inp):
    from .autograd import NoGradVariable
    raw = {k: ops.create(list(v.shape), False, v).getRawValue() for k, v in inp.items()}
    op = ops.batchNorm(1, 0.1, 1e-5, True)
    out, mean, std = op.calculateOutput(raw["x"], raw["running_mean"], raw["running_var"], raw["gamma"], raw["beta"])
    grad_in, grad_gamma, grad_beta = op.calculateGrads(raw["x"], raw["running_mean"], raw["running_var"], mean, std,
                                                       raw["gamma"], raw["grad_out"], True, True, True)
    res = {"out": out, "mean": mean, "std": std, "grad_in": grad_in, "grad_gamma": grad_gamma, "grad_beta": grad_beta}
    return {k: NoGradVariable(ops, v) for k, v in res.items()}


def _bytes_bn(d):
    full, c = d["n"] * d["c"] * d["h"] * d["w"], d["c"]
    # forward: statistics (read x), normalise (read x, write out); backward: sums (read x and gradOut),
    # input gradient (read x and gradOut, write); per-channel operands and results: 8 C forward, 6 C backward
    return 4 * (8 * full + 14 * c)


# ---- reductions over the geometries that have kernels of their own ------------------------------

# (shape at scale 1, axis, op): slabs staged in LDS, a streamed slab, a few rows over wide columns,
# rows that start off 16-byte boundaries, short rows
_REDUCE_SHAPES = [([65536, 16, 64], 1, "sum"), ([6710, 1000, 10], 1, "sum"), ([23, 2, 1456699], 1, "max"),
                  ([32752, 2049], 1, "argMax"), ([262144, 255], 1, "mean")]


def reduce_shapes_at(d):
    """The (shape, axis, op) list of the reduce_shapes workload at dims `d`."""
    return [([max(1, shape[0] // d["scale"])] + shape[1:], axis, op) for shape, axis, op in _REDUCE_SHAPES]


def _in_red(d):
    g = SplitMix64(11)
    return {f"x{i}": g.normal(shape) for i, (shape, _, _) in enumerate(reduce_shapes_at(d))}


def _run_red(ops, inp):
    out = {}
    for i, (shape, axis, op) in enumerate(_REDUCE_SHAPES):
        x = ops.create(list(inp[f"x{i}"].shape), False, inp[f"x{i}"])
        out[f"{op}{i}"] = getattr(x, op)(axis)
    return out


def _bytes_red(d):
    total = 0
    for shape, axis, _ in reduce_shapes_at(d):
        n = int(np.prod(shape, dtype=np.int64))
        total += 4 * (n + n // shape[axis])
    return total


# ---- indexed moves with index tensors as large as the data ---------------------------------------

def _in_idx(d):
    g = SplitMix64(12)
    rows, cols = d["rows"], d["cols"]
    def ints(shape, limit):
        return np.minimum(np.floor(g.uniform(shape, 0.0, float(limit))), np.float32(limit - 1)).astype(np.float32)
    return {"x": g.normal([rows, cols]), "along_cols": ints([rows, cols], cols), "along_rows": ints([rows, cols], rows),
            "row_list": ints([rows], rows)}


def _run_idx(ops, inp):
    from .autograd import NoGradVariable
    raw = {k: ops.create(list(v.shape), False, v).getRawValue() for k, v in inp.items()}
    x = raw["x"]
    gathered = x.gather(1, raw["along_cols"])
    assigned = ops.zerosLike(x)
    assigned.inplaceScatter(1, raw["along_cols"], x)
    added = ops.zerosLike(x)
    added.inplaceScatterAdd(0, raw["along_rows"], x)
    selected = x.indexSelect(0, raw["row_list"])
    summed = ops.zerosLike(x)
    summed.indexAdd(0, raw["row_list"], selected, 1.0)
    res = {"gathered": gathered, "assigned": assigned, "added": added, "selected": selected, "summed": summed}
    return {k: NoGradVariable(ops, v) for k, v in res.items()}


def _bytes_idx(d):
    n, rows = d["rows"] * d["cols"], d["rows"]
    # gather 12 N; three zerosLike 4 N each; assign 12 N; add 16 N; indexSelect 8 N + list; indexAdd 12 N + list
    return 72 * n + 8 * rows



# ---- indexed moves with skewed positions, flat tensors and short index rows ------------------------
# What an embedding gradient, a histogram and a top-k scatter ask of the indexed moves: positions drawn from a power law
# (floor(n u^4): element 0 takes n^(-1/4) of the draws), a flat tensor with twice as many entries as elements, index rows
# a thirty-second of the target's.

def _in_skew(d):
    g = SplitMix64(15)
    table, width, k, flat, rows, cols, short = d["table"], d["width"], d["k"], d["flat"], d["rows"], d["cols"], d["short"]
    def skewed(shape, limit):
        u = g.uniform(shape, 0.0, 1.0).astype(np.float64)
        return np.minimum(np.floor(limit * u ** 4), limit - 1).astype(np.float32)
    def ints(shape, limit):
        return np.minimum(np.floor(g.uniform(shape, 0.0, float(limit))), np.float32(limit - 1)).astype(np.float32)
    return {"grad_rows": g.normal([k, width]), "tokens": skewed([k], table), "weights": g.normal([2 * flat]), "bins": ints([2 * flat], flat),
            "x": g.normal([rows, cols]), "hot_cols": skewed([rows, cols], cols), "few_cols": ints([rows, short], cols),
            "picked": g.normal([rows, short]), "table": np.zeros([table, width], np.float32), "flat": np.zeros([flat], np.float32)}


def _run_skew(ops, inp):
    from .autograd import NoGradVariable
    raw = {k: ops.create(list(v.shape), False, v).getRawValue() for k, v in inp.items()}
    table_grad = ops.zerosLike(raw["table"])
    table_grad.indexAdd(0, raw["tokens"], raw["grad_rows"], 1.0)                   # an embedding's gradient
    histogram = ops.zerosLike(raw["flat"])
    histogram.inplaceScatterAdd(0, raw["bins"], raw["weights"])                    # weighted counts on a flat tensor
    latest = ops.zerosLike(raw["flat"])
    latest.inplaceScatter(0, raw["bins"], raw["weights"])                          # the last entry of every bin
    row_sums = ops.zerosLike(raw["x"])
    row_sums.inplaceScatterAdd(1, raw["hot_cols"], raw["x"])                       # rows with a full bin
    placed = ops.zerosLike(raw["x"])
    placed.inplaceScatterAdd(1, raw["few_cols"], raw["picked"])                    # a few entries per row
    res = {"table_grad": table_grad, "histogram": histogram, "latest": latest, "row_sums": row_sums, "placed": placed}
    return {k: NoGradVariable(ops, v) for k, v in res.items()}


def _bytes_skew(d):
    table, width, k, flat, rows, cols, short = d["table"], d["width"], d["k"], d["flat"], d["rows"], d["cols"], d["short"]
    # zerosLike 4 N each; indexAdd 12 N_src + list; scatterAdd 16 N_index; scatter 12 N_index
    return (4 * (table * width + 2 * flat + 2 * rows * cols) + 12 * k * width + 4 * k + (16 + 12) * 2 * flat
            + 16 * rows * cols + 16 * rows * short)


# ---- layout moves on shapes that are not multiples of anything convenient --------------------------

# (shape at scale 1, permutation): a run of 8 floats kept innermost, a run of 3, a run of 33, a long
# odd run (one 16-byte side); then a range get whose box starts one float into every row
_LAYOUT_SHAPES = [([64, 512, 256, 8], [0, 2, 1, 3]), ([4096, 5461, 3], [1, 0, 2]), ([2048, 1024, 33], [1, 0, 2]),
                  ([4096, 5, 3277], [1, 0, 2])]
_LAYOUT_BOX = [8192, 8192]


def layout_shapes_at(d):
    """The (shape, permutation) list and the [rows, cols] of the boxed tensor at dims `d`."""
    return ([([max(1, shape[0] // d["scale"])] + shape[1:], perm) for shape, perm in _LAYOUT_SHAPES],
            [max(2, _LAYOUT_BOX[0] // d["scale"]), _LAYOUT_BOX[1]])


def _in_lay(d):
    g = SplitMix64(13)
    shapes, box = layout_shapes_at(d)
    inp = {f"x{i}": g.uniform(shape, -1.0, 1.0) for i, (shape, _) in enumerate(shapes)}
    inp["boxed"] = g.uniform(box, -1.0, 1.0)
    return inp


def _run_lay(ops, inp):
    from .shape_functions import ALL
    out = {}
    for i, (_, perm) in enumerate(_LAYOUT_SHAPES):
        x = ops.create(list(inp[f"x{i}"].shape), False, inp[f"x{i}"])
        out[f"permuted{i}"] = x.permute(*perm)
    boxed = ops.create(list(inp["boxed"].shape), False, inp["boxed"])
    out["box"] = boxed[ALL, (1, inp["boxed"].shape[1] - 3)]
    return out


def _bytes_lay(d):
    shapes, box = layout_shapes_at(d)
    total = sum(8 * int(np.prod(shape, dtype=np.int64)) for shape, _ in shapes)
    return total + 8 * box[0] * (box[1] - 3)



# ---- the transcendental maps that cfg2 does not use ----------------------------------------------

_UNARY_MAPS = ["tanh", "sigmoid", "sinh", "cosh", "sin", "cos", "tan", "asin", "acos", "atan"]


def _in_maps(d):
    g = SplitMix64(14)
    return {"x": g.uniform([d["n"]], -1.0, 1.0), "p": g.uniform([d["n"]], 0.01, 2.0)}


def _run_maps(ops, inp):
    x = ops.create(list(inp["x"].shape), False, inp["x"])
    p = ops.create(list(inp["p"].shape), False, inp["p"])
    out = {name: getattr(x, name)() for name in _UNARY_MAPS}
    out["pow1.5"] = p ** 1.5
    return out


def _bytes_maps(d):
    return 8 * d["n"] * (len(_UNARY_MAPS) + 1)


WORKLOADS: Dict[str, Workload] = {
    "unary_maps": Workload("unary_maps", "tanh sigmoid sinh cosh sin cos tan asin acos atan of x[2^26] in U(-1,1) and p pow 1.5 "
                                         "of p[2^26] in U(0.01,2), seed 14: one map per launch",
                           {"n": 1 << 26}, _in_maps, _run_maps, _bytes_maps),

    "layout_shapes": Workload("layout_shapes", "permutes that keep an innermost run of 8, 3, 33 and 3277 floats ([64,512,256,8], "
                                               "[4096,5461,3], [2048,1024,33], [4096,5,3277]) and a range get x[:, 1:8190] of "
                                               "[8192,8192]; U(-1,1), seed 13",
                              {"scale": 1}, _in_lay, _run_lay, _bytes_lay),

    "reduce_shapes": Workload("reduce_shapes", "axis reductions over a middle or last axis on five geometries of 2^26 elements each: "
                                               "[65536,16,64] sum, [6710,1000,10] sum, [23,2,1456699] max, [32752,2049] argMax, "
                                               "[262144,255] mean; N(0,1), seed 11",
                              {"scale": 1}, _in_red, _run_red, _bytes_red),
    "indexed_skew": Workload("indexed_skew", "indexAdd of 262144 rows of 256 floats into zerosLike([50000,256]) at power-law rows; "
                                             "inplaceScatterAdd and inplaceScatter of 2^23 entries into a flat zerosLike([2^22]); "
                                             "inplaceScatterAdd along axis 1 of [8192,8192] at power-law columns and of [8192,256] "
                                             "entries at uniform ones; seed 15",
                             {"table": 50000, "width": 256, "k": 262144, "flat": 1 << 22, "rows": 8192, "cols": 8192, "short": 256},
                             _in_skew, _run_skew, _bytes_skew),
    "indexed_moves": Workload("indexed_moves", "x[16384,4096] with index tensors of its own size: gather along axis 1, inplaceScatter "
                                               "along axis 1, inplaceScatterAdd along axis 0 (each into zerosLike(x)), indexSelect and "
                                               "indexAdd of 16384 rows; seed 12",
                              {"rows": 16384, "cols": 4096}, _in_idx, _run_idx, _bytes_idx),

    "batch_norm": Workload("batch_norm", "BatchNormOperation over axis 1 of NCHW [64,128,56,56], training mode: calculateOutput "
                                         "then calculateGrads (input, gamma and beta gradients); seed 10",
                           {"n": 64, "c": 128, "h": 56, "w": 56}, _in_bn, _run_bn, _bytes_bn),
    "transpose": Workload("transpose", "x.transpose(0, 1): x[8192,8192], U(-1,1), seed 7", {"rows": 8192, "cols": 8192},
                          _in_tr, _run_tr, _bytes_tr),
    "permute": Workload("permute", "x.permute(0,2,3,1) then .permute(0,3,1,2): NCHW [64,128,56,56] to NHWC and back, seed 8",
                        {"n": 64, "c": 128, "h": 56, "w": 56}, _in_perm, _run_perm, _bytes_perm),
    "broadcast_reuse": Workload("broadcast_reuse", "x[32,2047,1020] + y[1,2047,1020] and a[1,6,4,56860] * b[23,1,4,56860]: operands of 8 MB and "
                                                   "5-21 MB that repeat along a dim, in shapes that are multiples of nothing; U(-1,1), seed 16",
                                {"n": 32, "t": 2047, "h": 1020, "p": 23, "q": 6, "r": 4, "s": 56860}, _in_reuse, _run_reuse, _bytes_reuse),
    "broadcast_pairs": Workload("broadcast_pairs", "four broadcasts of two operands that are both smaller than the 128-134 MB result and do not "
                                                   "coalesce to an outer product: [1,196,1,2] - [4,1,20452,1], [246,1,4,1] / [1,206,4,165], "
                                                   "[111,5496,1] * [111,1,55], [2481,4,1,21] + [1,4,161,1]; seed 17",
                                {"scale": 1}, _in_pairs, _run_pairs, _bytes_pairs),
    "sum0_alone": Workload("sum0_alone", "x.sum(0) of x[16384,4096], N(0,1), seed 4: the column reduction of cfg5 with nothing before it "
                                         "(the tensor was read, never written, by the launches before)",
                           {"rows": 16384, "cols": 4096}, _in_sum0, _run_sum0, lambda d: 4 * (d["rows"] * d["cols"] + d["cols"])),
    "concat_mask": Workload("concat_mask", "concat([8192,4096],[8192,4096], axis=1); maskedFill(mask[8192], 0); range get "
                                           "of the right half; range fill of the left half; seed 9",
                            {"rows": 8192, "left": 4096, "right": 4096}, _in_cat, _run_cat, _bytes_cat),
    "max_backward": Workload("max_backward", "x.max(-1).sum().backward(): x[8192,8192], N(0,1), seed 5 "
                                             "(max, argMax, zerosLike, inplaceScatter, gradient +=)",
                             {"rows": 8192, "cols": 8192}, _in_max, _run_max, _bytes_max),
    "softmax_ce": Workload("softmax_ce", "logits.softmaxCrossEntropy(targets).backward(): logits[32768,2048], seed 6 "
                                         "(max, minus, exp, sum, div, clamp, log, gather, mean; scatter, +=, /=)",
                           {"batch": 32768, "classes": 2048}, _in_sce, _run_sce, _bytes_sce),
    "cfg1": Workload("cfg1", "y=(x+b)*x; sum(y): x[2048,1024], b[1024], U(-1,1), seed 0",
                     {"rows": 2048, "cols": 1024}, _in1, _run1, _bytes1,
                     lambda d: 4 * (2 * d["rows"] * d["cols"] + d["cols"] + 1)),                  # read x and b, write y and s
    "cfg2": Workload("cfg2", "z=exp(-(x pow 2))+log(abs(x)+1e-3): x[2^26], N(0,1), seed 1",
                     {"n": 1 << 26}, _in2, _run2, _bytes2, lambda d: 4 * 2 * d["n"]),              # read x, write z
    "cfg3": Workload("cfg3", "sum/mean over axis 0 and 1, max and argmax over axis 1: x[8192,8192], N(0,1), seed 2",
                     {"rows": 8192, "cols": 8192}, _in3, _run3, _bytes3,
                     lambda d: 4 * (d["rows"] * d["cols"] + 2 * d["cols"] + 4 * d["rows"])),     # one read of x, the six results
    "cfg4": Workload("cfg4", "act*scale+bias on NCHW [64,128,56,56] with [1,128,1,1] operands, then sum and mean "
                             "over axes (0,2,3); seed 3",
                     {"n": 64, "c": 128, "h": 56, "w": 56}, _in4, _run4, _bytes4,
                     lambda d: 4 * (2 * d["n"] * d["c"] * d["h"] * d["w"] + 4 * d["c"])),        # read act, write out; scale, bias, sum, mean
    "cfg5": Workload("cfg5", "loss=sum(((x*w)+b) pow 2); backward(): x[16384,4096], w[4096], b[1], seed 4",
                     {"rows": 16384, "cols": 4096}, _in5, _run5, _bytes5,
                     lambda d: 4 * (d["rows"] * d["cols"] + 2 * d["cols"] + 3)),                 # one read of x; w, b; loss, grad w, grad b
}
