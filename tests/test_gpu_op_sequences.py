"""Random programs of raw-tensor ops, run side by side on the HIP backend and on the CPU checker.

The library keeps notes about stores between calls (a fill that is owed, an index tensor already found
valid) and several entry points take different kernels depending on them, on aliasing and on what the
operands' shapes coalesce to. The single-op tests cannot reach the states that only a history of calls
produces, so here a seeded generator draws 30 to 60 ops over a pool of tensors: factories (data, fill,
zerosLike, one uploaded value), broadcast binary ops, in-place ops (also `a op= a` and ops on views that
share a store), scalar ops, single-rounding unary ops, comparisons, broadcastTo, max / min / argMax /
argMin, gather, scatter, scatterAdd, indexSelect, indexAdd (with random indexes, with argMax results and
with indexes that were used before and then changed), range get / set / fill, store-range get / set,
narrow, transpose, permute, maskedFill, concat, copy, shallow copy, view, inplaceFill, zeroOut,
inplaceResize, release. Nothing is read back while the program runs (a download would settle the notes
under test) except at the few points the generator itself draws; at the end every live tensor of the pool
is compared, bit for bit (NaN matches NaN). Only ops whose parity bar is bit-exact are drawn: axis sums and
the transcendental maps are left to their own tests.

A failure prints the program, one op per line, so that the sequence can be replayed by its seed."""
import numpy as np
import pytest

from oracle import jvm_oracle as jo
from parity import assert_bits_equal

pytestmark = pytest.mark.gpu

BINARY = ["plus", "minus", "times", "div"]
COMPARE = ["lt", "lte", "gt", "gte", "eq", "neq"]
UNARY = ["neg", "abs", "sign", "sqrt", "floor", "ceil", "round", "trunc", "reciprocal", "rsqrt"]
CONSTANTS = [0.0, -0.0, 1.0, -1.0, 2.0, 0.5, -2.5, 0.1, 3.0, 1e-3, 7.25]


class Slot:
    def __init__(self, g, c, bound=None):
        self.g, self.c, self.bound = g, c, bound      # bound: every value is an integer in [0, bound)

    @property
    def shape(self):
        return list(self.c.shape)

    @property
    def size(self):
        return int(np.prod(self.c.shape)) if self.c.shape else 1


def shares(s, t):
    """True when two slots are wrappers around one store (a shallow copy or a view of the other)."""
    return s.c.storeReference is t.c.storeReference


def broadcastable(a, b):
    try:
        np.broadcast_shapes(tuple(a), tuple(b))
        return True
    except ValueError:
        return False


class NotApplicable(Exception):
    """The pool holds no tensor that the drawn op could take: another op is drawn."""


class Program:
    def __init__(self, seed, hip, cpu, dims):
        self.rng = np.random.default_rng(seed)
        self.hip, self.cpu, self.dims = hip, cpu, list(dims)
        self.slots, self.log = [], []

    # ------------------------------------------------------------------ helpers
    def note(self, text):
        self.log.append(text)

    def add(self, g, c, bound=None):
        assert list(g.shape) == list(c.shape), f"shapes differ: {g.shape} against {c.shape}\n" + self.listing()
        self.slots.append(Slot(g, c, bound))
        return len(self.slots) - 1

    def maybe(self, pred=lambda s: True):
        cands = [i for i, s in enumerate(self.slots) if s is not None and pred(s)]
        return int(self.rng.choice(cands)) if cands else None

    def pick(self, pred=lambda s: True):
        i = self.maybe(pred)
        if i is None:
            raise NotApplicable()
        return i

    def variant(self):
        """The base dims with some of them 1, sometimes without the leading ones."""
        shape = [d if self.rng.random() < 0.7 else 1 for d in self.dims]
        if len(shape) > 1 and self.rng.random() < 0.25:
            shape = shape[int(self.rng.integers(1, len(shape))):]
        return shape

    def data(self, shape):
        x = self.rng.standard_normal(shape).astype(np.float32)
        if self.rng.random() < 0.5:
            x[self.rng.random(shape) < 0.1] = 0.0
        if self.rng.random() < 0.3:
            x = np.round(x * 4).astype(np.float32)         # ties for max / min and exact sums
        return x

    def both(self, shape, values):
        return self.hip.createRaw(shape, values), self.cpu.createRaw(shape, values)

    def listing(self):
        return "\n".join(f"{i:3d}  {t}" for i, t in enumerate(self.log))

    def compare(self, i, what):
        s = self.slots[i]
        assert_bits_equal(s.g.toArray(), s.c.toArray(), f"{what}: slot {i} {s.shape}\n{self.listing()}\n")

    # ------------------------------------------------------------------ factories
    def op_data(self):
        shape = self.variant()
        i = self.add(*self.both(shape, self.data(shape)))
        self.note(f"s{i} = data{shape}")

    def op_fill(self):
        shape, v = self.variant(), float(self.rng.choice(CONSTANTS))
        i = self.add(self.hip.createRawFill(shape, v), self.cpu.createRawFill(shape, v), 2 if v in (0.0, 1.0) and not np.signbit(v) else None)
        self.note(f"s{i} = fill{shape} {v}")

    def op_zeros_like(self):
        a = self.pick()
        i = self.add(self.hip.zerosLike(self.slots[a].g), self.cpu.zerosLike(self.slots[a].c), 1)
        self.note(f"s{i} = zerosLike(s{a})")

    def op_single(self):
        v = float(np.float32(self.rng.standard_normal()))
        i = self.add(*self.both([1], [v]))
        self.note(f"s{i} = data[1] {v}")

    # ------------------------------------------------------------------ elementwise
    def op_binary(self):
        a = self.pick()
        cap = 8 * int(np.prod(self.dims))                  # a flat view against a column would give their outer product
        b = self.pick(lambda s: broadcastable(s.shape, self.slots[a].shape)
                      and int(np.prod(np.broadcast_shapes(tuple(s.shape), tuple(self.slots[a].shape)))) <= cap)
        name = str(self.rng.choice(BINARY))
        sa, sb = self.slots[a], self.slots[b]
        i = self.add(sa.g._binary(name, sb.g), sa.c._binary(name, sb.c))
        self.note(f"s{i} = s{a} {name} s{b}   {sa.shape} {sb.shape}")

    def op_binary_assign(self):
        a = self.pick()
        b = self.pick(lambda s: s.shape == self.slots[a].shape)
        name = str(self.rng.choice(BINARY))
        sa, sb = self.slots[a], self.slots[b]
        sa.g._binary_assign(name, sb.g); sa.c._binary_assign(name, sb.c)
        sa.bound = None
        self.note(f"s{a} {name}= s{b}   {sa.shape}")

    def op_scalar(self):
        a, name, v, rev = self.pick(), str(self.rng.choice(BINARY)), float(self.rng.choice(CONSTANTS)), bool(self.rng.random() < 0.3)
        sa = self.slots[a]
        i = self.add(sa.g._scalar(name, v, rev), sa.c._scalar(name, v, rev))
        self.note(f"s{i} = s{a} {name} {v}{' reversed' if rev else ''}")

    def op_pow_one(self):
        """pow with the exponent 1, which the library answers with a copy that it puts off."""
        a = self.pick()
        sa = self.slots[a]
        i = self.add(sa.g._scalar("pow", 1.0), sa.c._scalar("pow", 1.0), sa.bound)
        self.note(f"s{i} = s{a} pow 1.0")

    def op_scalar_assign(self):
        a, name, v = self.pick(), str(self.rng.choice(BINARY)), float(self.rng.choice(CONSTANTS))
        sa = self.slots[a]
        sa.g._scalar_assign(name, v); sa.c._scalar_assign(name, v)
        sa.bound = None
        self.note(f"s{a} {name}= {v}")

    def op_unary(self):
        a, name = self.pick(), str(self.rng.choice(UNARY))
        sa = self.slots[a]
        i = self.add(sa.g._unary(name), sa.c._unary(name))
        self.note(f"s{i} = {name}(s{a})")

    def op_compare(self):
        a, name = self.pick(), str(self.rng.choice(COMPARE))
        sa = self.slots[a]
        if self.rng.random() < 0.5:
            v = float(self.rng.choice(CONSTANTS))
            i = self.add(sa.g._compare(name, v), sa.c._compare(name, v), 2)
            self.note(f"s{i} = s{a} {name} {v}")
        else:
            b = self.pick(lambda s: s.shape == sa.shape)             # comparisons take equal shapes
            sb = self.slots[b]
            i = self.add(sa.g._compare(name, sb.g), sa.c._compare(name, sb.c), 2)
            self.note(f"s{i} = s{a} {name} s{b}")

    def op_broadcast_to(self):
        a = self.pick(lambda s: len(s.shape) <= len(self.dims) and broadcastable(s.shape, self.dims)
                      and list(np.broadcast_shapes(tuple(s.shape), tuple(self.dims))) == self.dims and s.shape != self.dims)
        sa = self.slots[a]
        i = self.add(sa.g.broadcastTo(self.dims), sa.c.broadcastTo(self.dims), sa.bound)
        self.note(f"s{i} = s{a}.broadcastTo{self.dims}")

    def op_masked_fill(self):
        m = self.pick(lambda s: s.bound == 2)
        sm = self.slots[m]
        a = self.pick(lambda s: len(s.shape) >= len(sm.shape) and broadcastable(s.shape, sm.shape)
                      and list(np.broadcast_shapes(tuple(s.shape), tuple(sm.shape))) == s.shape)
        v = float(self.rng.choice(CONSTANTS))
        sa = self.slots[a]
        i = self.add(sa.g.maskedFill(sm.g, v), sa.c.maskedFill(sm.c, v))
        self.note(f"s{i} = s{a}.maskedFill(s{m}, {v})")

    # ------------------------------------------------------------------ reductions with exact results
    def op_extreme(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        axis, keep = int(self.rng.integers(0, len(sa.shape))), bool(self.rng.random() < 0.6)
        if len(sa.shape) == 1 and not keep:
            keep = True
        name = str(self.rng.choice(["max", "min", "argMax", "argMin"]))
        i = self.add(getattr(sa.g, name)(axis, keep), getattr(sa.c, name)(axis, keep),
                     sa.shape[axis] if name.startswith("arg") else sa.bound)
        self.note(f"s{i} = s{a}.{name}({axis}, keep={keep})")

    def op_exact_sum(self):
        """A sum of whole numbers that no float sum rounds: every order of adding gives the same bits. (The library puts
        some small sums off and folds two steps of a chain into one launch; what reads or writes the tensors in
        between must see the plain sequence.)"""
        a = self.pick(lambda s: s.bound is not None and len(s.shape) >= 1)
        sa = self.slots[a]
        axis, keep = int(self.rng.integers(0, len(sa.shape))), bool(self.rng.random() < 0.6)
        if len(sa.shape) == 1 and not keep:
            keep = True
        bound = (sa.bound - 1) * sa.shape[axis] + 1
        if bound > (1 << 24):
            raise NotApplicable()
        i = self.add(sa.g.sum(axis, keep), sa.c.sum(axis, keep), bound)
        self.note(f"s{i} = s{a}.sum({axis}, keep={keep})")

    # ------------------------------------------------------------------ indexed moves
    def index_for(self, target, axis, ishape=None):
        """A slot holding valid positions along `axis` of the slot `target`: an existing one that fits (and is not
        the target's own store), or a fresh one."""
        shape = target.shape
        fits = lambda s: (s.bound is not None and s.bound <= shape[axis] and len(s.shape) == len(shape)
                          and all(s.shape[d] <= shape[d] for d in range(len(shape)) if d != axis)
                          and (ishape is None or s.shape == ishape) and not shares(s, target))
        x = self.maybe(fits) if self.rng.random() < 0.5 else None
        if x is not None:
            return x
        if ishape is None:
            ishape = list(shape)
            ishape[axis] = max(1, int(shape[axis] * self.rng.uniform(0.3, 1.6)))
            for d in range(len(shape)):
                if d != axis and self.rng.random() < 0.3:
                    ishape[d] = max(1, ishape[d] // 2)
        values = self.rng.integers(0, shape[axis], size=ishape).astype(np.float32)
        x = self.add(*self.both(ishape, values), shape[axis])
        self.note(f"s{x} = positions{ishape} below {shape[axis]}")
        return x

    def op_gather(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        axis = int(self.rng.integers(0, len(sa.shape)))
        x = self.index_for(sa, axis)
        sx = self.slots[x]
        i = self.add(sa.g.gather(axis, sx.g), sa.c.gather(axis, sx.c), sa.bound)
        self.note(f"s{i} = s{a}.gather({axis}, s{x})   {sa.shape} {sx.shape}")

    def op_scatter(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        axis = int(self.rng.integers(0, len(sa.shape)))
        x = self.index_for(sa, axis)
        sx = self.slots[x]
        kind = self.rng.random()
        if kind < 0.2:
            v = float(self.rng.choice(CONSTANTS))
            sa.g.inplaceScatter(axis, sx.g, v); sa.c.inplaceScatter(axis, sx.c, v)
            self.note(f"s{a}.inplaceScatter({axis}, s{x}, {v})   {sa.shape} {sx.shape}")
        else:
            src = self.maybe(lambda s: not shares(s, sa) and len(s.shape) == len(sx.shape) and all(p >= q for p, q in zip(s.shape, sx.shape)))
            if src is None or self.rng.random() < 0.5:
                src = self.add(*self.both(sx.shape, self.data(sx.shape)))
                self.note(f"s{src} = data{sx.shape}")
            ss = self.slots[src]
            name = "inplaceScatterAdd" if kind < 0.6 else "inplaceScatter"
            getattr(sa.g, name)(axis, sx.g, ss.g); getattr(sa.c, name)(axis, sx.c, ss.c)
            self.note(f"s{a}.{name}({axis}, s{x}, s{src})   {sa.shape} {sx.shape} {ss.shape}")
        sa.bound = None

    def rows_for(self, target, n):
        x = self.maybe(lambda s: s.bound is not None and s.bound <= n and len(s.shape) == 1 and not shares(s, target)) if self.rng.random() < 0.4 else None
        if x is not None:
            return x
        k = max(1, int(n * self.rng.uniform(0.3, 2.0)))
        x = self.add(*self.both([k], self.rng.integers(0, n, size=[k]).astype(np.float32)), n)
        self.note(f"s{x} = positions[{k}] below {n}")
        return x

    def op_index_select(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        axis = int(self.rng.integers(0, len(sa.shape)))
        x = self.rows_for(sa, sa.shape[axis])
        sx = self.slots[x]
        i = self.add(sa.g.indexSelect(axis, sx.g), sa.c.indexSelect(axis, sx.c), sa.bound)
        self.note(f"s{i} = s{a}.indexSelect({axis}, s{x})   {sa.shape} {sx.shape}")

    def op_index_add(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        axis = int(self.rng.integers(0, len(sa.shape)))
        x = self.rows_for(sa, sa.shape[axis])
        sx = self.slots[x]
        shape = list(sa.shape); shape[axis] = sx.shape[0]
        if int(np.prod(shape)) > 8 * int(np.prod(self.dims)):
            return False
        src = self.maybe(lambda s: not shares(s, sa) and s.shape == shape)
        if src is None or self.rng.random() < 0.5:
            if self.rng.random() < 0.3:
                v = float(self.rng.choice(CONSTANTS))
                src = self.add(self.hip.createRawFill(shape, v), self.cpu.createRawFill(shape, v))
                self.note(f"s{src} = fill{shape} {v}")
            else:
                src = self.add(*self.both(shape, self.data(shape)))
                self.note(f"s{src} = data{shape}")
        alpha = float(self.rng.choice([1.0, 0.7, -2.0]))
        ss = self.slots[src]
        sa.g.indexAdd(axis, sx.g, ss.g, alpha); sa.c.indexAdd(axis, sx.c, ss.c, alpha)
        sa.bound = None
        self.note(f"s{a}.indexAdd({axis}, s{x}, s{src}, {alpha})   {sa.shape}")

    # ------------------------------------------------------------------ ranges and layout
    def box(self, shape):
        first = [int(self.rng.integers(0, d)) for d in shape]
        last = [int(self.rng.integers(f, d)) for f, d in zip(first, shape)]
        for d in range(len(shape)):
            if self.rng.random() < 0.5:
                first[d], last[d] = 0, shape[d] - 1
        return first, last

    def op_get_ranges(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        first, last = self.box(sa.shape)
        shape = [l - f + 1 for f, l in zip(first, last)]
        i = self.add(sa.g._get_ranges(first, last, shape), sa.c._get_ranges(first, last, shape), sa.bound)
        self.note(f"s{i} = s{a}[{first}..{last}]")

    def op_set_ranges(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        first, last = self.box(sa.shape)
        shape = [l - f + 1 for f, l in zip(first, last)]
        if self.rng.random() < 0.4:
            v = float(self.rng.choice(CONSTANTS))
            sa.g._set_ranges(first, last, v); sa.c._set_ranges(first, last, v)
            self.note(f"s{a}[{first}..{last}] = {v}")
        else:
            b = self.maybe(lambda s: not shares(s, sa) and s.shape == shape)
            if b is None:
                b = self.add(*self.both(shape, self.data(shape)))
                self.note(f"s{b} = data{shape}")
            sb = self.slots[b]
            sa.g._set_ranges(first, last, sb.g); sa.c._set_ranges(first, last, sb.c)
            self.note(f"s{a}[{first}..{last}] = s{b}")
        sa.bound = None

    def op_store_range(self):
        a = self.pick(lambda s: s.size >= 2)
        sa = self.slots[a]
        off = int(self.rng.integers(0, sa.size - 1)) if self.rng.random() < 0.6 else 0
        n = int(self.rng.integers(1, sa.size - off + 1))
        kind = self.rng.random()
        if kind < 0.4:
            i = self.add(sa.g._get_store_range(off, n, [n]), sa.c._get_store_range(off, n, [n]), sa.bound)
            self.note(f"s{i} = s{a}.store[{off}:{off + n}]")
        elif kind < 0.7:
            v = float(self.rng.choice(CONSTANTS))
            sa.g._set_store_range(off, n, v); sa.c._set_store_range(off, n, v)
            sa.bound = None
            self.note(f"s{a}.store[{off}:{off + n}] = {v}")
        else:
            b = self.pick(lambda s: s.size >= n and not shares(s, sa))
            sb = self.slots[b]
            sa.g._set_store_range(off, n, sb.g); sa.c._set_store_range(off, n, sb.c)
            sa.bound = None
            self.note(f"s{a}.store[{off}:{off + n}] = s{b}.store[0:{n}]")

    def op_narrow(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        axis = int(self.rng.integers(0, len(sa.shape)))
        start = int(self.rng.integers(0, sa.shape[axis]))
        length = int(self.rng.integers(1, sa.shape[axis] - start + 1))
        i = self.add(sa.g.narrow(axis, start, length), sa.c.narrow(axis, start, length), sa.bound)
        self.note(f"s{i} = s{a}.narrow({axis}, {start}, {length})")

    def op_transpose(self):
        a = self.pick(lambda s: len(s.shape) >= 2)
        sa = self.slots[a]
        axis = int(self.rng.integers(0, len(sa.shape) - 1))           # adjacent axes: kten-jvm's transpose is the axis swap there
        i = self.add(sa.g.transpose(axis, axis + 1), sa.c.transpose(axis, axis + 1), sa.bound)
        self.note(f"s{i} = s{a}.transpose({axis}, {axis + 1})")

    def op_permute(self):
        a = self.pick(lambda s: len(s.shape) >= 2)
        sa = self.slots[a]
        axes = [int(v) for v in self.rng.permutation(len(sa.shape))]
        i = self.add(sa.g.permute(axes), sa.c.permute(axes), sa.bound)
        self.note(f"s{i} = s{a}.permute({axes})")

    def op_concat(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        axis = int(self.rng.integers(0, len(sa.shape)))
        others = lambda s: len(s.shape) == len(sa.shape) and all(p == q for d, (p, q) in enumerate(zip(s.shape, sa.shape)) if d != axis)
        parts = [a] + [self.pick(others) for _ in range(int(self.rng.integers(1, 3)))]
        i = self.add(self.hip.concat(axis, [self.slots[p].g for p in parts]), self.cpu.concat(axis, [self.slots[p].c for p in parts]),
                     max(self.slots[p].bound for p in parts) if all(self.slots[p].bound is not None for p in parts) else None)
        self.note(f"s{i} = concat({axis}, {['s%d' % p for p in parts]})")

    # ------------------------------------------------------------------ housekeeping
    def op_copy(self):
        a = self.pick()
        sa = self.slots[a]
        kind = self.rng.random()
        if kind < 0.5:
            i = self.add(sa.g.copy(), sa.c.copy(), sa.bound)
            self.note(f"s{i} = s{a}.copy()")
        elif kind < 0.75:
            i = self.add(sa.g.copy(shallow=True), sa.c.copy(shallow=True), None)
            sa.bound = None                                            # one store behind two slots: either may change it
            self.note(f"s{i} = s{a}.copy(shallow)")
        else:
            i = self.add(sa.g.view([sa.size]), sa.c.view([sa.size]), None)
            sa.bound = None
            self.note(f"s{i} = s{a}.view([{sa.size}])")

    def op_inplace_fill(self):
        a, v = self.pick(), float(self.rng.choice(CONSTANTS))
        sa = self.slots[a]
        if self.rng.random() < 0.5:
            sa.g.inplaceFill(v); sa.c.inplaceFill(v)
            self.note(f"s{a}.inplaceFill({v})")
        else:
            self.hip.zeroOut(sa.g); self.cpu.zeroOut(sa.c)
            self.note(f"zeroOut(s{a})")
        sa.bound = None

    def op_resize(self):
        a = self.pick(lambda s: len(s.shape) >= 1)
        sa = self.slots[a]
        shape = list(sa.shape)
        d = int(self.rng.integers(0, len(shape)))
        shape[d] = max(1, int(shape[d] * self.rng.uniform(0.5, 1.5)))
        sa.g.inplaceResize(shape); sa.c.inplaceResize(shape)
        sa.bound = None
        self.note(f"s{a}.inplaceResize({shape})")

    def op_release(self):
        if sum(s is not None for s in self.slots) < 6:
            return False
        a = self.pick()
        self.slots[a].g.release()
        self.slots[a] = None
        self.note(f"release s{a}")

    def op_look(self):
        a = self.pick()
        self.note(f"read s{a}")
        self.compare(a, "read in the middle")

    def op_change_an_index(self):
        """An index tensor that an op has already taken is changed in place (times 0: still valid, other values)
        or overwritten by other positions, then used again by a later op."""
        x = self.pick(lambda s: s.bound is not None and s.bound > 2)
        sx = self.slots[x]
        if self.rng.random() < 0.5:
            sx.g._scalar_assign("times", 0.0); sx.c._scalar_assign("times", 0.0)
            self.note(f"s{x} times= 0.0")
        else:
            values = self.rng.integers(0, sx.bound, size=sx.shape).astype(np.float32)
            other_g, other_c = self.both(sx.shape, values)
            sx.g._set_store_range(0, sx.size, other_g); sx.c._set_store_range(0, sx.size, other_c)
            self.note(f"s{x}.store[0:{sx.size}] = new positions below {sx.bound}")

    TABLE = [("op_data", 5), ("op_fill", 6), ("op_zeros_like", 3), ("op_single", 2), ("op_binary", 10), ("op_binary_assign", 7),
             ("op_scalar", 5), ("op_pow_one", 3), ("op_scalar_assign", 4), ("op_unary", 3), ("op_compare", 3), ("op_broadcast_to", 3), ("op_masked_fill", 2),
             ("op_extreme", 5), ("op_exact_sum", 4), ("op_gather", 4), ("op_scatter", 6), ("op_index_select", 3), ("op_index_add", 4), ("op_get_ranges", 2),
             ("op_set_ranges", 3), ("op_store_range", 3), ("op_narrow", 2), ("op_transpose", 2), ("op_permute", 2), ("op_concat", 2),
             ("op_copy", 4), ("op_inplace_fill", 3), ("op_resize", 1), ("op_release", 3), ("op_look", 1), ("op_change_an_index", 2)]

    def run(self, n_ops):
        for _ in range(3):
            self.op_data()
        self.op_fill()
        names = [n for n, _ in self.TABLE]
        weights = np.array([w for _, w in self.TABLE], dtype=np.float64)
        weights /= weights.sum()
        done = 0
        while done < n_ops:
            name = str(self.rng.choice(names, p=weights))
            try:
                if getattr(self, name)() is not False:
                    done += 1
            except NotApplicable:
                continue
            except AssertionError:
                raise
            except Exception as e:
                raise AssertionError(f"{name} raised {type(e).__name__}: {e}\n{self.listing()}") from e
        for i, s in enumerate(self.slots):
            if s is not None:
                self.compare(i, "at the end")


def run_program(seed, hip, cpu, dims, n_ops):
    with hip.garbageCollector():
        Program(seed, hip, cpu, dims).run(n_ops)


SMALL = [[7, 5, 6], [3, 33], [2, 3, 4, 5], [65], [1, 9, 1], [12, 1, 17]]
MEDIUM = [[64, 48, 40], [300, 257], [16, 8, 24, 20], [70001], [129, 1031], [9, 4096], [24, 56, 56], [130, 20, 1, 64]]


@pytest.mark.parametrize("seed", range(240))
def test_small_programs(seed, hip):
    """Tensors of a few dozen to a few hundred values: the small-tensor kernels and every note."""
    run_program(10_000 + seed, hip, jo.JvmOracleOperations(), SMALL[seed % len(SMALL)], 60)


@pytest.mark.parametrize("seed", range(120))
def test_medium_programs(seed, hip):
    """Tensors of 10^4 to 10^5 values: the vectorised, tiled and LDS-staged kernels."""
    run_program(20_000 + seed, hip, jo.JvmOracleOperations(), MEDIUM[seed % len(MEDIUM)], 40)


LARGE = [[1024, 640], [96, 128, 80], [2048, 8, 48], [640, 1536]]


@pytest.mark.parametrize("seed", range(24))
def test_large_programs(seed, hip):
    """Tensors of 10^6 values: index tensors above the sizes where gather and scatter go through rows in LDS."""
    run_program(30_000 + seed, hip, jo.JvmOracleOperations(), LARGE[seed % len(LARGE)], 30)
