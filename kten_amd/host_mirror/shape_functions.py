"""Shape algebra used on both sides of the raw-tensor contract.

Host-side restatement of the part of the reference's
kten-api/src/main/kotlin/eu/redbean/kten/api/autograd/utils/ShapeFunctions.kt that the
broadcast / reduction path uses. Shapes are Python lists of ints; every function raises
ValueError where the reference throws IllegalArgumentException, before anything is
launched on the device.
"""
from typing import NamedTuple, List, Sequence


def to_store_size(shape: Sequence[int]) -> int:
    """ShapeFunctions.kt:344 — element count of a row-major store."""
    n = 1
    for d in shape:
        n *= d
    return n


def normalize_axis(shape: Sequence[int], axis: int) -> int:
    """ShapeFunctions.kt:41-48 — negative axes count from the end; out of range throws."""
    res = len(shape) + axis if axis < 0 else axis
    if res < 0 or res >= len(shape):
        raise ValueError(f"Cannot address axis: {axis} in tensor with dimensions: {len(shape)}")
    return res


def reshape(shape: Sequence[int], new_shape: Sequence[int]) -> List[int]:
    """ShapeFunctions.kt:11-39 — at most one -1 is inferred; element counts must match."""
    new_shape = list(new_shape)
    if any(d < -1 for d in new_shape):
        raise ValueError(f"Invalid shape: {new_shape}")
    inferred = [i for i, d in enumerate(new_shape) if d == -1]
    if len(inferred) > 1:
        raise ValueError(f"Cannot reshape to {new_shape}. Only one dimension can be inferred")
    res = list(new_shape)
    elements = to_store_size(shape)
    if inferred:
        res[inferred[0]] = 1
        known = to_store_size(res)
        res[inferred[0]] = elements // known if known else 0
    if elements != to_store_size(res):
        raise ValueError(f"Cannot reshape tensor with shape: {list(shape)} to shape: {new_shape}")
    return res


def squeeze(shape: Sequence[int], axis: int) -> List[int]:
    """ShapeFunctions.kt:50-59."""
    a = normalize_axis(shape, axis)
    if shape[a] != 1:
        raise ValueError(f"Cannot squeeze tensor with shape: {list(shape)} at axis: {axis}")
    res = list(shape)
    del res[a]
    return res


def unsqueeze(shape: Sequence[int], axis: int) -> List[int]:
    """ShapeFunctions.kt:61-71 — axis == len appends; a negative axis inserts after the
    dim it names, except -(len+1) which inserts in front."""
    n = len(shape)
    if axis == n:
        a = axis
    elif axis < 0:
        a = 0 if axis == -(n + 1) else normalize_axis(shape, axis) + 1
    else:
        a = normalize_axis(shape, axis)
    res = list(shape)
    res.insert(a, 1)
    return res


def aggregate_over(shape: Sequence[int], axis: int, keep_dimensions: bool) -> List[int]:
    """ShapeFunctions.kt:73-83 — the reduced dim becomes 1 and is dropped unless kept or
    the result would be 0-D."""
    a = normalize_axis(shape, axis)
    res = list(shape)
    res[a] = 1
    if not keep_dimensions and len(res) > 1:
        del res[a]
    return res


def infer_implicit_broadcast_shape(shape1: Sequence[int], shape2: Sequence[int]) -> List[int]:
    """ShapeFunctions.kt:168-185 — right-align, pad with leading 1s, each pair must be
    equal or contain a 1."""
    dims = max(len(shape1), len(shape2))
    s1 = [1] * (dims - len(shape1)) + list(shape1)
    s2 = [1] * (dims - len(shape2)) + list(shape2)
    out = []
    for a, b in zip(s1, s2):
        if a == b or a == 1 or b == 1:
            out.append(max(a, b))
        else:
            raise ValueError(
                f"Shape {s1} must match {s2} for every non-singleton dimensions (missing dimensions count as "
                "singleton dimension at the beginning of the shapes)")
    return out


def infer_explicit_broadcast_shape(shape: Sequence[int], target: Sequence[int]) -> List[int]:
    """ShapeFunctions.kt:187-201 — one-directional: `shape` must expand to `target`."""
    if len(shape) > len(target):
        raise ValueError(f"Tensor with shape: {list(shape)} cannot be broadcasted to shape: {list(target)}")
    padded = [1] * (len(target) - len(shape)) + list(shape)
    out = []
    for a, b in zip(padded, target):
        if a == b or a == 1:
            out.append(max(a, b))
        else:
            raise ValueError(
                f"Shape {list(shape)} must match {list(target)} for every non-singleton dimensions (missing "
                "dimensions count as singleton dimension at the beginning of the shapes)")
    return out


def normalize_index(shape: Sequence[int], index: Sequence[int]) -> List[int]:
    """ShapeFunctions.kt:203-215 — per-dim negative wrap and bounds check."""
    if len(index) > len(shape):
        raise ValueError(f"Cannot index tensor with shape: {list(shape)} with index: {list(index)}")
    out = []
    for size, item in zip(shape, index):
        n = size + item if item < 0 else item
        if n < 0 or n >= size:
            raise ValueError(f"Cannot index tensor with shape: {list(shape)} with index: {list(index)}")
        out.append(n)
    return out


def store_index(shape: Sequence[int], index: Sequence[int]) -> int:
    """Row-major offset of a full index (AbstractIndexing.kt:7-11,107-109)."""
    idx = normalize_index(shape, index)
    if len(idx) != len(shape):
        raise ValueError(f"Index {list(index)} does not address a single element of shape {list(shape)}")
    off = 0
    for size, i in zip(shape, idx):
        off = off * size + i
    return off


def outer_axis_inner(shape: Sequence[int], axis: int):
    """The [outer, axis, inner] view of a row-major tensor around a normalised axis."""
    return to_store_size(shape[:axis]), shape[axis], to_store_size(shape[axis + 1:])


def normalized_axis_scatter(shape: Sequence[int], axis: int, index_shape: Sequence[int], src_shape: Sequence[int]) -> int:
    """ShapeFunctions.kt:346-371 — target, index and source have equal dim counts; the index
    fits the source everywhere and the target everywhere but along the axis."""
    if len(shape) != len(index_shape) or len(shape) != len(src_shape):
        raise ValueError("Scatter expects tensors (target, index, source) to have the same dimensions, but got tensors "
                         f"with shapes: target: {list(shape)}, index: {list(index_shape)}, source: {list(src_shape)}")
    a = normalize_axis(shape, axis)
    for d in range(len(shape)):
        if index_shape[d] > src_shape[d]:
            raise ValueError("Scatter requires that index.shape[a] <= src.shape[a] for all axis 'a', but got tensors with "
                             f"shapes: index: {list(index_shape)}, src: {list(src_shape)}")
        if d != a and index_shape[d] > shape[d]:
            raise ValueError("Scatter requires that index.shape[a] <= target.shape[a] for all axis 'a', except the specified "
                             f"'axis' of the operation, but got tensors with shapes: index: {list(index_shape)}, target: {list(shape)}")
    return a


# ---------------------------------------------------------------- range indexing

class IntRange(NamedTuple):
    """A Kotlin `first..last` range: both ends inclusive."""
    first: int
    last: int


#: The reference's `all` range (kten-api/.../tensor/Constants.kt): every index of the dim.
ALL = IntRange(-2 ** 31, 2 ** 31 - 1)


def as_range(item) -> IntRange:
    """Accepts IntRange, ALL, or a (first, last) pair."""
    if isinstance(item, IntRange):
        return item
    if isinstance(item, (tuple, list)) and len(item) == 2:
        return IntRange(int(item[0]), int(item[1]))
    raise TypeError(f"Not an index range: {item!r}")


def normalized_indexed_shape(shape: Sequence[int], index: Sequence[int]):
    """ShapeFunctions.kt:232-238 — an Int index selects the sub-tensor under its leading
    dims; a full index selects one element, with shape [1]."""
    norm = normalize_index(shape, index)
    return norm, ([1] if len(norm) == len(shape) else list(shape[len(norm):]))


def normalize_range_index(shape: Sequence[int], index: Sequence) -> List[IntRange]:
    """ShapeFunctions.kt:240-259 — `all` becomes 0 until size; a range with a negative end has
    its negative ends wrapped; afterwards both ends must lie inside the dim, in order."""
    ranges = [as_range(r) for r in index]
    out = []
    invalid = len(ranges) > len(shape)
    for size, r in zip(shape, ranges):
        if r == ALL:
            r = IntRange(0, size - 1)
        elif r.first < 0 or r.last < 0:
            r = IntRange(size + r.first if r.first < 0 else r.first, size + r.last if r.last < 0 else r.last)
        if r.first < 0 or r.last < 0 or r.first >= size or r.last >= size or r.first > r.last:
            invalid = True
        out.append(r)
    if invalid:
        raise ValueError(f"Cannot index tensor with shape: {list(shape)} with index: {[tuple(r) for r in ranges]}")
    return out


def normalized_range_indexed_shape(shape: Sequence[int], index: Sequence):
    """ShapeFunctions.kt:261-268 — range lengths, then the unindexed trailing dims."""
    norm = normalize_range_index(shape, index)
    return norm, [r.last - r.first + 1 for r in norm] + list(shape[len(norm):])


def is_range_index(index) -> bool:
    """Kotlin picks the overload by type: IntArray or Array<IntRange>."""
    return len(index) > 0 and not all(isinstance(i, int) and not isinstance(i, bool) for i in index)


def store_range(shape: Sequence[int], norm_index: Sequence[int]):
    """AbstractIndexing.kt:43-54 SimpleTensorIndexing.storeRange as (offset, length)."""
    start = 0
    for size, i in zip(shape, norm_index):
        start = start * size + i
    sub = to_store_size(shape[len(norm_index):])
    return start * sub, sub


def full_ranges(shape: Sequence[int], norm_ranges: Sequence[IntRange]):
    """One (first, last) per dim: the given ranges, then every unindexed dim in full."""
    first = [r.first for r in norm_ranges] + [0] * (len(shape) - len(norm_ranges))
    last = [r.last for r in norm_ranges] + [s - 1 for s in shape[len(norm_ranges):]]
    return first, last


def index_select_norm_axis_shape(shape: Sequence[int], axis: int, index_shape: Sequence[int]):
    """ShapeFunctions.kt:270-278."""
    a = normalize_axis(shape, axis)
    if len(index_shape) != 1:
        raise ValueError(f"Index select requires singleton tensor as index, but got index tensor with shape: {list(index_shape)}")
    res = list(shape)
    res[a] = index_shape[0]
    return a, res


def index_add_check_shapes_norm_axis(shape: Sequence[int], axis: int, index_shape: Sequence[int], src_shape: Sequence[int]) -> int:
    """ShapeFunctions.kt:280-293."""
    if len(index_shape) != 1:
        raise ValueError(f"Index add requires index tensor to have 1 dimension, but got tensor with shape: {list(index_shape)}")
    a = normalize_axis(shape, axis)
    expected = list(shape)
    expected[a] = index_shape[0]
    if list(src_shape) != expected:
        raise ValueError("Index add expects source tensor to have same size as index size at the specified axis, and same size "
                         f"as this tensor for every other axis, but got source tensor with shape: {list(src_shape)} axis: {axis} "
                         f"and this tensor have shape: {list(shape)}")
    return a


def dot_shape(shape: Sequence[int], other: Sequence[int]) -> List[int]:
    """ShapeFunctions.kt:373-380."""
    if len(shape) != 1 or list(shape) != list(other):
        raise ValueError("Dot product can only applied to vectors (1D tensors) with same shape, but got tensors with shapes: "
                         f"{list(shape)} and {list(other)}")
    return [1]


def to_index_ranges(shape: Sequence[int]) -> List[IntRange]:
    """ShapeFunctions.kt:310-312."""
    return [IntRange(0, s - 1) for s in shape]


def transpose_normalize_axes(shape: Sequence[int], axis1: int, axis2: int):
    """ShapeFunctions.kt:115-129."""
    a1, a2 = normalize_axis(shape, axis1), normalize_axis(shape, axis2)
    if a1 == a2:
        raise ValueError(f"Transpose requires different axes as parameters, but got {axis1} (normalized: {a1}) "
                         f"and {axis2} (normalized: {a2})")
    res = list(shape)
    res[a1], res[a2] = shape[a2], shape[a1]
    return res, a1, a2


def permute(shape: Sequence[int], axes: Sequence[int]) -> List[int]:
    """ShapeFunctions.kt:106-113 — every dim must be named; negative axes are not accepted."""
    if len(shape) != len(axes) or not all(d in axes for d in range(len(shape))):
        raise ValueError(f"Tensor with shape: {list(shape)} cannot be permuted by axes: {list(axes)}. "
                         "All dimensions must be indexed.")
    return [shape[a] for a in axes]


def concat_shapes(shapes: Sequence[Sequence[int]], axis: int) -> List[int]:
    """ShapeFunctions.kt:85-104 — equal dim counts and equal sizes off the axis."""
    if len({len(s) for s in shapes}) == 1:
        a = normalize_axis(shapes[0], axis)
        rest = {tuple(s[:a]) + tuple(s[a + 1:]) for s in shapes}
        if len(rest) == 1:
            res = list(shapes[0])
            res[a] = sum(s[a] for s in shapes)
            return res
    raise ValueError(f"Cannot concatenate tensors with shapes: {[list(s) for s in shapes]} at axis: {axis} "
                     "(All tensors must have the same number of dimenisons, and have the same size at all dimenions "
                     "except at the dimension indexed by the axis)")
