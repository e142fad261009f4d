"""Shape / strides / offset algebra of tensor views — host-only, no device work.

Mirrors the metadata-only operations of the reference (nothing here touches data):
  shape_to_strides, is_C_contiguous, is_F_contiguous   src/arraymancer/tensor/data_structure.nim:129-178
  transpose                                             src/arraymancer/tensor/shapeshifting.nim:27-36
  slicer (a..b|step, inclusive ends, `^` from the end)  src/arraymancer/tensor/private/p_accessors_macros_read.nim:28-58
  broadcast / broadcast2                                src/arraymancer/tensor/private/p_shapeshifting.nim:76-134
Strides and offsets are in elements, as in the reference.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence, Tuple

MAXRANK = 6  # LASER_MAXRANK, src/arraymancer/laser/dynamic_stack_arrays.nim:6


@dataclass(frozen=True)
class Layout:
    shape: Tuple[int, ...]
    strides: Tuple[int, ...]
    offset: int = 0

    @property
    def rank(self) -> int:
        return len(self.shape)

    @property
    def size(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n


def shape_to_strides(shape: Sequence[int], order: str = "C") -> Tuple[int, ...]:
    strides = [0] * len(shape)
    acc = 1
    idx = range(len(shape) - 1, -1, -1) if order == "C" else range(len(shape))
    for i in idx:
        strides[i] = acc
        acc *= shape[i]
    return tuple(strides)


def contiguous(shape: Sequence[int], order: str = "C") -> Layout:
    shape = tuple(int(s) for s in shape)
    if len(shape) > MAXRANK:
        raise ValueError(f"rank {len(shape)} exceeds the maximum rank {MAXRANK}")
    return Layout(shape, shape_to_strides(shape, order), 0)


def is_C_contiguous(l: Layout) -> bool:
    cur = 1
    for i in range(l.rank - 1, -1, -1):
        if l.shape[i] != 1 and l.strides[i] != cur:   # strides of extent-1 axes are ignored
            return False
        cur *= l.shape[i]
    return True


def is_F_contiguous(l: Layout) -> bool:
    cur = 1
    for i in range(l.rank):
        if l.shape[i] != 1 and l.strides[i] != cur:
            return False
        cur *= l.shape[i]
    return True


def transpose(l: Layout) -> Layout:
    return Layout(l.shape[::-1], l.strides[::-1], l.offset)


def permute(l: Layout, dims: Sequence[int]) -> Layout:
    """The dimensions in the order `dims` (src/arraymancer/tensor/shapeshifting.nim:207-226): dimension i of the
    result is dimension dims[i] of the input; no data moves."""
    dims = tuple(int(d) for d in dims)
    if sorted(dims) != list(range(len(l.shape))):
        raise ValueError(f"permute: {dims} is not a permutation of the tensor's {len(l.shape)} dimensions")
    return Layout(tuple(l.shape[d] for d in dims), tuple(l.strides[d] for d in dims), l.offset)


def squeeze(l: Layout, axis: int | None = None) -> Layout:
    """Drops the dimensions of extent 1 (all of them, keeping rank >= 1, or the one at `axis` if it has extent 1 and the
    rank is above 1): squeezeImpl, src/arraymancer/tensor/private/p_shapeshifting.nim:157-177."""
    if axis is None:
        keep = [i for i, n in enumerate(l.shape) if n != 1] or [len(l.shape) - 1]
        return Layout(tuple(l.shape[i] for i in keep), tuple(l.strides[i] for i in keep), l.offset)
    if not 0 <= axis < len(l.shape):
        raise IndexError(f"squeeze: axis {axis} outside the tensor's rank {len(l.shape)}")
    if len(l.shape) > 1 and l.shape[axis] == 1:
        return Layout(l.shape[:axis] + l.shape[axis + 1:], l.strides[:axis] + l.strides[axis + 1:], l.offset)
    return l


def unsqueeze(l: Layout, axis: int) -> Layout:
    """Inserts a dimension of extent 1 at `axis`, with the stride the reference gives it
    (unsqueezeImpl, private/p_shapeshifting.nim:179-191)."""
    if not 0 <= axis <= len(l.shape):
        raise IndexError(f"unsqueeze: axis {axis} outside 0..{len(l.shape)}")
    stride = 1 if axis >= len(l.shape) else l.shape[axis] * l.strides[axis]
    return Layout(l.shape[:axis] + (1,) + l.shape[axis:], l.strides[:axis] + (stride,) + l.strides[axis:], l.offset)


class Step:
    """One slice in the reference's notation: first..last|step with INCLUSIVE ends;
    `first_from_end` / `last_from_end` are the `^n` forms (index = extent - n)."""

    __slots__ = ("a", "b", "step", "a_from_end", "b_from_end")

    def __init__(self, a, b, step=1, a_from_end=False, b_from_end=False):
        self.a, self.b, self.step = int(a), int(b), int(step)
        self.a_from_end, self.b_from_end = a_from_end, b_from_end


def slicer(l: Layout, slices: Sequence[Step]) -> Layout:
    if len(slices) > l.rank:
        raise IndexError(f"Rank of slice expression ({len(slices)}) is larger than the tensor rank. "
                         f"Tensor shape{list(l.shape)}.")
    shape, strides, offset = list(l.shape), list(l.strides), l.offset
    for i, s in enumerate(slices):
        a = shape[i] - s.a if s.a_from_end else s.a
        b = shape[i] - s.b if s.b_from_end else s.b
        if not (0 <= a < shape[i]) or not (0 <= b < shape[i]):
            raise IndexError(f"slice {a}..{b} out of bounds for axis {i} of extent {shape[i]}")
        if s.step == 0 or (a < b and s.step < 0) or (a > b and s.step > 0):
            raise IndexError(f"slice {a}..{b}|{s.step}: step has the wrong sign")
        offset += a * strides[i]
        strides[i] *= s.step
        shape[i] = abs(b - a) // abs(s.step) + 1   # |b - a| div step + 1 (same sign: truncation == floor)
    return Layout(tuple(shape), tuple(strides), offset)


def py_index(l: Layout, key) -> Layout:
    """Python indexing (ints, slices with exclusive stop, Ellipsis-free) expressed through the
    same offset/stride arithmetic. An integer index keeps its axis with extent 1, as slicing
    does in the reference."""
    if not isinstance(key, tuple):
        key = (key,)
    if len(key) > l.rank:
        raise IndexError(f"too many indices ({len(key)}) for a rank-{l.rank} tensor")
    shape, strides, offset = list(l.shape), list(l.strides), l.offset
    for i, k in enumerate(key):
        if isinstance(k, Step):
            sub = slicer(Layout((shape[i],), (strides[i],), 0), [k])
            offset += sub.offset
            shape[i], strides[i] = sub.shape[0], sub.strides[0]
        elif isinstance(k, slice):
            start, stop, step = k.indices(shape[i])
            n = len(range(start, stop, step))
            offset += (start * strides[i]) if n > 0 else 0
            strides[i] *= step
            shape[i] = n
        else:
            idx = int(k)
            if idx < 0:
                idx += shape[i]
            if not 0 <= idx < shape[i]:
                raise IndexError(f"index {k} out of bounds for axis {i} of extent {shape[i]}")
            offset += idx * strides[i]
            shape[i] = 1
    return Layout(tuple(shape), tuple(strides), offset)


def broadcast(l: Layout, shape: Sequence[int]) -> Layout:
    shape = tuple(int(s) for s in shape)
    if l.rank != len(shape):
        raise ValueError(f"broadcast: rank {l.rank} tensor cannot take a rank-{len(shape)} shape")
    new_shape, new_strides = list(l.shape), list(l.strides)
    for i in range(l.rank):
        if l.shape[i] == 1:
            if shape[i] != 1:
                new_shape[i] = shape[i]
                new_strides[i] = 0
        elif l.shape[i] != shape[i]:
            raise ValueError(f"The broadcasted size of the tensor {list(shape)}, must match existing size "
                             f"{list(l.shape)} for non-singleton dimension")
    return Layout(tuple(new_shape), tuple(new_strides), l.offset)


def broadcast2(a: Layout, b: Layout) -> Tuple[Layout, Layout]:
    if a.rank != b.rank:
        raise ValueError(f"Broadcasting error: ranks differ ({a.rank} and {b.rank})")
    sa, sta, sb, stb = [], [], [], []
    for i in range(a.rank):
        x, y = a.shape[i], b.shape[i]
        if x == y:
            sa.append(x); sb.append(x); sta.append(a.strides[i]); stb.append(b.strides[i])
        elif x == 1:
            sa.append(y); sb.append(y); sta.append(0); stb.append(b.strides[i])
        elif y == 1:
            sa.append(x); sb.append(x); sta.append(a.strides[i]); stb.append(0)
        else:
            raise ValueError("Broadcasting error: non-singleton dimensions must be the same in both tensors. "
                             f"Tensors' shapes were: {list(a.shape)} and {list(b.shape)}")
    return Layout(tuple(sa), tuple(sta), a.offset), Layout(tuple(sb), tuple(stb), b.offset)


def extent_in_storage(l: Layout) -> Tuple[int, int]:
    """Lowest and highest element index (inclusive) a view touches in its storage."""
    if l.size == 0:
        return l.offset, l.offset - 1
    lo = hi = l.offset
    for n, s in zip(l.shape, l.strides):
        if s >= 0:
            hi += (n - 1) * s
        else:
            lo += (n - 1) * s
    return lo, hi
