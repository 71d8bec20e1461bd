"""Shape / view algebra mirroring dlf's ``Shape`` for the axis primitives.

Follows dlf/include/tensor/shape.h:51-366 and dlf/src/tensor/shape.cpp:21-135,
362-460, 608-640 and the view helpers ``moveaxis`` / ``flip``
(dlf/include/tensor/reorder.h:439-513).  Strides are kept as signed Python
integers: where the reference lets a negative step wrap around as ``size_t``,
the same memory walk is expressed here by the negative number itself.
"""
from __future__ import annotations

from typing import Iterable, List, Optional, Sequence


class ShapeError(ValueError):
    """Counterpart of dlf::shape_error."""


def norm_axis(rank: int, axis: int) -> int:
    if axis < 0:
        axis += rank
    if axis < 0 or axis >= rank:
        raise ShapeError("axis has incorrect value")
    return axis


def norm_axes(rank: int, axes: Iterable[int], allow_duplicates: bool = False) -> List[int]:
    out = [norm_axis(rank, a) for a in axes]
    if not allow_duplicates and len(set(out)) != len(out):
        raise ShapeError("axes has duplicates")
    return out


class Shape:
    """Extents, element strides and an element offset."""

    __slots__ = ("extents", "strides", "offset")

    def __init__(self, extents: Sequence[int], strides: Optional[Sequence[int]] = None, offset: int = 0):
        self.extents = tuple(int(e) for e in extents)
        for e in self.extents:
            if e <= 0:
                raise ShapeError("extent must be positive")
        if strides is None:
            st, size = [], 1
            for e in reversed(self.extents):
                st.append(size)
                size *= e
            self.strides = tuple(reversed(st))
        else:
            if len(strides) != len(self.extents):
                raise ShapeError("strides and extents differ in length")
            self.strides = tuple(int(s) for s in strides)
        self.offset = int(offset)

    # -- basic queries ------------------------------------------------------
    @property
    def rank(self) -> int:
        return len(self.extents)

    @property
    def size(self) -> int:
        s = 1
        for e in self.extents:
            s *= e
        return s

    def extent(self, i: int) -> int:
        return self.extents[i]

    def stride(self, i: int) -> int:
        return self.strides[i]

    def is_contiguous(self) -> bool:
        size = 1
        for e, s in zip(reversed(self.extents), reversed(self.strides)):
            if s == 0 and e == 1:
                continue
            if s != size:
                return False
            size *= e
        return True

    def linear_offset(self, index: int) -> int:
        off = self.offset
        for e, s in zip(reversed(self.extents), reversed(self.strides)):
            off += (index % e) * s
            index //= e
        return off

    def __eq__(self, other) -> bool:
        return isinstance(other, Shape) and self.extents == other.extents

    def __repr__(self) -> str:
        return "Shape(%s, strides=%s, offset=%d)" % (list(self.extents), list(self.strides), self.offset)

    # -- views --------------------------------------------------------------
    def transpose(self, perm: Optional[Sequence[int]] = None) -> "Shape":
        if perm is None:
            if self.rank == 1:
                return Shape((self.extents[0], 1), (self.strides[0], 0), self.offset)
            perm = list(reversed(range(self.rank)))
        perm = list(perm)
        if sorted(perm) != list(range(self.rank)):
            raise ShapeError("transpose: invalid permutation")
        return Shape([self.extents[p] for p in perm], [self.strides[p] for p in perm], self.offset)

    def slice(self, starts: Sequence[int], ends: Sequence[int],
              axes: Optional[Sequence[int]] = None, steps: Optional[Sequence[int]] = None) -> "Shape":
        if len(starts) != len(ends) or len(starts) > self.rank:
            raise ShapeError("slice: incorrect value for starts and ends")
        axes = list(range(len(starts))) if not axes else list(axes)
        if len(axes) != len(starts):
            raise ShapeError("slice: axes has incorrect length")
        steps = [1] * len(starts) if not steps else list(steps)
        if len(steps) != len(starts):
            raise ShapeError("slice: steps has incorrect length")
        if any(s == 0 for s in steps):
            raise ShapeError("slice: step cannot be 0")

        ext, st = list(self.extents), list(self.strides)
        offset = self.offset
        seen = set()
        clamp = lambda v, lo, hi: max(lo, min(hi, v))
        for i, axis in enumerate(axes):
            axis = norm_axis(self.rank, axis)
            if axis in seen:
                raise ShapeError("slice: axes has duplicates")
            seen.add(axis)
            dim, step = self.extents[axis], steps[i]
            start = starts[i] + (dim if starts[i] < 0 else 0)
            start = clamp(start, 0, dim - 1) if step < 0 else clamp(start, 0, dim)
            end = ends[i] + (dim if ends[i] < 0 else 0)
            end = clamp(end, -1, dim) if step < 0 else clamp(end, 0, dim)
            # C++ integer division truncates toward zero
            num = end - start - (-1 if step < 0 else 1)
            q = abs(num) // abs(step)
            if (num < 0) != (step < 0):
                q = -q
            count = q + 1
            if count < 0:
                raise ShapeError("slice: incorrect start and end value")
            if count == 0:
                count = 1
            ext[axis] = count
            st[axis] = self.strides[axis] * step
            offset += start * self.strides[axis]
        return Shape(ext, st, offset)

    def moveaxis(self, source: int, destination: int) -> "Shape":
        src = norm_axis(self.rank, source)
        dst = norm_axis(self.rank, destination)
        order = [k for k in range(self.rank) if k != src]
        order.insert(dst, src)
        return self.transpose(order)

    def flip(self, axes: Optional[Sequence[int]] = None) -> "Shape":
        axes = list(range(self.rank)) if not axes else norm_axes(self.rank, axes, True)
        int_min = -(2 ** 31)
        return self.slice([-1] * len(axes), [int_min] * len(axes), axes, [-1] * len(axes))
