"""Host front-ends of the axis primitives, mirroring dlf's tensor API.

These functions do what dlf's header front-ends do before they reach the
``gpgpu::dnn`` boundary: normalise axes, build the moved-axis / transposed
strided view, size the output, then hand extents, strides, offsets and buffers
to a backend.  Reference: dlf/include/tensor/reduce.h:68-377,
reduce_detail.h:9-38,149-165, reorder.h:1120-1300.

A backend provides storage allocation and the six boundary calls; the shipped
backend is the HIP library (``dlf_amd.hip_backend``).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np

from .shape import Shape, ShapeError, norm_axes, norm_axis

DTYPE_CODES = {np.dtype(np.float32): 0, np.dtype(np.float64): 1,
               np.dtype(np.int32): 2, np.dtype(np.int64): 3,
               np.dtype(np.float16): 4, np.dtype(np.int16): 5, np.dtype(np.bool_): 6,
               np.dtype(np.complex64): 7, np.dtype(np.complex128): 8}

REDUCE_NAMES = ("reduce_sum", "reduce_mean", "reduce_max", "reduce_min", "reduce_log_sum_exp",
                "reduce_sum_exp", "reduce_log_sum", "reduce_prod", "reduce_asum",
                "reduce_sum_square", "reduce_nrm2", "reduce_amax", "reduce_amin")
SCAN_NAMES = ("cumsum", "cumprod", "cummax", "cummin")


def dtype_code(dtype) -> int:
    try:
        return DTYPE_CODES[np.dtype(dtype)]
    except KeyError:
        raise TypeError("unsupported element type %r" % (dtype,))


class Tensor:
    """A shape plus backend storage; views share storage (TensorView / DevTensorView)."""

    def __init__(self, backend, shape: Shape, storage, dtype):
        self.backend = backend
        self.shape = shape
        self.storage = storage
        self.dtype = np.dtype(dtype)

    # -- construction -------------------------------------------------------
    @classmethod
    def empty(cls, backend, extents: Sequence[int], dtype) -> "Tensor":
        shape = Shape(extents)
        return cls(backend, shape, backend.alloc(np.dtype(dtype), shape.size), dtype)

    @classmethod
    def from_numpy(cls, backend, array: np.ndarray) -> "Tensor":
        array = np.ascontiguousarray(array)
        shape = Shape(array.shape if array.ndim else ())
        return cls(backend, shape, backend.upload(array.reshape(-1)), array.dtype)

    # -- queries ------------------------------------------------------------
    @property
    def rank(self) -> int:
        return self.shape.rank

    @property
    def size(self) -> int:
        return self.shape.size

    def extent(self, i: int) -> int:
        return self.shape.extents[i]

    def numpy(self) -> np.ndarray:
        """Host copy of the viewed elements (``DevTensor::read``)."""
        flat = self.backend.download(self.storage)
        sh = self.shape
        item = flat.dtype.itemsize
        view = np.lib.stride_tricks.as_strided(
            flat[sh.offset:], shape=sh.extents, strides=[s * item for s in sh.strides], writeable=False)
        return np.array(view)

    # -- views --------------------------------------------------------------
    def view(self, shape: Shape) -> "Tensor":
        return Tensor(self.backend, shape, self.storage, self.dtype)

    def transpose(self, perm: Optional[Sequence[int]] = None) -> "Tensor":
        return self.view(self.shape.transpose(perm))

    def slice(self, starts, ends, axes=None, steps=None) -> "Tensor":
        return self.view(self.shape.slice(starts, ends, axes, steps))

    def moveaxis(self, source: int, destination: int) -> "Tensor":
        return self.view(self.shape.moveaxis(source, destination))

    def flip(self, axes=None) -> "Tensor":
        return self.view(self.shape.flip(axes))

    def contiguous(self) -> "Tensor":
        """The viewed elements in row-major order in storage of their own (the reference's
        reorder(X, Y)); on the device when the backend can copy a strided view there."""
        copy = getattr(self.backend, "copy_view", None)
        if copy is not None:
            return Tensor(self.backend, Shape(list(self.shape.extents)), copy(self.storage, self.shape), self.dtype)
        return Tensor.from_numpy(self.backend, self.numpy())


# ---------------------------------------------------------------------------
# reduce (reduce.h:68-129, reduce_detail.h:9-38,91-101)

def prepare_reduce(x_shape: Shape, axes: Sequence[int], keepdims: bool) -> Tuple[Shape, List[int], int, int]:
    """Returns (transposed view, output extents, m, n)."""
    rank = x_shape.rank
    axes = norm_axes(rank, axes, True)
    reduced = set(range(rank)) if not axes else set(axes)
    out_dims, perm = [], []
    m = n = 1
    for i in range(rank):
        if i not in reduced:
            out_dims.append(x_shape.extents[i])
            perm.append(i)
        elif keepdims:
            out_dims.append(1)
    for i in range(rank):
        if i in reduced:
            perm.append(i)
            n *= x_shape.extents[i]
        else:
            m *= x_shape.extents[i]
    return x_shape.transpose(perm), out_dims, m, n


def reduce(name: str, X: Tensor, axes: Sequence[int] = (), keepdims: bool = False) -> Tensor:
    if isinstance(axes, int):
        axes = [axes]
    view, out_dims, m, n = prepare_reduce(X.shape, list(axes), keepdims)
    Y = Tensor.empty(X.backend, out_dims, X.dtype)
    X.backend.reduce(name, dtype_code(X.dtype), m, n, view, X.storage, Y.shape, Y.storage)
    return Y


def count(X: Tensor, value, axes: Sequence[int] = (), keepdims: bool = False) -> Tensor:
    """Number of elements equal to `value` over `axes` (reduce.h:160-198); int32 result."""
    if isinstance(axes, int):
        axes = [axes]
    view, out_dims, m, n = prepare_reduce(X.shape, list(axes), keepdims)
    Y = Tensor.empty(X.backend, out_dims, np.int32)
    X.backend.count(dtype_code(X.dtype), m, n, value, view, X.storage, Y.shape, Y.storage)
    return Y


def nonzero(X: Tensor, row_major: bool = False) -> Optional[Tensor]:
    """Coordinates of the non-zero elements (reduce.h:419-450): an [n, rank] int32 tensor, or
    [rank, n] when row_major; None when there is none (the reference clears the output)."""
    size = X.size
    counts = Tensor.empty(X.backend, [size], np.int32)
    counts_shape = Shape(X.shape.extents)           # contiguous, the input's extents
    X.backend.scan_nonzero(dtype_code(X.dtype), 1, size, False,
                           _as_row(X.shape), X.storage, _as_row(counts_shape), counts.storage)
    n = int(X.backend.read_element(counts.storage, size - 1))
    if n == 0:
        return None
    rank = X.rank
    Y = Tensor.empty(X.backend, [rank, n] if row_major else [n, rank], np.int32)
    X.backend.gather_indices(size, n, row_major, list(X.shape.extents), counts.storage, Y.storage)
    return Y


def _as_row(shape: Shape) -> Shape:
    """The view itself: scan_nonzero(1, size, ...) walks all of it as one row, in row-major
    order of the extents, which is how the reference passes it (reduce.h:426-429)."""
    return shape


def _make_reduce(name):
    def f(X: Tensor, axes: Sequence[int] = (), keepdims: bool = False) -> Tensor:
        return reduce(name, X, axes, keepdims)
    f.__name__ = name
    f.__doc__ = "dlf::%s (reduce.h:84-129)" % name
    return f


for _n in REDUCE_NAMES:
    globals()[_n] = _make_reduce(_n)


# ---------------------------------------------------------------------------
# argmax / argmin (reduce.h:204-234, reduce_detail.h:149-165)

def arg_reduce(name: str, X: Tensor, axis: int, keepdims: bool = True, index_dtype=np.int32) -> Tensor:
    axis = norm_axis(X.rank, axis)
    y_dims = list(X.shape.extents)
    if keepdims:
        y_dims[axis] = 1
    else:
        del y_dims[axis]
    view = X.shape.moveaxis(axis, -1)
    Y = Tensor.empty(X.backend, y_dims, index_dtype)
    k = view.extents[-1]
    X.backend.arg_reduce(name, dtype_code(X.dtype), dtype_code(index_dtype), view.size // k, k,
                         view, X.storage, Y.shape, Y.storage)
    return Y


def argmax(X: Tensor, axis: int, keepdims: bool = True, index_dtype=np.int32) -> Tensor:
    return arg_reduce("argmax", X, axis, keepdims, index_dtype)


def argmin(X: Tensor, axis: int, keepdims: bool = True, index_dtype=np.int32) -> Tensor:
    return arg_reduce("argmin", X, axis, keepdims, index_dtype)


# ---------------------------------------------------------------------------
# scan (reduce.h:240-377)

def scan(name: str, X: Tensor, axis: int = -1, exclusive: bool = False, reverse: bool = False,
         out: Optional[Tensor] = None) -> Tensor:
    axis = norm_axis(X.rank, axis)
    n = X.shape.extents[axis]
    m = X.size // n
    Y = out if out is not None else Tensor.empty(X.backend, X.shape.extents, X.dtype)
    if Y.shape.extents != X.shape.extents or Y.dtype != X.dtype:
        raise ShapeError("scan: output does not match input")
    xs = X.shape.moveaxis(axis, -1)
    ys = Y.shape.moveaxis(axis, -1)
    if reverse:
        xs = xs.flip([-1])
        ys = ys.flip([-1])
    X.backend.scan(name, dtype_code(X.dtype), m, n, exclusive, xs, X.storage, ys, Y.storage)
    return Y


def cumsum(X, axis=-1, exclusive=False, reverse=False, out=None):
    return scan("cumsum", X, axis, exclusive, reverse, out)


def cumprod(X, axis=-1, exclusive=False, reverse=False, out=None):
    return scan("cumprod", X, axis, exclusive, reverse, out)


def cummax(X, axis=-1, reverse=False, out=None):
    return scan("cummax", X, axis, False, reverse, out)


def cummin(X, axis=-1, reverse=False, out=None):
    return scan("cummin", X, axis, False, reverse, out)


# ---------------------------------------------------------------------------
# sort / argsort / top_k (reorder.h:1120-1300)

def _copy_into(X: Tensor, Y: Tensor) -> None:
    Y.storage = X.backend.upload(X.numpy().reshape(-1))
    Y.shape = Shape(X.shape.extents)


def sort(X: Tensor, axis: int = -1, descending: bool = False, out: Optional[Tensor] = None) -> Tensor:
    axis = norm_axis(X.rank, axis)
    Y = out if out is not None else Tensor.empty(X.backend, X.shape.extents, X.dtype)
    if X.shape.extents[axis] > 1:
        xs, ys = X.shape.moveaxis(axis, -1), Y.shape.moveaxis(axis, -1)
        X.backend.sort(int(descending), dtype_code(X.dtype), xs, X.storage, ys, Y.storage)
    elif Y is not X:
        _copy_into(X, Y)
    return Y


def argsort(X: Tensor, axis: int = -1, descending: bool = False, values: Optional[Tensor] = None,
            index_dtype=np.int32, with_values: bool = False):
    """Index-only argsort returns I; with ``values`` (or with_values) returns (Y, I)."""
    axis = norm_axis(X.rank, axis)
    I = Tensor.empty(X.backend, X.shape.extents, index_dtype)
    Y = values
    if Y is None and with_values:
        Y = Tensor.empty(X.backend, X.shape.extents, X.dtype)
    if X.shape.extents[axis] > 1:
        xs, is_ = X.shape.moveaxis(axis, -1), I.shape.moveaxis(axis, -1)
        ys = Y.shape.moveaxis(axis, -1) if Y is not None else None
        X.backend.argsort(int(descending), dtype_code(X.dtype), dtype_code(index_dtype), xs, X.storage,
                          ys, Y.storage if Y is not None else None, is_, I.storage)
    else:
        if Y is not None and Y is not X:
            _copy_into(X, Y)
        I.storage = X.backend.upload(np.zeros(I.size, dtype=index_dtype))
    return (Y, I) if Y is not None else I


def top_k(X: Tensor, k: int, axis: int = -1, largest: bool = True, index_dtype=np.int32):
    axis = norm_axis(X.rank, axis)
    k = min(int(k), X.shape.extents[axis])
    out_dims = list(X.shape.extents)
    out_dims[axis] = k
    Y = Tensor.empty(X.backend, out_dims, X.dtype)
    I = Tensor.empty(X.backend, out_dims, index_dtype)
    xs, ys, is_ = X.shape.moveaxis(axis, -1), Y.shape.moveaxis(axis, -1), I.shape.moveaxis(axis, -1)
    X.backend.top_k(k, int(largest), dtype_code(X.dtype), dtype_code(index_dtype),
                    xs, X.storage, ys, Y.storage, is_, I.storage)
    return Y, I


def merge(A: Tensor, B: Tensor, axis: int = -1, descending: bool = False, out: Optional[Tensor] = None) -> Tensor:
    """Merges two tensors sorted along `axis` into one sorted tensor (reorder.h:1061-1114):
    the other extents must agree; equal elements keep A's before B's."""
    rank = A.rank
    if B.rank != rank:
        raise ShapeError("merge: incompatible shape")
    axis = norm_axis(rank, axis)
    dims = []
    for i in range(rank):
        if i == axis:
            dims.append(A.extent(i) + B.extent(i))
        elif A.extent(i) != B.extent(i):
            raise ShapeError("merge: incompatible shape")
        else:
            dims.append(A.extent(i))
    C = out if out is not None else Tensor.empty(A.backend, dims, A.dtype)
    if list(C.shape.extents) != dims:
        raise ShapeError("merge: output shape")
    a, b, c = A.shape.moveaxis(axis, -1), B.shape.moveaxis(axis, -1), C.shape.moveaxis(axis, -1)
    A.backend.merge(1 if descending else 0, dtype_code(A.dtype), a, A.storage, b, B.storage, c, C.storage)
    return C


def _softmax_family(name: str, X: Tensor, axis: int) -> Tensor:
    """dlf/include/tensor/dnn.h:447-531: the tensor is flattened to [m, n] with m the product
    of the extents before `axis` (default 1) and each row is normalised.  A non-contiguous
    input is copied first, as the reference's reorder(X, Y) does."""
    axis = norm_axis(X.rank, axis)
    m = 1
    for i in range(axis):
        m *= X.extent(i)
    n = X.size // m
    src = X if X.shape.is_contiguous() else X.contiguous()
    Y = Tensor.empty(X.backend, list(X.shape.extents), X.dtype)
    X.backend.softmax(name, dtype_code(X.dtype), m, n, src.storage, src.shape.offset, Y.storage, 0)
    return Y


def softmax(X: Tensor, axis: int = 1) -> Tensor:
    return _softmax_family("softmax", X, axis)


def logsoftmax(X: Tensor, axis: int = 1) -> Tensor:
    return _softmax_family("logsoftmax", X, axis)


def hardmax(X: Tensor, axis: int = 1) -> Tensor:
    return _softmax_family("hardmax", X, axis)


def gather_elements(X: np.ndarray, I: np.ndarray, axis: int) -> np.ndarray:
    """Host helper of the reference's property tests (reorder_detail.h:190-207)."""
    return np.take_along_axis(X, I.astype(np.int64), axis=axis)
