"""TEST INFRASTRUCTURE ONLY -- Python binding of the CPU oracle (oracle/dlf_oracle.cpp).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module.  It offers the same backend interface as the HIP backend so the
front-ends in dlf_amd.frontend drive it with identical arguments, plus fp64
evaluators for tolerance checks.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_char_p, c_int, c_int64, c_void_p, POINTER

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdlf_oracle.so")
_I64P = POINTER(c_int64)
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(LIB_PATH) or \
            os.path.getmtime(LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "dlf_oracle.cpp")):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "libdlf_oracle.so"],
                       check=True, capture_output=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.dlf_oracle_threads.restype = c_int
    return _lib


def _arr(values):
    values = list(values)
    return (c_int64 * max(1, len(values)))(*values)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


def _check(status, where):
    if status != 0:
        raise RuntimeError("%s failed with status %d" % (where, status))


class OracleBackend:
    """numpy-backed storage; calls restate dlf's CPU Tensor algorithms."""

    name = "oracle"

    def __init__(self, topk_mode: int = 1):
        # 1: specification order (stable, lowest index on ties); 0: the reference's heap
        self.topk_mode = topk_mode
        self.lib = lib()

    def alloc(self, dtype, count):
        return np.zeros(max(1, count), dtype=dtype)

    @staticmethod
    def _wide(dtype, inputs, outputs, fn):
        """16-bit and bool elements go through the 32-bit restatement: half -> float and
        int16 / bool -> int32 are exact and order preserving, and every result that is an
        element (not an index or a count) converts back exactly or, for sums, with the one
        rounding the 16-bit result type requires.  fn(code, inputs, outputs) makes the call."""
        if dtype not in (4, 5, 6):
            return fn(dtype, list(inputs), list(outputs))
        to, code = (np.float32, 0) if dtype == 4 else (np.int32, 2)
        cache = {}

        def widen(a):
            if a is None:
                return None
            if id(a) not in cache:
                cache[id(a)] = a.astype(to)
            return cache[id(a)]
        ins = [widen(a) for a in inputs]
        outs = [widen(a) for a in outputs]
        r = fn(code, ins, outs)
        for a, b in zip(outputs, outs):
            if a is not None:
                a[...] = b.astype(a.dtype)
        return r

    def upload(self, flat):
        return np.array(flat, copy=True).reshape(-1)

    def download(self, storage):
        return storage

    def reduce(self, name, dtype, m, n, xs, x, ys, y):
        return self._wide(dtype, [x], [y], lambda dtype, i, o: self._reduce_impl(name, dtype, m, n, xs, i[0], ys, o[0]))

    def _reduce_impl(self, name, dtype, m, n, xs, x, ys, y):
        _check(self.lib.dlf_oracle_reduce(
            c_char_p(name.encode()), c_int(dtype), c_int64(m), c_int64(n),
            c_int(xs.rank), _arr(xs.extents), _arr(xs.strides), _ptr(x), c_int64(xs.offset),
            c_int(ys.rank), _arr(ys.extents), _arr(ys.strides), _ptr(y), c_int64(ys.offset)), "oracle reduce")

    def arg_reduce(self, name, dtype, index_dtype, rows, k, xs, x, ys, y):
        return self._wide(dtype, [x], [], lambda dtype, i, o: self._arg_reduce_impl(name, dtype, index_dtype, rows, k, xs, i[0], ys, y))

    def _arg_reduce_impl(self, name, dtype, index_dtype, rows, k, xs, x, ys, y):
        out = y if y.dtype == np.int32 else np.zeros(y.shape, dtype=np.int32)
        _check(self.lib.dlf_oracle_arg_reduce(
            c_char_p(name.encode()), c_int(dtype), c_int64(rows), c_int64(k),
            c_int(xs.rank), _arr(xs.extents), _arr(xs.strides), _ptr(x), c_int64(xs.offset),
            c_int(ys.rank), _arr(ys.extents), _arr(ys.strides), _ptr(out), c_int64(ys.offset)), "oracle arg_reduce")
        if out is not y:
            y[...] = out

    def scan(self, name, dtype, m, n, exclusive, xs, x, ys, y):
        return self._wide(dtype, [x], [y], lambda dtype, i, o: self._scan_impl(name, dtype, m, n, exclusive, xs, i[0], ys, o[0]))

    def _scan_impl(self, name, dtype, m, n, exclusive, xs, x, ys, y):
        _check(self.lib.dlf_oracle_scan(
            c_char_p(name.encode()), c_int(dtype), c_int64(m), c_int64(n), c_int(int(bool(exclusive))),
            c_int(xs.rank), _arr(xs.extents), _ptr(x), c_int64(xs.offset), _arr(xs.strides),
            _ptr(y), c_int64(ys.offset), _arr(ys.strides)), "oracle scan")

    def sort(self, direction, dtype, xs, x, ys, y):
        return self._wide(dtype, [x], [y], lambda dtype, i, o: self._sort_impl(direction, dtype, xs, i[0], ys, o[0]))

    def _sort_impl(self, direction, dtype, xs, x, ys, y):
        _check(self.lib.dlf_oracle_sort(
            c_int(direction), c_int(dtype), c_int(xs.rank), _arr(xs.extents),
            _ptr(x), c_int64(xs.offset), _arr(xs.strides),
            _ptr(y), c_int64(ys.offset), _arr(ys.strides)), "oracle sort")

    def argsort(self, direction, dtype, index_dtype, xs, x, ys, y, is_, i):
        return self._wide(dtype, [x], [y], lambda dtype, ins, o, idx=i: self._argsort_impl(direction, dtype, index_dtype, xs, ins[0], ys, o[0], is_, idx))

    def _argsort_impl(self, direction, dtype, index_dtype, xs, x, ys, y, is_, i):
        out = i if i.dtype == np.int32 else np.zeros(i.shape, dtype=np.int32)
        _check(self.lib.dlf_oracle_argsort(
            c_int(direction), c_int(dtype), c_int(xs.rank), _arr(xs.extents),
            _ptr(x), c_int64(xs.offset), _arr(xs.strides),
            _ptr(y), c_int64(ys.offset if ys is not None else 0),
            _arr(ys.strides) if ys is not None else None,
            _ptr(out), c_int64(is_.offset), _arr(is_.strides)), "oracle argsort")
        if out is not i:
            i[...] = out

    def top_k(self, limit, direction, dtype, index_dtype, xs, x, ys, y, is_, i):
        return self._wide(dtype, [x], [y], lambda dtype, ins, o, idx=i: self._top_k_impl(limit, direction, dtype, index_dtype, xs, ins[0], ys, o[0], is_, idx))

    def _top_k_impl(self, limit, direction, dtype, index_dtype, xs, x, ys, y, is_, i):
        _check(self.lib.dlf_oracle_top_k(
            c_int(self.topk_mode), c_int64(limit), c_int(direction), c_int(1), c_int(dtype),
            c_int(xs.rank), _arr(xs.extents), _arr(ys.extents),
            _ptr(x), c_int64(xs.offset), _arr(xs.strides),
            _ptr(y), c_int64(ys.offset), _arr(ys.strides),
            _ptr(i), c_int64(is_.offset), _arr(is_.strides), c_int(i.dtype.itemsize)), "oracle top_k")

    def count(self, dtype, m, n, value, xs, x, ys, y):
        return self._wide(dtype, [x], [], lambda dtype, i, o: self._count_impl(dtype, m, n, value, xs, i[0], ys, y))

    def _count_impl(self, dtype, m, n, value, xs, x, ys, y):
        v = np.array([value], dtype=x.dtype)
        _check(self.lib.dlf_oracle_count(
            c_int(dtype), c_int64(m), c_int64(n), _ptr(v),
            c_int(xs.rank), _arr(xs.extents), _arr(xs.strides), _ptr(x), c_int64(xs.offset),
            c_int(ys.rank), _arr(ys.extents), _arr(ys.strides), _ptr(y), c_int64(ys.offset)), "oracle count")

    def scan_nonzero(self, dtype, m, n, exclusive, xs, x, ys, y):
        return self._wide(dtype, [x], [], lambda dtype, i, o: self._scan_nonzero_impl(dtype, m, n, exclusive, xs, i[0], ys, y))

    def _scan_nonzero_impl(self, dtype, m, n, exclusive, xs, x, ys, y):
        _check(self.lib.dlf_oracle_scan_nonzero(
            c_int(dtype), c_int64(m), c_int64(n), c_int(int(bool(exclusive))),
            c_int(xs.rank), _arr(xs.extents), _ptr(x), c_int64(xs.offset), _arr(xs.strides),
            _ptr(y), c_int64(ys.offset), _arr(ys.strides)), "oracle scan_nonzero")

    def gather_indices(self, m, n, row_major, dims, counts, out):
        _check(self.lib.dlf_oracle_gather_indices(
            c_int64(m), c_int64(n), c_int(int(bool(row_major))), c_int(len(dims)), _arr(dims),
            _ptr(counts), _ptr(out)), "oracle gather_indices")

    def softmax(self, name, dtype, m, n, x, x_offset, y, y_offset):
        return self._wide(dtype, [x], [y], lambda dtype, i, o: self._softmax_impl(name, dtype, m, n, i[0], x_offset, o[0], y_offset))

    def _softmax_impl(self, name, dtype, m, n, x, x_offset, y, y_offset):
        kind = {"softmax": 0, "logsoftmax": 1, "hardmax": 2}[name]
        if y is not x or y_offset != x_offset:
            y[y_offset:y_offset + m * n] = x[x_offset:x_offset + m * n]
        rows = y[y_offset:y_offset + m * n]
        _check(self.lib.dlf_oracle_softmax(c_int(kind), c_int(dtype), c_int64(m), c_int64(n), _ptr(rows)), "oracle " + name)

    def merge(self, direction, dtype, xs, x, ys, y, zs, z):
        return self._wide(dtype, [x, y], [z], lambda dtype, i, o: self._merge_impl(direction, dtype, xs, i[0], ys, i[1], zs, o[0]))

    def _merge_impl(self, direction, dtype, xs, x, ys, y, zs, z):
        _check(self.lib.dlf_oracle_merge(
            c_int(direction), c_int(dtype), c_int(zs.rank),
            _arr(xs.extents), _arr(xs.strides), _ptr(x), c_int64(xs.offset),
            _arr(ys.extents), _arr(ys.strides), _ptr(y), c_int64(ys.offset),
            _arr(zs.extents), _arr(zs.strides), _ptr(z), c_int64(zs.offset)), "oracle merge")

    def read_element(self, storage, index):
        return storage[index]

    def synchronize(self):
        pass


def reduce_f64(name, dtype, m, n, xs, x) -> np.ndarray:
    """fp64 evaluation of a reducer over the same view: one double per output row."""
    if dtype == 4:
        dtype, x = 0, x.astype(np.float32)
    out = np.zeros(m, dtype=np.float64)
    _check(lib().dlf_oracle_reduce_f64(
        c_char_p(name.encode()), c_int(dtype), c_int64(m), c_int64(n),
        c_int(xs.rank), _arr(xs.extents), _arr(xs.strides), _ptr(x), c_int64(xs.offset), _ptr(out)),
        "oracle reduce_f64")
    return out


def scan_f64(name, dtype, m, n, exclusive, xs, x, with_abs=True):
    """fp64 scan of the view, contiguous [m, n]; also the running sum of |x| when asked."""
    if dtype == 4:
        dtype, x = 0, x.astype(np.float32)
    out = np.zeros((m, n), dtype=np.float64)
    mag = np.zeros((m, n), dtype=np.float64) if with_abs else None
    _check(lib().dlf_oracle_scan_f64(
        c_char_p(name.encode()), c_int(dtype), c_int64(m), c_int64(n), c_int(int(bool(exclusive))),
        c_int(xs.rank), _arr(xs.extents), _ptr(x), c_int64(xs.offset), _arr(xs.strides),
        _ptr(out), _ptr(mag)), "oracle scan_f64")
    return out, mag


def threads() -> int:
    return lib().dlf_oracle_threads()


def set_threads(n: int) -> None:
    lib().dlf_oracle_set_threads(c_int(n))
