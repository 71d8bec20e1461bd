"""ctypes binding of libdlfx.so (the C ABI in include/dlfx.h) plus the backend
object the front-ends call.  PyTorch is used only to own device memory and to
name the HIP stream work is enqueued on.

There is no fallback: if the library is missing or a call fails, this raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p, POINTER

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdlfx.so")

_I64P = POINTER(c_int64)


class DlfxError(RuntimeError):
    def __init__(self, status: int, text: str, where: str):
        super().__init__("%s: %s (status %d)" % (where, text, status))
        self.status = status


def _declare(lib):
    view = [c_int, _I64P, _I64P]
    lib.dlfx_version.restype = c_int
    lib.dlfx_status_string.restype = c_char_p
    lib.dlfx_status_string.argtypes = [c_int]
    lib.dlfx_last_hip_error.restype = c_int
    lib.dlfx_set_tuning.restype = c_int
    lib.dlfx_set_tuning.argtypes = [c_char_p, c_int64]

    lib.dlfx_reduce_scratch_bytes.restype = c_size_t
    lib.dlfx_reduce_scratch_bytes.argtypes = [c_int, c_int64, c_int64]
    lib.dlfx_reduce.restype = c_int
    lib.dlfx_reduce.argtypes = ([c_void_p, c_char_p, c_int, c_int64, c_int64] + view + [c_void_p, c_int64]
                                + view + [c_void_p, c_int64, c_void_p, c_size_t])

    lib.dlfx_reduce_static.restype = c_int
    lib.dlfx_reduce_static.argtypes = ([c_void_p, c_char_p, c_int, c_int64, c_int64] + view + [c_void_p, c_int64]
                                       + view + [c_void_p, c_int64])

    lib.dlfx_logits_head.restype = c_int
    lib.dlfx_logits_head.argtypes = [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                     c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p]

    lib.dlfx_arg_reduce_scratch_bytes.restype = c_size_t
    lib.dlfx_arg_reduce_scratch_bytes.argtypes = [c_int, c_int64, c_int64]
    lib.dlfx_arg_reduce.restype = c_int
    lib.dlfx_arg_reduce.argtypes = ([c_void_p, c_char_p, c_int, c_int, c_int64, c_int64] + view
                                    + [c_void_p, c_int64] + view + [c_void_p, c_int64, c_void_p, c_size_t])

    lib.dlfx_scan_scratch_bytes.restype = c_size_t
    lib.dlfx_scan_scratch_bytes.argtypes = [c_int, c_int64, c_int64]
    lib.dlfx_scan.restype = c_int
    lib.dlfx_scan.argtypes = [c_void_p, c_char_p, c_int, c_int64, c_int64, c_int, c_int, _I64P,
                              c_void_p, c_int64, _I64P, c_void_p, c_int64, _I64P, c_void_p, c_size_t]

    lib.dlfx_sort_scratch_bytes.restype = c_size_t
    lib.dlfx_sort_scratch_bytes.argtypes = [c_int, c_int64, c_int64]
    lib.dlfx_sort.restype = c_int
    lib.dlfx_sort.argtypes = [c_void_p, c_int, c_int, c_int, _I64P, c_void_p, c_int64, _I64P,
                              c_void_p, c_int64, _I64P, c_void_p, c_size_t]

    lib.dlfx_argsort_scratch_bytes.restype = c_size_t
    lib.dlfx_argsort_scratch_bytes.argtypes = [c_int, c_int64, c_int64]
    lib.dlfx_argsort.restype = c_int
    lib.dlfx_argsort.argtypes = [c_void_p, c_int, c_int, c_int, c_int, _I64P, c_void_p, c_int64, _I64P,
                                 c_void_p, c_int64, _I64P, c_void_p, c_int64, _I64P, c_void_p, c_size_t]

    lib.dlfx_top_k_scratch_bytes.restype = c_size_t
    lib.dlfx_top_k_scratch_bytes.argtypes = [c_int, c_int64, c_int64, c_int64]
    lib.dlfx_top_k.restype = c_int
    lib.dlfx_top_k.argtypes = [c_void_p, c_int64, c_int, c_int, c_int, c_int, _I64P, _I64P,
                               c_void_p, c_int64, _I64P, c_void_p, c_int64, _I64P,
                               c_void_p, c_int64, _I64P, c_void_p, c_size_t]
    lib.dlfx_count_scratch_bytes.restype = c_size_t
    lib.dlfx_count_scratch_bytes.argtypes = [c_int, c_int64, c_int64]
    lib.dlfx_count.restype = c_int
    lib.dlfx_count.argtypes = ([c_void_p, c_int, c_int64, c_int64, c_void_p] + view + [c_void_p, c_int64]
                               + view + [c_void_p, c_int64, c_void_p, c_size_t])

    lib.dlfx_scan_nonzero_scratch_bytes.restype = c_size_t
    lib.dlfx_scan_nonzero_scratch_bytes.argtypes = [c_int, c_int64, c_int64]
    lib.dlfx_scan_nonzero.restype = c_int
    lib.dlfx_scan_nonzero.argtypes = [c_void_p, c_int, c_int64, c_int64, c_int, c_int, _I64P,
                                      c_void_p, c_int64, _I64P, c_void_p, c_int64, _I64P, c_void_p, c_size_t]

    lib.dlfx_softmax.restype = c_int
    lib.dlfx_softmax.argtypes = [c_void_p, c_char_p, c_int, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_size_t]
    lib.dlfx_softmax_scratch_bytes.restype = c_size_t
    lib.dlfx_softmax_scratch_bytes.argtypes = [c_int, c_int64, c_int64]

    lib.dlfx_merge_scratch_bytes.restype = c_size_t
    lib.dlfx_merge_scratch_bytes.argtypes = [c_int, c_int64, c_int64]
    lib.dlfx_merge.restype = c_int
    lib.dlfx_merge.argtypes = [c_void_p, c_int, c_int, c_int, _I64P, _I64P, c_void_p, c_int64,
                               _I64P, _I64P, c_void_p, c_int64, _I64P, _I64P, c_void_p, c_int64, c_void_p, c_size_t]

    lib.dlfx_gather_indices.restype = c_int
    lib.dlfx_gather_indices.argtypes = [c_void_p, c_int64, c_int64, c_int, c_int, _I64P,
                                        c_void_p, c_int64, c_void_p, c_int64]
    lib.dlfx_copy.restype = c_int
    lib.dlfx_copy.argtypes = [c_void_p, c_int, c_int, _I64P, c_void_p, c_int64, _I64P, c_void_p, c_int64, _I64P]
    lib.dlfx_fill.restype = c_int
    lib.dlfx_fill.argtypes = [c_void_p, c_int, c_int, _I64P, _I64P, c_void_p, c_int64, c_void_p]
    return lib


_lib = None

# Every symbol include/dlfx.h declares.
EXPORTS = ("dlfx_version", "dlfx_status_string", "dlfx_last_hip_error", "dlfx_set_tuning",
           "dlfx_reduce_scratch_bytes", "dlfx_reduce", "dlfx_reduce_static", "dlfx_logits_head",
           "dlfx_arg_reduce_scratch_bytes", "dlfx_arg_reduce",
           "dlfx_scan_scratch_bytes", "dlfx_scan",
           "dlfx_sort_scratch_bytes", "dlfx_sort",
           "dlfx_argsort_scratch_bytes", "dlfx_argsort",
           "dlfx_top_k_scratch_bytes", "dlfx_top_k",
           "dlfx_count_scratch_bytes", "dlfx_count",
           "dlfx_scan_nonzero_scratch_bytes", "dlfx_scan_nonzero", "dlfx_gather_indices",
           "dlfx_merge_scratch_bytes", "dlfx_merge", "dlfx_softmax_scratch_bytes", "dlfx_softmax",
           "dlfx_copy", "dlfx_fill")


def load_library():
    """Loads libdlfx.so; raises when it has not been built (no fallback exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libdlfx.so is not built: run `python -m dlf_amd.build` "
                               "(or __graft_entry__.build()) first; expected at " + LIB_PATH)
        _lib = _declare(ctypes.CDLL(LIB_PATH))
    return _lib


def _arr(values):
    values = list(values)
    return (c_int64 * max(1, len(values)))(*values)


def _check(status: int, where: str):
    if status != 0:
        lib = load_library()
        text = lib.dlfx_status_string(status).decode()
        if status == -6:
            text += " (hipError %d)" % lib.dlfx_last_hip_error()
        raise DlfxError(status, text, where)


_NP_TO_TORCH = None


def _torch_dtype(np_dtype):
    global _NP_TO_TORCH
    import torch
    if _NP_TO_TORCH is None:
        _NP_TO_TORCH = {np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64,
                        np.dtype(np.int32): torch.int32, np.dtype(np.int64): torch.int64,
                        np.dtype(np.float16): torch.float16, np.dtype(np.int16): torch.int16,
                        np.dtype(np.bool_): torch.bool,
                        np.dtype(np.complex64): torch.complex64, np.dtype(np.complex128): torch.complex128}
    return _NP_TO_TORCH[np.dtype(np_dtype)]


def _dtype_code_of(torch_dtype, torch):
    return {torch.float32: 0, torch.float64: 1, torch.int32: 2, torch.int64: 3, torch.float16: 4, torch.int16: 5,
            torch.bool: 6, torch.complex64: 7, torch.complex128: 8}[torch_dtype]


class HipBackend:
    """Backend whose six boundary calls go through the C ABI onto the current HIP stream."""

    name = "hip"

    def __init__(self, device: str = "cuda:0"):
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("no HIP device visible to PyTorch")
        self.torch = torch
        self.device = torch.device(device)
        self.lib = load_library()
        self._scratch = None
        self._retired = []

    # -- storage ------------------------------------------------------------
    def alloc(self, dtype, count: int):
        return self.torch.empty(max(1, count), dtype=_torch_dtype(dtype), device=self.device)

    def upload(self, flat: np.ndarray):
        return self.torch.from_numpy(np.ascontiguousarray(flat)).to(self.device)

    def download(self, storage) -> np.ndarray:
        return storage.cpu().numpy()

    def copy_view(self, storage, shape):
        """Row-major device copy of a strided view (dlfx_copy: the reference's reorder(X, Y))."""
        out = self.torch.empty(max(1, shape.size), dtype=storage.dtype, device=self.device)
        if shape.size == 0:              # an empty slice: nothing to move
            return out
        dense = []
        size = 1
        for e in reversed(shape.extents):
            dense.insert(0, size)
            size *= e
        self.copy(_dtype_code_of(storage.dtype, self.torch), shape.extents, storage, shape.offset, shape.strides, out, 0, dense)
        return out

    def copy(self, dtype, extents, x, x_offset, x_strides, y, y_offset, y_strides, defer=False):
        return self._issue(self.lib.dlfx_copy, "dlfx_copy", (dtype, len(extents), _arr(extents)),
                           (x.data_ptr(), x_offset, _arr(x_strides), y.data_ptr(), y_offset, _arr(y_strides)), defer, (x, y))

    def fill(self, dtype, extents, strides, x, x_offset, value, defer=False):
        host_types = {0: np.float32, 1: np.float64, 2: np.int32, 3: np.int64, 4: np.float16, 5: np.int16,
                      6: np.bool_, 7: np.complex64, 8: np.complex128}
        v = np.array([value], dtype=host_types[dtype])
        call = self._issue(self.lib.dlfx_fill, "dlfx_fill", (dtype, len(extents), _arr(extents), _arr(strides)),
                           (x.data_ptr(), x_offset, v.ctypes.data_as(c_void_p)), defer, (x,))
        if call is None:
            return None
        return lambda v=v: call()

    def wrap(self, tensor):
        """Use an existing contiguous 1-D device tensor as storage."""
        return tensor

    def scratch(self, nbytes: int):
        if nbytes == 0:
            return None, 0
        if self._scratch is None or self._scratch.numel() < nbytes:
            # deferred calls keep pointers into earlier buffers: retire, do not free
            if self._scratch is not None:
                self._retired.append(self._scratch)
            self._scratch = self.torch.empty(nbytes, dtype=self.torch.uint8, device=self.device)
        return self._scratch.data_ptr(), nbytes

    def _stream(self):
        return self.torch.cuda.current_stream(self.device).cuda_stream

    # -- boundary calls -----------------------------------------------------
    # Each method marshals its arguments once and either issues the call or, with
    # defer=True, returns a closure that re-issues it (used by the benchmark so
    # that the timed region holds the C-ABI call and nothing else).
    def _issue(self, fn, where, head, tail, defer, keep=()):
        torch, device = self.torch, self.device

        def call(_keep=keep):        # the closure owns the buffers whose addresses it passes
            _check(fn(torch.cuda.current_stream(device).cuda_stream, *head, *tail), where)
        if defer:
            return call
        call()
        return None

    def reduce(self, name, dtype, m, n, xs, x, ys, y, defer=False):
        sp, sb = self.scratch(self.lib.dlfx_reduce_scratch_bytes(dtype, m, n))
        return self._issue(self.lib.dlfx_reduce, "dlfx_reduce(%s)" % name,
                           (name.encode(), dtype, m, n),
                           (xs.rank, _arr(xs.extents), _arr(xs.strides), x.data_ptr(), xs.offset,
                            ys.rank, _arr(ys.extents), _arr(ys.strides), y.data_ptr(), ys.offset, sp, sb), defer, (x, y))

    def reduce_static(self, name, dtype, m, n, xs, x, ys, y, defer=False):
        """dlfx_reduce_static: the same reduction with the library's own static device scratch."""
        return self._issue(self.lib.dlfx_reduce_static, "dlfx_reduce_static(%s)" % name,
                           (name.encode(), dtype, m, n),
                           (xs.rank, _arr(xs.extents), _arr(xs.strides), x.data_ptr(), xs.offset,
                            ys.rank, _arr(ys.extents), _arr(ys.strides), y.data_ptr(), ys.offset), defer, (x, y))

    def logits_head(self, dtype, m, n, x, x_offset, row_stride, sums, maxs, argmaxs, lses, k, best_values, best_indices,
                    defer=False):
        """dlfx_logits_head: sum, max, argmax, log-sum-exp and the k best of every row in one launch;
        any output (a device tensor) may be None."""
        def ptr(t):
            return None if t is None else t.data_ptr()
        return self._issue(self.lib.dlfx_logits_head, "dlfx_logits_head", (dtype, m, n),
                           (x.data_ptr(), x_offset, row_stride, ptr(sums), ptr(maxs), ptr(argmaxs), ptr(lses), k,
                            ptr(best_values), ptr(best_indices)), defer,
                           (x, sums, maxs, argmaxs, lses, best_values, best_indices))

    def arg_reduce(self, name, dtype, index_dtype, rows, k, xs, x, ys, y, defer=False):
        sp, sb = self.scratch(self.lib.dlfx_arg_reduce_scratch_bytes(dtype, rows, k))
        return self._issue(self.lib.dlfx_arg_reduce, "dlfx_arg_reduce(%s)" % name,
                           (name.encode(), dtype, index_dtype, rows, k),
                           (xs.rank, _arr(xs.extents), _arr(xs.strides), x.data_ptr(), xs.offset,
                            ys.rank, _arr(ys.extents), _arr(ys.strides), y.data_ptr(), ys.offset, sp, sb), defer, (x, y))

    def scan(self, name, dtype, m, n, exclusive, xs, x, ys, y, defer=False):
        sp, sb = self.scratch(self.lib.dlfx_scan_scratch_bytes(dtype, m, n))
        return self._issue(self.lib.dlfx_scan, "dlfx_scan(%s)" % name,
                           (name.encode(), dtype, m, n, int(bool(exclusive))),
                           (xs.rank, _arr(xs.extents), x.data_ptr(), xs.offset, _arr(xs.strides),
                            y.data_ptr(), ys.offset, _arr(ys.strides), sp, sb), defer, (x, y))

    def sort(self, direction, dtype, xs, x, ys, y, defer=False):
        n = xs.extents[-1]
        sp, sb = self.scratch(self.lib.dlfx_sort_scratch_bytes(dtype, xs.size // n, n))
        return self._issue(self.lib.dlfx_sort, "dlfx_sort", (direction, dtype),
                           (xs.rank, _arr(xs.extents), x.data_ptr(), xs.offset, _arr(xs.strides),
                            y.data_ptr(), ys.offset, _arr(ys.strides), sp, sb), defer, (x, y))

    def argsort(self, direction, dtype, index_dtype, xs, x, ys, y, is_, i, defer=False):
        n = xs.extents[-1]
        sp, sb = self.scratch(self.lib.dlfx_argsort_scratch_bytes(dtype, xs.size // n, n))
        return self._issue(self.lib.dlfx_argsort, "dlfx_argsort", (direction, dtype, index_dtype),
                           (xs.rank, _arr(xs.extents), x.data_ptr(), xs.offset, _arr(xs.strides),
                            y.data_ptr() if y is not None else None,
                            ys.offset if ys is not None else 0,
                            _arr(ys.strides) if ys is not None else None,
                            i.data_ptr(), is_.offset, _arr(is_.strides), sp, sb), defer, (x, y, i))

    def top_k(self, limit, direction, dtype, index_dtype, xs, x, ys, y, is_, i, defer=False):
        n = xs.extents[-1]
        sp, sb = self.scratch(self.lib.dlfx_top_k_scratch_bytes(dtype, xs.size // n, n, limit))
        return self._issue(self.lib.dlfx_top_k, "dlfx_top_k", (limit, direction, dtype, index_dtype),
                           (xs.rank, _arr(xs.extents), _arr(ys.extents),
                            x.data_ptr(), xs.offset, _arr(xs.strides),
                            y.data_ptr(), ys.offset, _arr(ys.strides),
                            i.data_ptr(), is_.offset, _arr(is_.strides), sp, sb), defer, (x, y, i))

    def count(self, dtype, m, n, value, xs, x, ys, y, defer=False):
        sp, sb = self.scratch(self.lib.dlfx_count_scratch_bytes(dtype, m, n))
        host_types = {0: np.float32, 1: np.float64, 2: np.int32, 3: np.int64, 4: np.float16, 5: np.int16,
                      7: np.complex64, 8: np.complex128}
        v = np.array([value], dtype=host_types[dtype])       # one host element of the input's type
        keep = v.ctypes.data_as(c_void_p)
        call = self._issue(self.lib.dlfx_count, "dlfx_count", (dtype, m, n, keep),
                           (xs.rank, _arr(xs.extents), _arr(xs.strides), x.data_ptr(), xs.offset,
                            ys.rank, _arr(ys.extents), _arr(ys.strides), y.data_ptr(), ys.offset, sp, sb), defer, (x, y))
        if call is None:
            return None
        return lambda v=v: call()      # the closure keeps the host value alive

    def scan_nonzero(self, dtype, m, n, exclusive, xs, x, ys, y, defer=False):
        sp, sb = self.scratch(self.lib.dlfx_scan_nonzero_scratch_bytes(dtype, m, n))
        return self._issue(self.lib.dlfx_scan_nonzero, "dlfx_scan_nonzero", (dtype, m, n, int(bool(exclusive))),
                           (xs.rank, _arr(xs.extents), x.data_ptr(), xs.offset, _arr(xs.strides),
                            y.data_ptr(), ys.offset, _arr(ys.strides), sp, sb), defer, (x, y))

    def gather_indices(self, m, n, row_major, dims, counts, out, defer=False):
        return self._issue(self.lib.dlfx_gather_indices, "dlfx_gather_indices", (m, n, int(bool(row_major))),
                           (len(dims), _arr(dims), counts.data_ptr(), 0, out.data_ptr(), 0), defer, (counts, out))

    def softmax(self, name, dtype, m, n, x, x_offset, y, y_offset, defer=False):
        sp, sb = self.scratch(self.lib.dlfx_softmax_scratch_bytes(dtype, m, n))
        return self._issue(self.lib.dlfx_softmax, "dlfx_softmax(%s)" % name, (name.encode(), dtype, m, n),
                           (x.data_ptr(), x_offset, y.data_ptr(), y_offset, sp, sb), defer, (x, y))

    def merge(self, direction, dtype, xs, x, ys, y, zs, z, defer=False):
        n = zs.extents[-1]
        sp, sb = self.scratch(self.lib.dlfx_merge_scratch_bytes(dtype, zs.size // n, n))
        return self._issue(self.lib.dlfx_merge, "dlfx_merge", (direction, dtype, zs.rank),
                           (_arr(xs.extents), _arr(xs.strides), x.data_ptr(), xs.offset,
                            _arr(ys.extents), _arr(ys.strides), y.data_ptr(), ys.offset,
                            _arr(zs.extents), _arr(zs.strides), z.data_ptr(), zs.offset, sp, sb), defer, (x, y, z))

    def read_element(self, storage, index):
        """One element of a device buffer on the host (synchronises the stream)."""
        return storage[index].item()

    def set_tuning(self, key: str, value: int):
        _check(self.lib.dlfx_set_tuning(key.encode(), value), "dlfx_set_tuning(%s)" % key)

    def synchronize(self):
        self.torch.cuda.synchronize(self.device)
