"""dlfx_reduce_static (no scratch argument, no allocation: partial accumulators live in a static
device array of the library) against dlfx_reduce on the same inputs, through the C ABI.

Each case issues two calls in a row, the second with a smaller input, so that the second call
finds the first one's partials in the array.  Integer sums and max / min must be equal bit for
bit; fp32 sums must agree within 4 ulp x log2(n) of max(|sum|, sum |x_i|) (both entry points run
the same kernels in the same order, so in practice they are equal too, which is also asserted).
"""
import ctypes

import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor, prepare_reduce
from dlf_amd.hip_backend import load_library
from helpers import normal, randint, ulp_bound

pytestmark = pytest.mark.gpu


def reduce_both(hip, name, x, axes):
    """(dlfx_reduce result, dlfx_reduce_static result) as flat numpy arrays."""
    X = Tensor.from_numpy(hip, x)
    view, out_dims, m, n = prepare_reduce(X.shape, list(axes), False)
    code = F.dtype_code(X.dtype)
    Yd = Tensor.empty(hip, out_dims, X.dtype)
    Ys = Tensor.empty(hip, out_dims, X.dtype)
    Ys.storage.fill_(0)
    hip.reduce(name, code, m, n, view, X.storage, Yd.shape, Yd.storage)
    hip.reduce_static(name, code, m, n, view, X.storage, Ys.shape, Ys.storage)
    hip.synchronize()
    return Yd.numpy().reshape(-1), Ys.numpy().reshape(-1), n


def check(hip, name, x, axes):
    want, got, n = reduce_both(hip, name, x, axes)
    if x.dtype.kind == "f" and name in ("reduce_sum", "reduce_mean"):
        scale = np.maximum(np.abs(want.astype(np.float64)), np.abs(x.astype(np.float64)).sum() / max(1, want.size))
        assert (np.abs(got.astype(np.float64) - want) <= ulp_bound(n, scale)).all(), name
    assert np.array_equal(got, want), name


# (first shape, second smaller shape, reduced axes): every pair needs partial accumulators in both calls
PAIRS = [
    ((1 << 24,), (1 << 20,), [0]),                  # one long row cut into many workgroups
    ((3, 1 << 21), (2, 70001), [1]),                # a few long rows, ragged second
    ((2, 8192, 96), (1, 700, 64), [1]),             # strided reduced axis, contiguous kept axis (column kernel)
    ((4, 2048, 7, 9), (2, 515, 3, 20), [1]),        # the same over a merged inner extent
]


@pytest.mark.parametrize("first,second,axes", PAIRS)
@pytest.mark.parametrize("name,dtype", [("reduce_sum", np.float32), ("reduce_sum", np.int32), ("reduce_max", np.float32),
                                        ("reduce_min", np.int64), ("reduce_mean", np.float64)])
def test_static_scratch_matches_caller_scratch_twice_in_a_row(hip_backend, first, second, axes, name, dtype):
    lib = load_library()
    for seed, shape in ((11, first), (12, second)):
        count = int(np.prod(shape))
        m = count // int(np.prod([shape[a] for a in axes]))
        assert lib.dlfx_reduce_scratch_bytes(F.dtype_code(dtype), m, count // m) > 0
        if np.dtype(dtype).kind == "f":
            x = normal(seed, count).astype(dtype).reshape(shape)
        else:
            x = randint(seed, count, -1000, 1000).astype(dtype).reshape(shape)
        check(hip_backend, name, x, axes)


def test_short_rows_and_argument_errors(hip_backend):
    # rows that need no partials go through the same entry point
    x = normal(13, 256 * 1000).astype(np.float32).reshape(256, 1000)
    check(hip_backend, "reduce_sum", x, [1])
    check(hip_backend, "reduce_log_sum_exp", x, [1])
    lib = load_library()
    dims = (ctypes.c_int64 * 2)(4, 8)
    st = (ctypes.c_int64 * 2)(8, 1)
    one = (ctypes.c_int64 * 1)(4)
    s1 = (ctypes.c_int64 * 1)(1)
    fake = ctypes.c_void_p(0x1000)
    assert lib.dlfx_reduce_static(None, b"reduce_sum", 0, 4, 9, 2, dims, st, fake, 0, 1, one, s1, fake, 0) == -1
    assert lib.dlfx_reduce_static(None, b"nope", 0, 4, 8, 2, dims, st, fake, 0, 1, one, s1, fake, 0) == -3
    assert lib.dlfx_reduce_static(None, b"reduce_sum", 0, 0, 8, 2, dims, st, fake, 0, 1, one, s1, fake, 0) == -1
