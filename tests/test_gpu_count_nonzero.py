"""count / nonzero: HIP path vs the CPU oracle, bit-exact (integer results).

count is the reference's reduce with Map x == value (reduce.h:151-158); nonzero is
scan_nonzero + a read of the total + gather_indices (reduce.h:419-450)."""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import randint, normal

pytestmark = pytest.mark.gpu


def both(hip, orc, x):
    return Tensor.from_numpy(hip, x), Tensor.from_numpy(orc, x)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
@pytest.mark.parametrize("axes,keep", [((), False), ((0,), False), ((1,), True), ((2,), False), ((0, 2), True)])
def test_count_axes(hip_backend, oracle_backend, dtype, axes, keep):
    x = randint(80, 6 * 40 * 130, -3, 4).astype(dtype).reshape(6, 40, 130)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for value in (0, 3, 7):
        g = F.count(Xh, value, axes, keep).numpy()
        assert g.dtype == np.int32
        assert np.array_equal(g, F.count(Xo, value, axes, keep).numpy())
    # a non-contiguous view
    g = F.count(Xh.transpose([2, 0, 1]), 1, axes, keep).numpy()
    assert np.array_equal(g, F.count(Xo.transpose([2, 0, 1]), 1, axes, keep).numpy())


def test_count_long_rows_and_special_values(hip_backend, oracle_backend):
    x = randint(81, 3 * (1 << 20), 0, 5).astype(np.float32).reshape(3, 1 << 20)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    assert np.array_equal(F.count(Xh, 2.0, [1]).numpy(), F.count(Xo, 2.0, [1]).numpy())
    assert np.array_equal(F.count(Xh, 2.0).numpy(), (x == 2.0).sum().astype(np.int32))
    s = np.array([0.0, -0.0, np.nan, 1.5, np.inf, -0.0], dtype=np.float32)
    S = Tensor.from_numpy(hip_backend, s)
    assert F.count(S, 0.0).numpy() == 3 and F.count(S, np.nan).numpy() == 0 and F.count(S, np.inf).numpy() == 1


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_nonzero_views(hip_backend, oracle_backend, dtype):
    x = (randint(82, 7 * 33 * 50, 0, 3) * randint(83, 7 * 33 * 50, 0, 2)).astype(dtype).reshape(7, 33, 50)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for vh, vo, ref in ((Xh, Xo, x), (Xh.transpose([1, 2, 0]), Xo.transpose([1, 2, 0]), x.transpose(1, 2, 0)),
                        (Xh.slice([1], [49], [2], [3]), Xo.slice([1], [49], [2], [3]), x[:, :, 1:49:3])):
        for row_major in (False, True):
            g = F.nonzero(vh, row_major).numpy()
            assert np.array_equal(g, F.nonzero(vo, row_major).numpy())
        assert np.array_equal(F.nonzero(vh).numpy(), np.argwhere(ref != 0))
    assert F.nonzero(Tensor.from_numpy(hip_backend, np.zeros((5, 6), dtype=dtype))) is None


def test_nonzero_large_uses_chained_tiles(hip_backend, oracle_backend):
    # 3 * 2^20 elements: the running count crosses many 64 KB tiles of one row
    x = (normal(84, 3 << 20) > 1.0).astype(np.float32).reshape(3, 1 << 10, 1 << 10)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    g = F.nonzero(Xh).numpy()
    assert np.array_equal(g, F.nonzero(Xo).numpy())
    assert np.array_equal(g, np.argwhere(x != 0))
    # negative zero is zero, NaN is not
    s = np.array([[0.0, -0.0], [np.nan, 2.0]], dtype=np.float32)
    assert F.nonzero(Tensor.from_numpy(hip_backend, s)).numpy().tolist() == [[1, 0], [1, 1]]


def test_gather_indices_ignores_counts_beyond_n(hip_backend):
    # counts that run past the n the caller sized the output for must not be written anywhere
    from dlf_amd.frontend import dtype_code
    from dlf_amd.shape import Shape
    x = np.ones((4, 8), dtype=np.float32)
    X = Tensor.from_numpy(hip_backend, x)
    counts = Tensor.empty(hip_backend, [32], np.int32)
    hip_backend.scan_nonzero(dtype_code(np.float32), 1, 32, False, X.shape, X.storage, Shape([4, 8]), counts.storage)
    out = Tensor.from_numpy(hip_backend, np.full((20, 2), -7, dtype=np.int32))
    hip_backend.gather_indices(32, 5, False, [4, 8], counts.storage, out.storage)       # room for 5 of the 32
    got = out.numpy()
    assert got[:5].tolist() == [[0, 0], [0, 1], [0, 2], [0, 3], [0, 4]]
    assert (got[5:] == -7).all()
