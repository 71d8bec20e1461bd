"""merge: HIP path vs the CPU oracle (the reference's serial merge), bit-exact, including the
order of equal elements that differ in their bits (-0.0 / +0.0: first input first)."""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import randint, normal, full_range_i64

pytestmark = pytest.mark.gpu


def sorted_rows(dtype, seed, rows, n, desc, dup):
    if n == 0:
        return np.zeros((rows, 0), dtype=dtype)
    if dup:
        a = randint(seed, rows * n, -20, 20).astype(dtype)
    elif np.dtype(dtype).kind == "i":
        a = full_range_i64(seed, rows * n).astype(dtype)
    else:
        a = (normal(seed, rows * n) * 100).astype(dtype)
    a = np.sort(a.reshape(rows, n), axis=1, kind="stable")      # (the default kind mis-sorts float16 on some hosts)
    return a[:, ::-1].copy() if desc else a


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
@pytest.mark.parametrize("na,nb", [(1, 1), (1, 9), (100, 3), (2000, 3000), (2048, 2048), (5000, 4097), (70001, 12345)])
def test_merge_rows(hip_backend, oracle_backend, dtype, na, nb):
    for desc in (False, True):
        for dup in (False, True):
            a = sorted_rows(dtype, 90 + na, 3, na, desc, dup)
            b = sorted_rows(dtype, 91 + nb, 3, nb, desc, dup)
            g = F.merge(Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(hip_backend, b), -1, desc).numpy()
            w = F.merge(Tensor.from_numpy(oracle_backend, a), Tensor.from_numpy(oracle_backend, b), -1, desc).numpy()
            assert np.array_equal(g, w), (desc, dup)


def test_merge_batches_and_other_axes(hip_backend, oracle_backend):
    # UniformTest.cpp:2277-2283 (batch of rows) and a merge along the first axis of a 3-d tensor
    a = np.sort(randint(92, 100, 0, 1000).astype(np.int32).reshape(10, 10), axis=-1)
    b = np.sort(randint(93, 100, 0, 1000).astype(np.int32).reshape(10, 10), axis=-1)
    g = F.merge(Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(hip_backend, b)).numpy()
    assert np.array_equal(g, np.sort(np.concatenate([a, b], axis=1), axis=1))
    x = np.sort(randint(94, 300 * 4 * 5, 0, 50).astype(np.float32).reshape(300, 4, 5), axis=0)
    y = np.sort(randint(95, 500 * 4 * 5, 0, 50).astype(np.float32).reshape(500, 4, 5), axis=0)
    for be_pair in ((hip_backend, oracle_backend),):
        g = F.merge(Tensor.from_numpy(be_pair[0], x), Tensor.from_numpy(be_pair[0], y), 0).numpy()
        w = F.merge(Tensor.from_numpy(be_pair[1], x), Tensor.from_numpy(be_pair[1], y), 0).numpy()
        assert np.array_equal(g, w) and np.array_equal(g, np.sort(np.concatenate([x, y], axis=0), axis=0))


def test_merge_first_input_first_on_ties(hip_backend):
    a = np.array([[-1.0, 0.0, 0.0, 2.0]], dtype=np.float32)
    b = np.array([[-0.0, -0.0, 2.0]], dtype=np.float32)
    got = F.merge(Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(hip_backend, b)).numpy()[0]
    assert np.signbit(got).tolist() == [True, False, False, True, True, False, False]
    # long runs of equal keys across many tiles: the signs show which input an element came from
    za = np.zeros((2, 9000), dtype=np.float32)
    zb = -np.zeros((2, 7000), dtype=np.float32)
    got = F.merge(Tensor.from_numpy(hip_backend, za), Tensor.from_numpy(hip_backend, zb)).numpy()
    assert not np.signbit(got[:, :9000]).any() and np.signbit(got[:, 9000:]).all()


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64, np.float16, np.int16])
def test_merge_short_rows_packed_into_workgroups(hip_backend, oracle_backend, dtype):
    """Output rows of up to 2048 elements: several rows per workgroup, a team of 1 to 256
    threads per row.  Every team size and its neighbours, one-element sides, row counts that
    do not fill the last workgroup."""
    cases = [(1, 1), (1, 2), (2, 2), (3, 2), (4, 5), (8, 8), (9, 8), (17, 15), (32, 32), (33, 32), (64, 64), (100, 29),
             (128, 128), (129, 128), (1, 300), (511, 1), (512, 512), (513, 512), (1024, 1024), (1500, 549)]
    for idx, (na, nb) in enumerate(cases):
        rows = (1, 3, 67, 300)[idx % 4]
        for desc in (False, True):
            a = sorted_rows(dtype, 400 + idx, rows, na, desc, idx % 2 == 0)
            b = sorted_rows(dtype, 500 + idx, rows, nb, desc, idx % 2 == 0)
            g = F.merge(Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(hip_backend, b), -1, desc).numpy()
            w = F.merge(Tensor.from_numpy(oracle_backend, a), Tensor.from_numpy(oracle_backend, b), -1, desc).numpy()
            assert np.array_equal(g, w), (na, nb, rows, desc)
    # equal keys that differ in their bits: first input first, in every row of a packed workgroup
    za = np.zeros((500, 20), dtype=np.float32)
    zb = -np.zeros((500, 12), dtype=np.float32)
    got = F.merge(Tensor.from_numpy(hip_backend, za), Tensor.from_numpy(hip_backend, zb)).numpy()
    assert not np.signbit(got[:, :20]).any() and np.signbit(got[:, 20:]).all()


def test_merge_short_rows_of_views(hip_backend, oracle_backend):
    """Short rows along a strided axis and into a transposed output."""
    x = np.sort(randint(601, 40 * 6 * 50, -99, 99).astype(np.int32).reshape(40, 6, 50), axis=0)
    y = np.sort(randint(602, 24 * 6 * 50, -99, 99).astype(np.int32).reshape(24, 6, 50), axis=0)
    g = F.merge(Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(hip_backend, y), 0).numpy()
    w = F.merge(Tensor.from_numpy(oracle_backend, x), Tensor.from_numpy(oracle_backend, y), 0).numpy()
    assert np.array_equal(g, w) and np.array_equal(g, np.sort(np.concatenate([x, y], axis=0), axis=0))
    a = np.sort(normal(603, 300 * 70).astype(np.float32).reshape(300, 70), axis=1)
    b = np.sort(normal(604, 300 * 30).astype(np.float32).reshape(300, 30), axis=1)
    Ah, Bh = Tensor.from_numpy(hip_backend, a[:, ::-1].copy()).flip([1]), Tensor.from_numpy(hip_backend, b)
    got = F.merge(Ah, Bh).numpy()
    assert np.array_equal(got, np.sort(np.concatenate([a, b], axis=1), axis=1, kind="stable"))
