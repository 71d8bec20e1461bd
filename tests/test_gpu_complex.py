"""Complex elements (the reference's float2 / double2 instantiations of reduce, count and scan,
gpgpu/src/gdnn.cpp:865-875, 922-932, 975-984) on the HIP path.

Checked against numpy in complex128 (closed forms) to a stated bound, and against the CPU oracle
(std::complex arithmetic in the element type, as the reference's host templates) within the
oracle's own serial rounding.  count is exact."""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import normal, randint

pytestmark = pytest.mark.gpu


def cplx(seed, shape, dtype, scale=1.0):
    n = int(np.prod(shape))
    return ((normal(seed, n) + 1j * normal(seed + 1000, n)) * scale).astype(dtype).reshape(shape)


def close(got, want, rel, scale=None):
    scale = np.abs(want) if scale is None else scale
    return (np.abs(got.astype(np.complex128) - want) <= rel * scale + 1e-30).all()


@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
@pytest.mark.parametrize("axes", [(), (0,), (1,), (2,), (0, 2)])
def test_complex_reductions(hip_backend, oracle_backend, dtype, axes):
    x = cplx(160, (5, 37, 130), dtype, 0.7)
    X, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
    ax = axes if axes else None
    n = x.size // max(1, np.sum(x, axis=ax).size)
    eps = np.finfo(dtype).eps
    tol = 4 * max(1.0, np.log2(n)) * eps
    x128 = x.astype(np.complex128)
    mag = np.abs(x128).sum(axis=ax)
    want = {
        "reduce_sum": (x128.sum(axis=ax), mag),
        "reduce_mean": (x128.mean(axis=ax), mag / n),
        "reduce_asum": (np.abs(x128).sum(axis=ax) + 0j, mag),
        "reduce_sum_square": ((x128 * x128).sum(axis=ax), (np.abs(x128) ** 2).sum(axis=ax)),
        "reduce_nrm2": (np.sqrt((np.abs(x128) ** 2).sum(axis=ax)) + 0j, None),
        "reduce_sum_exp": (np.exp(x128).sum(axis=ax), np.abs(np.exp(x128)).sum(axis=ax)),
    }
    for name, (w, scale) in want.items():
        got = F.reduce(name, X, axes).numpy()
        assert got.dtype == dtype
        assert close(got.reshape(-1), np.asarray(w).reshape(-1), tol, None if scale is None else np.asarray(scale).reshape(-1)), name
        ref = F.reduce(name, Xo, axes).numpy()                     # serial folds in the element type
        assert close(ref.reshape(-1), np.asarray(w).reshape(-1), n * eps, None if scale is None else np.asarray(scale).reshape(-1)), name
    for name, inner in (("reduce_log_sum", x128.sum(axis=ax)), ("reduce_log_sum_exp", np.exp(x128).sum(axis=ax))):
        got = F.reduce(name, X, axes).numpy().reshape(-1).astype(np.complex128)
        w = np.log(np.asarray(inner).reshape(-1))
        cond = np.asarray(want["reduce_sum" if name == "reduce_log_sum" else "reduce_sum_exp"][1]).reshape(-1) / np.abs(np.asarray(inner).reshape(-1))
        assert (np.abs(got - w) <= tol * cond + 4 * eps * (1 + np.abs(w))).all(), name
    for name in ("reduce_max", "reduce_min", "reduce_amax", "reduce_amin"):
        with pytest.raises(Exception):
            F.reduce(name, X, axes)


@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
def test_complex_prod_nrm2_and_reference_vector(hip_backend, dtype):
    # dlf/test/UniformTest.cpp:2060-2063: nrm2 of {3+4i, 5+12i} is sqrt(194)
    x = np.array([3 + 4j, 5 + 12j], dtype=dtype)
    got = F.reduce("reduce_nrm2", Tensor.from_numpy(hip_backend, x), (0,)).numpy()
    assert abs(got.reshape(-1)[0] - np.sqrt(194.0)) <= 4 * np.finfo(dtype).eps * 14
    # products of numbers on the unit circle stay on it: arguments add up
    ph = (normal(161, 4 * 300) * 0.3).reshape(4, 300)
    u = np.exp(1j * ph).astype(dtype)
    got = F.reduce("reduce_prod", Tensor.from_numpy(hip_backend, u), (1,)).numpy().astype(np.complex128)
    want = np.exp(1j * np.angle(u.astype(np.complex128)).sum(axis=1))
    assert (np.abs(got - want) <= 300 * np.finfo(dtype).eps).all()
    # the logarithm takes the principal branch in every quadrant
    for z in (-4 + 0j, -3 - 4j, 3 - 4j, -1e-3 + 1e-9j, 2 + 5j):
        v = np.array([[z, 0]], dtype=dtype)
        got = F.reduce("reduce_log_sum", Tensor.from_numpy(hip_backend, v), (1,)).numpy().astype(np.complex128)[0]
        assert abs(got - np.log(np.complex128(v[0, 0]))) <= (1e-5 if dtype == np.complex64 else 1e-12)


@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
def test_complex_count(hip_backend, oracle_backend, dtype):
    re = randint(162, 6 * 5000, 0, 3).reshape(6, 5000)
    im = randint(163, 6 * 5000, 0, 3).reshape(6, 5000)
    x = (re + 1j * im).astype(dtype)
    X, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
    for value in (1 + 2j, 0j, 2 + 0j, 5 + 5j):
        for axes in ((), (0,), (1,)):
            got = F.count(X, value, axes).numpy()
            assert np.array_equal(got, F.count(Xo, value, axes).numpy())
            assert np.array_equal(got.reshape(-1), np.asarray((x == dtype(value)).sum(axis=axes if axes else None)).reshape(-1))


@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
@pytest.mark.parametrize("n", [1, 9, 300, 1500, 5000, 70000])
def test_complex_scans(hip_backend, oracle_backend, dtype, n):
    x = cplx(164 + n, (3, n), dtype, 0.5)
    X, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
    eps = np.finfo(dtype).eps
    x128 = x.astype(np.complex128)
    mag = np.cumsum(np.abs(x128), axis=1)
    for exclusive in (False, True):
        for reverse in (False, True):
            got = F.cumsum(X, 1, exclusive, reverse).numpy().astype(np.complex128)
            src = x128[:, ::-1] if reverse else x128
            w = np.cumsum(src, axis=1)
            if exclusive:
                w = np.concatenate([np.zeros((3, 1)), w[:, :-1]], axis=1)
            m_ = np.cumsum(np.abs(src), axis=1)
            if reverse:
                w, m_ = w[:, ::-1], m_[:, ::-1]
            assert (np.abs(got - w) <= 4 * max(1.0, np.log2(n)) * eps * m_ + 1e-30).all(), (exclusive, reverse)
    ref = F.cumsum(Xo, 1).numpy().astype(np.complex128)
    assert (np.abs(ref - np.cumsum(x128, axis=1)) <= n * eps * mag).all()
    # running products of unit-modulus numbers
    u = np.exp(1j * normal(165 + n, 3 * n).reshape(3, n) * 0.2).astype(dtype)
    got = F.cumprod(Tensor.from_numpy(hip_backend, u), 1).numpy().astype(np.complex128)
    want = np.exp(1j * np.cumsum(np.angle(u.astype(np.complex128)), axis=1))
    steps = np.arange(1, n + 1)[None, :]
    assert (np.abs(got - want) <= 4 * steps * eps).all()
    for name in ("cummax", "cummin"):
        with pytest.raises(Exception):
            getattr(F, name)(X, 1)


def test_complex_scan_other_axis_and_in_place(hip_backend):
    x = cplx(166, (40, 6, 5), np.complex64)
    X = Tensor.from_numpy(hip_backend, x)
    got = F.cumsum(X, 0).numpy()
    assert np.allclose(got, np.cumsum(x.astype(np.complex128), axis=0), rtol=1e-5, atol=1e-5)
    F.cumsum(X, 1, out=X)
    assert np.allclose(X.numpy(), np.cumsum(x.astype(np.complex128), axis=1), rtol=1e-5, atol=1e-5)
