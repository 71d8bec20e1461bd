"""Pins the CPU oracle against independent library routines (numpy) and closed
forms, on strided / transposed / flipped views, so that a dropped term, wrong
index or transposed operand in the restatement fails here."""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import normal, randint, full_range_i64, uniform01


def T(be, a):
    return Tensor.from_numpy(be, a)


@pytest.mark.parametrize("axes,keep", [((), False), ((0,), False), ((1,), True), ((2,), False),
                                       ((0, 2), False), ((1, 2), True), ((-1,), False)])
def test_reduce_int_matches_numpy(oracle_backend, axes, keep):
    x = randint(11, 7 * 9 * 300, -50, 50).astype(np.int64).reshape(7, 9, 300)
    X = T(oracle_backend, x)
    ax = tuple(a % 3 for a in axes) or None
    assert np.array_equal(F.reduce_sum(X, axes, keep).numpy(), x.sum(axis=ax, keepdims=keep))
    assert np.array_equal(F.reduce_max(X, axes, keep).numpy(), x.max(axis=ax, keepdims=keep))
    assert np.array_equal(F.reduce_min(X, axes, keep).numpy(), x.min(axis=ax, keepdims=keep))
    n = x.size // x.sum(axis=ax, keepdims=keep).size
    # integer mean truncates toward zero (C++ division), unlike numpy's floor division
    want = np.trunc(x.sum(axis=ax, keepdims=keep) / n).astype(np.int64)
    assert np.array_equal(F.reduce_mean(X, axes, keep).numpy(), want)


def test_reduce_int32_sum_wraps(oracle_backend):
    x = np.full((3, 5000), 2**30, dtype=np.int32)
    got = F.reduce_sum(T(oracle_backend, x), [1]).numpy()
    assert np.array_equal(got, x.astype(np.int64).sum(axis=1).astype(np.int32))


def test_reduce_float_close_to_numpy_f64(oracle_backend):
    x = normal(12, 40 * 5000).astype(np.float32).reshape(40, 5000)
    X = T(oracle_backend, x)
    x64 = x.astype(np.float64)
    np.testing.assert_allclose(F.reduce_sum(X, [1]).numpy(), x64.sum(axis=1), rtol=0, atol=1e-3)
    np.testing.assert_allclose(F.reduce_mean(X, [0]).numpy(), x64.mean(axis=0), rtol=0, atol=1e-5)
    np.testing.assert_allclose(F.reduce_log_sum_exp(X, [1]).numpy(), np.log(np.exp(x64).sum(axis=1)), rtol=1e-5)
    np.testing.assert_allclose(F.reduce_sum_square(X, [1]).numpy(), (x64 * x64).sum(axis=1), rtol=1e-5)
    np.testing.assert_allclose(F.reduce_nrm2(X, [1]).numpy(), np.sqrt((x64 * x64).sum(axis=1)), rtol=1e-5)
    np.testing.assert_allclose(F.reduce_asum(X, [1]).numpy(), np.abs(x64).sum(axis=1), rtol=1e-5)
    assert np.array_equal(F.reduce_amax(X, [1]).numpy(), np.abs(x).max(axis=1))
    assert np.array_equal(F.reduce_amin(X, [1]).numpy(), np.abs(x).min(axis=1))


def test_log_sum_exp_is_naive_and_overflows(oracle_backend):
    # xfn.h:779-791: log(sum(exp(x))) without a max shift
    x = np.array([[1.0, 2.0, 3.0], [100.0, 0.0, 0.0]], dtype=np.float32)
    got = F.reduce_log_sum_exp(T(oracle_backend, x), [1]).numpy()
    assert np.isclose(got[0], np.log(np.exp(1.0) + np.exp(2.0) + np.exp(3.0)), rtol=1e-6)
    assert np.isposinf(got[1])


def test_reduce_f64_evaluator(oracle_backend):
    from oracle import oracle as O
    x = normal(13, 6 * 4000).astype(np.float32).reshape(6, 4000)
    X = T(oracle_backend, x)
    view, _, m, n = F.prepare_reduce(X.shape, [1], False)
    got = O.reduce_f64("reduce_sum", 0, m, n, view, X.storage)
    np.testing.assert_allclose(got, x.astype(np.float64).sum(axis=1), rtol=1e-13)
    view, _, m, n = F.prepare_reduce(X.shape, [0], False)
    got = O.reduce_f64("reduce_mean", 0, m, n, view, X.storage)
    np.testing.assert_allclose(got, x.astype(np.float64).mean(axis=0), rtol=1e-13)


@pytest.mark.parametrize("axis", [0, 1, 2, -1])
@pytest.mark.parametrize("keep", [True, False])
def test_argmax_argmin_match_numpy_first_occurrence(oracle_backend, axis, keep):
    x = randint(14, 6 * 7 * 50, 0, 5).astype(np.int32).reshape(6, 7, 50)   # many ties
    X = T(oracle_backend, x)
    want_max = np.argmax(x, axis=axis)
    want_min = np.argmin(x, axis=axis)
    if keep:
        want_max, want_min = np.expand_dims(want_max, axis), np.expand_dims(want_min, axis)
    assert np.array_equal(F.argmax(X, axis, keep).numpy(), want_max)
    assert np.array_equal(F.argmin(X, axis, keep).numpy(), want_min)


def test_argmax_transposed_view(oracle_backend):
    # DNNTest.cpp:1011-1017: argmax(X.transpose(), 0) == argmax(X, -1).transpose()
    x = randint(15, 4 * 5 * 6, 0, 100).astype(np.int32).reshape(4, 5, 6)
    X = T(oracle_backend, x)
    a = F.argmax(X.transpose(), 0).numpy()
    b = F.argmax(X, -1).numpy().transpose()
    assert np.array_equal(a, b)


def test_argmax_nan_rule(oracle_backend):
    x = np.array([[1.0, np.nan, 2.0], [np.nan, 5.0, 7.0]], dtype=np.float32)
    assert F.argmax(T(oracle_backend, x), 1, False).numpy().tolist() == [2, 0]


@pytest.mark.parametrize("axis", [0, 1, 2])
@pytest.mark.parametrize("exclusive", [False, True])
@pytest.mark.parametrize("reverse", [False, True])
def test_cumsum_int_matches_numpy(oracle_backend, axis, exclusive, reverse):
    x = randint(16, 5 * 3000 * 4, 0, 100).astype(np.int32).reshape(5, 3000, 4)
    got = F.cumsum(T(oracle_backend, x), axis, exclusive, reverse).numpy()
    xx = np.flip(x, axis) if reverse else x
    want = np.cumsum(xx, axis=axis, dtype=np.int32)
    if exclusive:
        want = want - xx
    if reverse:
        want = np.flip(want, axis)
    assert np.array_equal(got, want)


def test_cumprod_cummax_cummin(oracle_backend):
    x = randint(17, 3 * 2500, 1, 3).astype(np.int64).reshape(3, 2500)
    assert np.array_equal(F.cumprod(T(oracle_backend, x), 1).numpy(), np.cumprod(x, axis=1))
    y = normal(18, 3 * 2500).astype(np.float32).reshape(3, 2500)
    assert np.array_equal(F.cummax(T(oracle_backend, y), 1).numpy(), np.maximum.accumulate(y, axis=1))
    assert np.array_equal(F.cummin(T(oracle_backend, y), 1).numpy(), np.minimum.accumulate(y, axis=1))


def test_cumsum_in_place_and_random_int_property(oracle_backend):
    # UniformTest.cpp:2188-2189 uses a [2, 100000] random int tensor
    x = full_range_i64(19, 2 * 100000).astype(np.int32).reshape(2, 100000)
    X = T(oracle_backend, x)
    F.cumsum(X, 1, out=X)
    assert np.array_equal(X.numpy(), np.cumsum(x, axis=1, dtype=np.int32))


def test_scan_f64_evaluator(oracle_backend):
    from oracle import oracle as O
    x = normal(20, 3 * 5000).astype(np.float32).reshape(3, 5000)
    X = T(oracle_backend, x)
    y, mag = O.scan_f64("cumsum", 0, 3, 5000, False, X.shape, X.storage)
    np.testing.assert_allclose(y, np.cumsum(x.astype(np.float64), axis=1), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(mag, np.cumsum(np.abs(x.astype(np.float64)), axis=1), rtol=1e-12)


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
@pytest.mark.parametrize("axis", [0, 1, 2])
@pytest.mark.parametrize("desc", [False, True])
def test_sort_matches_numpy(oracle_backend, dtype, axis, desc):
    x = randint(21, 4 * 1500 * 3, -1000, 1000).astype(dtype).reshape(4, 1500, 3)
    got = F.sort(T(oracle_backend, x), axis, desc).numpy()
    want = np.sort(x, axis=axis)
    if desc:
        want = np.flip(want, axis)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("n", [1, 2, 10, 99, 100, 101, 500, 501, 1000, 1001, 2500, 10000])
def test_sort_sizes_and_in_place(oracle_backend, n):
    x = randint(22 + n, 2 * n, 0, 2000).astype(np.int32).reshape(2, n)
    X = T(oracle_backend, x)
    F.sort(X, -1, out=X)
    assert np.array_equal(X.numpy(), np.sort(x, axis=-1))


@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("desc", [False, True])
def test_argsort_is_stable_like_numpy(oracle_backend, axis, desc):
    x = randint(23, 300 * 7, 0, 8).astype(np.int32).reshape(300, 7)          # heavy duplicates
    X = T(oracle_backend, x)
    I = F.argsort(X, axis, desc).numpy()
    key = -x.astype(np.int64) if desc else x
    want = np.argsort(key, axis=axis, kind="stable")
    assert np.array_equal(I, want)
    Y, I2 = F.argsort(X, axis, desc, with_values=True)
    assert np.array_equal(I2.numpy(), want)
    assert np.array_equal(Y.numpy(), np.take_along_axis(x, want, axis=axis))


def test_argsort_long_rows_stable(oracle_backend):
    x = (uniform01(24, 3 * 20000) * 64).astype(np.float32).astype(np.int64).astype(np.float32).reshape(3, 20000)
    I = F.argsort(T(oracle_backend, x), -1).numpy()
    assert np.array_equal(I, np.argsort(x, axis=-1, kind="stable"))


@pytest.mark.parametrize("largest", [True, False])
@pytest.mark.parametrize("k", [1, 5, 50, 256])
def test_top_k_spec_and_heap_agree_on_values(oracle_backend, largest, k):
    from oracle.oracle import OracleBackend
    x = np.round(normal(25, 20 * 3000) * 2 * 256) / 256          # ties occur
    x = x.astype(np.float32).reshape(20, 3000)
    ys, is_ = F.top_k(T(oracle_backend, x), k, -1, largest)
    yh, ih = F.top_k(T(OracleBackend(topk_mode=0), x), k, -1, largest)
    ys, is_, yh, ih = ys.numpy(), is_.numpy(), yh.numpy(), ih.numpy()
    key = -x.astype(np.float64) if largest else x.astype(np.float64)
    order = np.argsort(key, axis=-1, kind="stable")[:, :k]
    assert np.array_equal(is_, order)                                   # lowest index on ties
    assert np.array_equal(ys, np.take_along_axis(x, order, axis=-1))
    assert np.array_equal(yh, ys)                                       # reference heap: same values
    assert np.array_equal(np.take_along_axis(x, ih.astype(np.int64), axis=-1), yh)


def test_top_k_axis_and_clamp(oracle_backend):
    x = randint(26, 6 * 9, 0, 1000).astype(np.int64).reshape(6, 9)
    y, i = F.top_k(T(oracle_backend, x), 100, 0, True, index_dtype=np.int64)
    assert y.numpy().shape == (6, 9)                                    # k clamps to the extent
    assert np.array_equal(y.numpy(), np.flip(np.sort(x, axis=0), 0))
    assert i.numpy().dtype == np.int64


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
@pytest.mark.parametrize("axes,keep", [((), False), ((0,), False), ((1,), True), ((0, 2), False), ((-1,), True)])
def test_count_matches_numpy(oracle_backend, dtype, axes, keep):
    x = randint(31, 5 * 6 * 70, -3, 4).astype(dtype).reshape(5, 6, 70)
    ax = tuple(a % 3 for a in axes) or None
    for view, ref in ((T(oracle_backend, x), x), (T(oracle_backend, x).transpose([2, 0, 1]), x.transpose(2, 0, 1))):
        for value in (0, 2, -3, 9):
            got = F.count(view, value, axes, keep).numpy()
            assert got.dtype == np.int32
            assert np.array_equal(got, (ref == value).sum(axis=ax, keepdims=keep))


def test_count_float_special_values(oracle_backend):
    x = np.array([0.0, -0.0, np.nan, 1.5, np.inf, -0.0], dtype=np.float32)
    X = T(oracle_backend, x)
    assert F.count(X, 0.0).numpy() == 3              # -0.0 == 0.0
    assert F.count(X, np.nan).numpy() == 0           # NaN equals nothing
    assert F.count(X, np.inf).numpy() == 1


@pytest.mark.parametrize("dtype", [np.float32, np.int64])
def test_nonzero_matches_numpy(oracle_backend, dtype):
    x = (randint(32, 4 * 5 * 37, 0, 3) * (randint(33, 4 * 5 * 37, 0, 2))).astype(dtype).reshape(4, 5, 37)
    for view, ref in ((T(oracle_backend, x), x), (T(oracle_backend, x).transpose([1, 2, 0]), x.transpose(1, 2, 0)),
                      (T(oracle_backend, x).slice([1], [36], [2], [3]), x[:, :, 1:36:3])):
        want = np.argwhere(ref != 0).astype(np.int32)           # row-major order of the view
        assert np.array_equal(F.nonzero(view).numpy(), want)
        assert np.array_equal(F.nonzero(view, True).numpy(), want.T)
    assert F.nonzero(T(oracle_backend, np.zeros((3, 4), dtype=dtype))) is None


@pytest.mark.parametrize("dtype", [np.int32, np.float64])
@pytest.mark.parametrize("desc", [False, True])
def test_merge_matches_numpy(oracle_backend, dtype, desc):
    # UniformTest.cpp:2250-2283: merge of sorted inputs == std::merge (one sorted sequence)
    for na, nb in ((2000, 3000), (1, 7), (500, 0 + 1), (1500, 1500)):
        a = np.sort(randint(40, 3 * na, -1000, 1000).astype(dtype).reshape(3, na), axis=1)
        b = np.sort(randint(41, 3 * nb, -1000, 1000).astype(dtype).reshape(3, nb), axis=1)
        if desc:
            a, b = a[:, ::-1].copy(), b[:, ::-1].copy()
        want = np.sort(np.concatenate([a, b], axis=1), axis=1)
        if desc:
            want = want[:, ::-1]
        got = F.merge(T(oracle_backend, a), T(oracle_backend, b), -1, desc).numpy()
        assert np.array_equal(got, want)
    # along axis 0 of transposed data
    a = np.sort(randint(42, 40 * 6, 0, 50).astype(dtype).reshape(40, 6), axis=0)
    b = np.sort(randint(43, 25 * 6, 0, 50).astype(dtype).reshape(25, 6), axis=0)
    got = F.merge(T(oracle_backend, a), T(oracle_backend, b), 0).numpy()
    assert np.array_equal(got, np.sort(np.concatenate([a, b], axis=0), axis=0))


def test_merge_keeps_first_input_first_on_ties(oracle_backend):
    a = np.array([-1.0, 0.0, 0.0, 2.0], dtype=np.float32)
    b = np.array([-0.0, -0.0, 2.0], dtype=np.float32)
    got = F.merge(T(oracle_backend, a), T(oracle_backend, b)).numpy()
    assert got.tolist() == [-1.0, 0.0, 0.0, 0.0, 0.0, 2.0, 2.0]
    assert np.signbit(got).tolist() == [True, False, False, True, True, False, False]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_softmax_family_matches_closed_forms(oracle_backend, dtype):
    from scipy.special import softmax as sp_softmax, log_softmax as sp_log_softmax
    x = (normal(50, 6 * 5 * 40) * 3).astype(dtype).reshape(6, 5, 40)
    X = T(oracle_backend, x)
    tol = 2e-6 if dtype == np.float32 else 1e-13
    for axis in (0, 1, 2, -1):
        a = axis % 3
        m = int(np.prod(x.shape[:a]))
        flat = x.reshape(m, -1).astype(np.float64)
        assert np.allclose(F.softmax(X, axis).numpy().reshape(m, -1), sp_softmax(flat, axis=1), rtol=tol * 50, atol=tol)
        assert np.allclose(F.logsoftmax(X, axis).numpy().reshape(m, -1), sp_log_softmax(flat, axis=1), rtol=tol * 50, atol=tol * 50)
        hm = F.hardmax(X, axis).numpy().reshape(m, -1)
        want = np.zeros_like(flat)
        want[np.arange(m), flat.argmax(axis=1)] = 1
        assert np.array_equal(hm, want)
    # a transposed input is copied to row-major order first (dnn.h:452: reorder(X, Y))
    Xt = X.transpose([2, 0, 1])
    xt = x.transpose(2, 0, 1)
    assert np.allclose(F.softmax(Xt, 1).numpy().reshape(40, -1), sp_softmax(xt.reshape(40, -1).astype(np.float64), axis=1),
                       rtol=tol * 50, atol=tol)


# ---------------------------------------------------------------- 16-bit element types
# The oracle widens float16 / int16 / bool exactly to float / int32 and narrows the result:
# checked here against numpy on the 16-bit arrays themselves (stable sorts: numpy's default
# float16 sort returned unsorted rows on this host).
@pytest.mark.parametrize("dtype", [np.float16, np.int16])
def test_sixteen_bit_order_ops_match_numpy(oracle_backend, dtype):
    x = (normal(140, 4 * 500) * 20).astype(dtype).reshape(4, 500)
    X = Tensor.from_numpy(oracle_backend, x)
    assert np.array_equal(F.sort(X, -1).numpy(), np.sort(x, axis=1, kind="stable"))
    assert F.sort(X, -1).numpy().dtype == dtype
    assert np.array_equal(F.argsort(X, -1).numpy(), np.argsort(x, axis=1, kind="stable"))
    assert np.array_equal(F.argsort(X, -1, True).numpy(), np.argsort(-x.astype(np.float64), axis=1, kind="stable"))
    assert np.array_equal(F.argmax(X, 1, False).numpy(), x.argmax(axis=1))
    assert np.array_equal(F.argmin(X, 0, False).numpy(), x.argmin(axis=0))
    assert np.array_equal(F.reduce("reduce_max", X, (1,)).numpy(), x.max(axis=1))
    Y, I = F.top_k(X, 7, -1)
    want = np.argsort(-x.astype(np.float64), axis=1, kind="stable")[:, :7]
    assert np.array_equal(I.numpy(), want) and np.array_equal(Y.numpy(), np.take_along_axis(x, want, 1))
    a, b = np.sort(x, axis=1, kind="stable"), np.sort(x[::-1] * 1, axis=1, kind="stable")
    assert np.array_equal(F.merge(Tensor.from_numpy(oracle_backend, a), Tensor.from_numpy(oracle_backend, b)).numpy(),
                          np.sort(np.concatenate([a, b], 1), axis=1, kind="stable"))
    assert np.array_equal(F.count(X, dtype(3), (1,)).numpy(), (x == dtype(3)).sum(axis=1))
    assert np.array_equal(F.nonzero(X).numpy(), np.argwhere(x != 0))


def test_half_sums_round_once(oracle_backend):
    x = (normal(141, 3 * 200) * 0.5).astype(np.float16).reshape(3, 200)
    X = Tensor.from_numpy(oracle_backend, x)
    got = F.reduce("reduce_sum", X, (1,)).numpy()
    assert got.dtype == np.float16
    # the float sum of 200 halves of this size is within an ulp32 or two of exact; its half
    # rounding is one of the two halves around the exact sum
    exact = x.astype(np.float64).sum(axis=1)
    assert (np.abs(got.astype(np.float64) - exact) <= np.abs(exact) * 2.0 ** -10 + 2.0 ** -24).all()
    cs = F.cumsum(X, 1).numpy().astype(np.float64)
    ce = np.cumsum(x.astype(np.float64), axis=1)
    assert (np.abs(cs - ce) <= np.abs(ce) * 2.0 ** -10 + 1e-4).all()
    assert np.array_equal(F.cummax(X, 1).numpy(), np.maximum.accumulate(x, axis=1))


def test_bool_nonzero(oracle_backend):
    b = randint(142, 6 * 40, 0, 3).reshape(6, 40) == 0
    assert np.array_equal(F.nonzero(Tensor.from_numpy(oracle_backend, b)).numpy(), np.argwhere(b))


# ---------------------------------------------------------------- complex elements
@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
def test_complex_reduce_count_scan_match_numpy(oracle_backend, dtype):
    n = 4 * 9 * 50
    x = ((normal(143, n) + 1j * normal(144, n)) * 0.7).astype(dtype).reshape(4, 9, 50)
    X = Tensor.from_numpy(oracle_backend, x)
    x128 = x.astype(np.complex128)
    rtol = 200 * np.finfo(dtype).eps
    for axes in ((), (1,), (0, 2)):
        ax = axes if axes else None
        cases = {"reduce_sum": x128.sum(axis=ax), "reduce_mean": x128.mean(axis=ax),
                 "reduce_asum": np.abs(x128).sum(axis=ax), "reduce_sum_square": (x128 * x128).sum(axis=ax),
                 "reduce_nrm2": np.sqrt((np.abs(x128) ** 2).sum(axis=ax)),
                 "reduce_sum_exp": np.exp(x128).sum(axis=ax), "reduce_log_sum": np.log(x128.sum(axis=ax)),
                 "reduce_log_sum_exp": np.log(np.exp(x128).sum(axis=ax))}
        for name, want in cases.items():
            got = F.reduce(name, X, axes).numpy()
            assert got.dtype == dtype
            assert np.allclose(got.reshape(-1), np.asarray(want).reshape(-1), rtol=rtol, atol=rtol * 50), name
    u = np.exp(1j * normal(145, 3 * 40).reshape(3, 40)).astype(dtype)
    U = Tensor.from_numpy(oracle_backend, u)
    assert np.allclose(F.reduce("reduce_prod", U, (1,)).numpy(), u.astype(np.complex128).prod(axis=1), rtol=rtol, atol=rtol)
    assert np.allclose(F.cumprod(U, 1).numpy(), np.cumprod(u.astype(np.complex128), axis=1), rtol=rtol, atol=rtol)
    assert np.allclose(F.cumsum(X, 1, exclusive=True).numpy()[:, 1:], np.cumsum(x128, axis=1)[:, :-1], rtol=rtol, atol=rtol * 50)
    y = (randint(146, 200, 0, 2) + 1j * randint(147, 200, 0, 2)).astype(dtype).reshape(4, 50)
    assert np.array_equal(F.count(Tensor.from_numpy(oracle_backend, y), 1 + 1j, (1,)).numpy(), (y == 1 + 1j).sum(axis=1))
    for name in ("reduce_max", "reduce_amin"):
        with pytest.raises(Exception):
            F.reduce(name, X, ())
    with pytest.raises(Exception):
        F.cummax(X, 1)


def test_complex_nrm2_reference_vector(oracle_backend):
    # dlf/test/UniformTest.cpp:2060-2063
    x = np.array([3 + 4j, 5 + 12j], dtype=np.complex64)
    got = F.reduce("reduce_nrm2", Tensor.from_numpy(oracle_backend, x), (0,)).numpy()
    assert got.reshape(-1)[0] == np.complex64(np.sqrt(np.float32(194.0)))
