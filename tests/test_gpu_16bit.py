"""16-bit element types (IEEE half, int16) and bool inputs on the HIP path vs the CPU oracle.

The oracle widens them exactly (half -> float, int16 / bool -> int32), so order-based results
(sort, argsort, top_k, merge, argmax, hardmax, count, nonzero) must match bit for bit; half sums
and scans are formed in fp32 and rounded once: |got - exact| <= 1 half ulp of the result plus
the fp32 bound 4 * log2(n) * eps32 * sum|x|."""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor, dtype_code
from oracle import oracle as O
from helpers import normal, randint

pytestmark = pytest.mark.gpu


def both(hip, orc, x):
    return Tensor.from_numpy(hip, x), Tensor.from_numpy(orc, x)


def halfs(seed, shape, scale=1.0):
    return (normal(seed, int(np.prod(shape))) * scale).astype(np.float16).reshape(shape)


def shorts(seed, shape, lo=-30000, hi=30000):
    return randint(seed, int(np.prod(shape)), lo, hi).astype(np.int16).reshape(shape)


@pytest.mark.parametrize("n", [1, 7, 100, 1000, 4097, 70001])
def test_sort_argsort_merge_bit_exact(hip_backend, oracle_backend, n):
    for x in (halfs(120 + n, (3, n), 10), shorts(121 + n, (3, n)), shorts(122 + n, (3, n), -5, 5),
              np.round(halfs(123 + n, (3, n), 3))):
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for desc in (False, True):
            assert np.array_equal(F.sort(Xh, -1, desc).numpy(), F.sort(Xo, -1, desc).numpy())
            Yh, Ih = F.argsort(Xh, -1, desc, with_values=True)
            Yo, Io = F.argsort(Xo, -1, desc, with_values=True)
            assert np.array_equal(Ih.numpy(), Io.numpy()) and np.array_equal(Yh.numpy().view(np.uint16), Yo.numpy().view(np.uint16))
        # (numpy's default sort of float16 returned unsorted rows on this host: use the stable kind)
        a = np.sort(x, axis=1, kind="stable")
        b = np.sort(x[:, ::-1] * 1, axis=1, kind="stable")[:, : max(1, n // 2)]
        g = F.merge(Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(hip_backend, b)).numpy()
        w = F.merge(Tensor.from_numpy(oracle_backend, a), Tensor.from_numpy(oracle_backend, b)).numpy()
        assert g.dtype == x.dtype and np.array_equal(g, w)


def test_sort_other_axis_and_signed_zero(hip_backend, oracle_backend):
    x = shorts(124, (40, 6, 5), -100, 100)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    assert np.array_equal(F.sort(Xh, 0).numpy(), np.sort(x, axis=0, kind="stable"))
    assert np.array_equal(F.argsort(Xh, 1, True).numpy(), F.argsort(Xo, 1, True).numpy())
    z = np.array([[0.0, -0.0, 1.0, -0.0, 0.0, -1.0]], dtype=np.float16)
    Y, I = F.argsort(Tensor.from_numpy(hip_backend, z), -1, with_values=True)
    assert I.numpy().tolist() == [[5, 0, 1, 3, 4, 2]]
    assert np.array_equal(np.signbit(Y.numpy()), np.signbit(z[0][I.numpy()[0]])[None, :])


@pytest.mark.parametrize("axes", [(), (0,), (1,), (2,), (0, 2)])
def test_half_reductions(hip_backend, oracle_backend, axes):
    x = halfs(125, (6, 40, 130), 0.5)       # sums of squares stay below the largest half
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for name in ("reduce_max", "reduce_min", "reduce_amax", "reduce_amin"):
        assert np.array_equal(F.reduce(name, Xh, axes).numpy(), F.reduce(name, Xo, axes).numpy()), name
    view, out_dims, m, n = F.prepare_reduce(Xo.shape, list(axes), False)
    for name in ("reduce_sum", "reduce_mean", "reduce_asum", "reduce_sum_square", "reduce_nrm2", "reduce_log_sum_exp"):
        got = F.reduce(name, Xh, axes).numpy().astype(np.float64).reshape(-1)
        exact = O.reduce_f64(name, dtype_code(np.float16), m, n, view, Xo.storage)
        mag = O.reduce_f64("reduce_asum", dtype_code(np.float16), m, n, view, Xo.storage)
        if name in ("reduce_sum_square", "reduce_nrm2", "reduce_log_sum_exp", "reduce_asum"):
            mag = np.abs(exact)
        if name == "reduce_mean":
            mag = mag / n
        half_ulp = np.abs(exact) * 2.0 ** -10 + 2.0 ** -24
        bound = half_ulp + 4 * max(1.0, np.log2(n)) * np.finfo(np.float32).eps * np.maximum(mag, np.abs(exact))
        assert (np.abs(got - exact) <= bound).all(), name
    assert np.array_equal(F.count(Xh, np.float16(0.5), axes).numpy(), F.count(Xo, np.float16(0.5), axes).numpy())


def test_argmax_argmin_half_and_int16(hip_backend, oracle_backend):
    for x in (np.round(halfs(126, (5, 33, 70), 3)), shorts(127, (5, 33, 70), -50, 50)):
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for axis in (0, 1, 2):
            assert np.array_equal(F.argmax(Xh, axis).numpy(), F.argmax(Xo, axis).numpy())
            assert np.array_equal(F.argmin(Xh, axis, False).numpy(), F.argmin(Xo, axis, False).numpy())
    long_rows = np.round(halfs(128, (2, 100000), 5))
    Xh, Xo = both(hip_backend, oracle_backend, long_rows)
    assert np.array_equal(F.argmax(Xh, 1).numpy(), F.argmax(Xo, 1).numpy())


@pytest.mark.parametrize("shape,axes", [((8, 21, 64, 64), (1,)), ((4, 100, 30, 30), (1,)), ((4096, 128), (0,)), ((5000, 67), (0,)), ((64, 3, 25, 25), (1,)),
                                        ((16, 50, 6, 20), (0, 2)), ((3, 70000, 6), (1,)), ((2, 9, 5000), (1,))])
def test_two_byte_columns_reduced_in_pairs(hip_backend, oracle_backend, shape, axes):
    """Reductions and arg-reductions over axes that are not the innermost: a lane takes two
    neighbouring two-byte columns in one 4-byte access where every pair starts on a 4-byte
    boundary (an even innermost extent, even strides, an aligned base) and one column otherwise
    (odd extents, views that start at an odd element).  Extrema, counts and positions are exact;
    sums are held to the half-ulp + fp32 bound."""
    n = int(np.prod([shape[a] for a in axes]))
    last = len(shape) - 1
    w = shape[last]
    xh = np.round(halfs(130, shape, 3) * 4) / 4                     # quarter steps: ties among the extrema
    xs = shorts(131, shape, -40, 40)
    for x in (xh, xs):
        Xh, Xo = both(hip_backend, oracle_backend, x)
        views = [(Xh, Xo, x)]
        for lo, hi in ((2, w), (1, w - 1), (0, w - 1)):
            if hi - lo >= 1:
                views.append((Xh.slice([lo], [hi], [last]), Xo.slice([lo], [hi], [last]), x[..., lo:hi]))
        views.append((Xh.slice([0], [w], [last], [2]), Xo.slice([0], [w], [last], [2]), x[..., ::2]))
        for Vh, Vo, v in views:
            if len(axes) == 1:
                assert np.array_equal(F.argmax(Vh, axes[0]).numpy(), F.argmax(Vo, axes[0]).numpy())
                assert np.array_equal(F.argmin(Vh, axes[0], False).numpy(), F.argmin(Vo, axes[0], False).numpy())
                assert np.array_equal(F.argmax(Vh, axes[0], True, np.int64).numpy(), F.argmax(Vo, axes[0], True, np.int64).numpy())
            if x.dtype == np.float16:
                assert np.array_equal(F.reduce("reduce_max", Vh, axes).numpy(), v.max(axis=axes))
                assert np.array_equal(F.reduce("reduce_min", Vh, axes, True).numpy(), v.min(axis=axes, keepdims=True))
                assert np.array_equal(F.count(Vh, np.float16(0.25), axes).numpy(), (v == np.float16(0.25)).sum(axis=axes))
                got = F.reduce("reduce_sum", Vh, axes).numpy().astype(np.float64)
                exact, mag = v.astype(np.float64).sum(axis=axes), np.abs(v.astype(np.float64)).sum(axis=axes)
                bound = np.abs(exact) * 2.0 ** -10 + 2.0 ** -24 + 4 * max(1.0, np.log2(n)) * np.finfo(np.float32).eps * mag
                assert (np.abs(got - exact) <= bound).all()


@pytest.mark.parametrize("n", [5, 300, 5000, 70000])
def test_half_scans(hip_backend, oracle_backend, n):
    x = halfs(129 + n, (3, n), 0.5)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for exclusive in (False, True):
        for reverse in (False, True):
            got = F.cumsum(Xh, 1, exclusive, reverse).numpy().astype(np.float64)
            xs = Xo.shape.flip([1]) if reverse else Xo.shape
            exact, mag = O.scan_f64("cumsum", dtype_code(np.float16), 3, n, exclusive, xs, Xo.storage)
            if reverse:
                exact, mag = exact[:, ::-1], mag[:, ::-1]
            bound = np.abs(exact) * 2.0 ** -10 + 2.0 ** -24 + 4 * max(1.0, np.log2(n)) * np.finfo(np.float32).eps * mag
            assert (np.abs(got - exact) <= bound).all(), (exclusive, reverse)
    assert np.array_equal(F.cummax(Xh, 1).numpy(), np.maximum.accumulate(x, axis=1))
    assert np.array_equal(F.cummin(Xh, 0).numpy(), np.minimum.accumulate(x, axis=0))


def test_nonzero_half_and_bool(hip_backend, oracle_backend):
    h = (halfs(130, (7, 33, 50)) * (randint(131, 7 * 33 * 50, 0, 2).reshape(7, 33, 50))).astype(np.float16)
    b = randint(132, 9 * 1000, 0, 3).reshape(9, 1000) == 0
    for x in (h, b):
        Xh = Tensor.from_numpy(hip_backend, x)
        assert np.array_equal(F.nonzero(Xh).numpy(), np.argwhere(x != 0))
        assert np.array_equal(F.nonzero(Xh.transpose(), True).numpy(), np.array(np.nonzero(x.transpose())))


@pytest.mark.parametrize("n,k", [(5, 5), (100, 1), (1000, 5), (4096, 50), (5000, 256), (32000, 50), (65536, 1000), (70000, 7)])
def test_top_k_bit_exact(hip_backend, oracle_backend, n, k):
    # rows up to 65536 elements are selected from registers; longer ones take the argsort path
    for x in (halfs(133 + n, (3, n), 10), np.round(halfs(134 + n, (3, n), 2)), shorts(135 + n, (3, n)), shorts(136 + n, (3, n), -3, 3)):
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for largest in (True, False):
            Yh, Ih = F.top_k(Xh, k, -1, largest)
            Yo, Io = F.top_k(Xo, k, -1, largest)
            assert np.array_equal(Ih.numpy(), Io.numpy()), (x.dtype, largest)
            assert np.array_equal(Yh.numpy().view(np.uint16), Yo.numpy().view(np.uint16))


def test_top_k_other_axis_int16(hip_backend, oracle_backend):
    x = shorts(137, (300, 7, 9), -20, 20)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for axis in (0, 1):
        Yh, Ih = F.top_k(Xh, 3, axis)
        Yo, Io = F.top_k(Xo, 3, axis)
        assert np.array_equal(Ih.numpy(), Io.numpy()) and np.array_equal(Yh.numpy(), Yo.numpy())


@pytest.mark.parametrize("n", [1, 7, 512, 1000, 2048, 5000, 16384, 32000, 40000])
def test_softmax_family_half(hip_backend, oracle_backend, n):
    # half rows are widened to float, the float result rounded once: one half ulp of the exact
    # value plus the fp32 error of the row sum
    x = halfs(138 + n, (5, n), 3)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    soft = e / e.sum(axis=1, keepdims=True)
    logsoft = (x64 - x64.max(axis=1, keepdims=True)) - np.log(e.sum(axis=1, keepdims=True))
    slack = 8 * max(1.0, np.log2(n)) * np.finfo(np.float32).eps
    got = F.softmax(Xh).numpy().astype(np.float64)
    assert (np.abs(got - soft) <= soft * (2.0 ** -10 + slack) + 2.0 ** -24).all()
    got = F.logsoftmax(Xh).numpy().astype(np.float64)
    assert (np.abs(got - logsoft) <= np.abs(logsoft) * 2.0 ** -10 + slack * (1 + np.abs(logsoft)) + 2.0 ** -24).all()
    assert np.array_equal(F.hardmax(Xh).numpy(), F.hardmax(Xo).numpy())
    # and the oracle's widened fp32 path rounds to the same or a neighbouring half
    ref = F.softmax(Xo).numpy().astype(np.float64)
    assert (np.abs(ref - soft) <= soft * (2.0 ** -10 + slack * 8) + 2.0 ** -24).all()
