"""reduce / arg_reduce: HIP path vs the CPU oracle on the same seeded inputs.

Integer results and indices must be bit-exact.  fp32 results are compared with
the fp64 evaluation of the oracle.  Sums (reduce_sum / mean / asum / sum_square)
are held to the strict relative bound |got - o64| <= 4 ulp(fp32) * log2(n) * |o64|
(plus n * eps(fp64) * sum |f(x_i)|, what accumulating in fp64 itself may lose
when the terms cancel); the other reducers to 4 ulp(fp32) * log2(n) * scale with
scale = max(|o64|, sum |f(x_i)|) or max(|o64|, 1).
"""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor, prepare_reduce
from helpers import normal, randint, uniform01, ulp_bound
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def both(hip, orc, x):
    return Tensor.from_numpy(hip, x), Tensor.from_numpy(orc, x)


STRICT = ("reduce_sum", "reduce_mean", "reduce_asum", "reduce_sum_square")


def check_float_reduce(name, Xh, Xo, axes, keepdims=False):
    got = F.reduce(name, Xh, axes, keepdims).numpy().reshape(-1).astype(np.float64)
    view, _, m, n = prepare_reduce(Xo.shape, list(axes), keepdims)
    code = F.dtype_code(Xo.dtype)
    want = O.reduce_f64(name, code, m, n, view, Xo.storage)
    mag_name = {"reduce_sum": "reduce_asum", "reduce_mean": "reduce_asum", "reduce_asum": "reduce_asum",
                "reduce_sum_square": "reduce_sum_square", "reduce_sum_exp": "reduce_sum_exp"}.get(name)
    if name in ("reduce_max", "reduce_min", "reduce_amax", "reduce_amin"):
        assert np.array_equal(got, want), name
        return
    if mag_name:
        mag = O.reduce_f64(mag_name, code, m, n, view, Xo.storage)
        if name == "reduce_mean":
            mag = mag / n
        scale = np.maximum(np.abs(want), mag)
    else:
        scale = np.maximum(np.abs(want), 1.0)      # log / sqrt finals: well conditioned
    err = np.abs(got - want)
    if name in STRICT and Xo.dtype == np.float32:
        # fp64 accumulation and one rounding to fp32: relative to the result itself
        bound = ulp_bound(n, np.abs(want)) + n * np.finfo(np.float64).eps * mag
    else:
        bound = ulp_bound(n, scale)
    bad = err > bound
    assert not bad.any(), "%s: %d outputs off, worst %g (bound %g)" % (
        name, bad.sum(), (err / np.maximum(bound, 1e-300)).max(), 1.0)
    # the reference-association oracle (fp32 accumulation) must agree to the looser bound
    ref = F.reduce(name, Xo, axes, keepdims).numpy().reshape(-1).astype(np.float64)
    assert (np.abs(ref - want) <= ulp_bound(n, scale) * 8).all()


SHAPES = [
    ((256, 1000), [1]),            # logits head
    ((7, 33, 129), [2]), ((7, 33, 129), [1]), ((7, 33, 129), [0]), ((7, 33, 129), [0, 2]),
    ((7, 33, 129), []), ((3, 70000), [1]), ((1, 300001), [1]), ((5000, 3), [1]), ((5000, 3), [0]),
    ((4, 16, 14, 14), [2, 3]), ((4, 64, 14, 14), [1]), ((2, 3, 5, 7, 4), [1, 3]), ((1,), []),
    ((65, 17), [0]), ((2, 40000, 9), [1]),
]


@pytest.mark.parametrize("shape,axes", SHAPES)
@pytest.mark.parametrize("keep", [False, True])
def test_int_reductions_bit_exact(hip_backend, oracle_backend, shape, axes, keep):
    for dtype, lo, hi in ((np.int32, -100, 100), (np.int64, -10**12, 10**12)):
        x = randint(31, int(np.prod(shape)), lo, hi).astype(dtype).reshape(shape)
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for name in ("reduce_sum", "reduce_max", "reduce_min", "reduce_mean", "reduce_asum", "reduce_amax"):
            g = F.reduce(name, Xh, axes, keep).numpy()
            w = F.reduce(name, Xo, axes, keep).numpy()
            assert g.shape == w.shape and np.array_equal(g, w), (name, dtype)


@pytest.mark.parametrize("shape,axes", SHAPES)
def test_float_reductions_within_tolerance(hip_backend, oracle_backend, shape, axes):
    x = normal(32, int(np.prod(shape))).astype(np.float32).reshape(shape)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for name in ("reduce_sum", "reduce_mean", "reduce_max", "reduce_min", "reduce_log_sum_exp",
                 "reduce_sum_exp", "reduce_asum", "reduce_sum_square", "reduce_nrm2", "reduce_amax", "reduce_amin"):
        check_float_reduce(name, Xh, Xo, axes)


def test_float64_reductions(hip_backend, oracle_backend):
    x = normal(33, 37 * 4099).reshape(37, 4099)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for axes in ([1], [0]):
        for name in ("reduce_sum", "reduce_max", "reduce_mean", "reduce_log_sum_exp"):
            g = F.reduce(name, Xh, axes).numpy()
            w = F.reduce(name, Xo, axes).numpy()
            np.testing.assert_allclose(g, w, rtol=1e-12, atol=1e-12)


def test_int32_sum_wraps_and_mean_truncates(hip_backend, oracle_backend):
    x = np.full((3, 50000), 2**30 + 7, dtype=np.int32)
    x[1] *= -1
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for name in ("reduce_sum", "reduce_mean"):
        assert np.array_equal(F.reduce(name, Xh, [1]).numpy(), F.reduce(name, Xo, [1]).numpy())
    y = np.array([[-7, 2, 2], [7, -2, -2]], dtype=np.int32)
    assert F.reduce_mean(Tensor.from_numpy(hip_backend, y), [1]).numpy().tolist() == [-1, 1]


def test_log_sum_exp_overflow_is_inf(hip_backend):
    x = np.array([[1.0, 2.0, 3.0], [100.0, 0.0, 0.0]], dtype=np.float32)
    got = F.reduce_log_sum_exp(Tensor.from_numpy(hip_backend, x), [1]).numpy()
    assert np.isclose(got[0], np.log(np.exp(1.0) + np.exp(2.0) + np.exp(3.0)), rtol=1e-6)
    assert np.isposinf(got[1])


def test_unaligned_and_sliced_rows(hip_backend, oracle_backend):
    # rows that start off a 16-byte boundary and views with offsets / steps
    x = randint(34, 13 * 1003, -9, 9).astype(np.int32).reshape(13, 1003)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for args in (([1, 3], [12, 1000]), ([0, 1000], [13, 1], None, [2, -3]), ([2, 5], [3, 6])):
        vh, vo = Xh.slice(*args), Xo.slice(*args)
        for axes in ([0], [1], []):
            assert np.array_equal(F.reduce_sum(vh, axes).numpy(), F.reduce_sum(vo, axes).numpy())
            assert np.array_equal(F.argmax(vh, -1).numpy(), F.argmax(vo, -1).numpy())


def test_transposed_and_broadcast_like_views(hip_backend, oracle_backend):
    x = randint(35, 6 * 50 * 70, -5, 5).astype(np.int64).reshape(6, 50, 70)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for perm in ([2, 0, 1], [1, 2, 0], [2, 1, 0]):
        for axes in ([0], [1], [2], [0, 1], [1, 2]):
            g = F.reduce_sum(Xh.transpose(perm), axes).numpy()
            w = F.reduce_sum(Xo.transpose(perm), axes).numpy()
            assert np.array_equal(g, w), (perm, axes)


ARG_SHAPES = [((256, 1000), 1), ((6, 7, 50), 0), ((6, 7, 50), 1), ((6, 7, 50), 2), ((3, 100000), 1),
              ((1, 1), 0), ((4, 64, 14, 14), 1), ((70000, 2), 1), ((2, 30000, 5), 1), ((9, 20000), 1)]


@pytest.mark.parametrize("shape,axis", ARG_SHAPES)
@pytest.mark.parametrize("keep", [True, False])
def test_argmax_argmin_bit_exact_with_ties(hip_backend, oracle_backend, shape, axis, keep):
    for dtype in (np.int32, np.float32, np.int64, np.float64):
        x = randint(36, int(np.prod(shape)), 0, 6).astype(dtype).reshape(shape)      # heavy ties
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for fn in (F.argmax, F.argmin):
            g, w = fn(Xh, axis, keep).numpy(), fn(Xo, axis, keep).numpy()
            assert g.dtype == np.int32 and g.shape == w.shape and np.array_equal(g, w)
    g64 = F.argmax(Xh, axis, keep, index_dtype=np.int64).numpy()
    assert g64.dtype == np.int64 and np.array_equal(g64, F.argmax(Xo, axis, keep).numpy())


def test_argmax_all_equal_rows_and_nan_rule(hip_backend, oracle_backend):
    x = np.zeros((5, 3000), dtype=np.float32)
    assert not F.argmax(Tensor.from_numpy(hip_backend, x), 1, False).numpy().any()
    x = np.full((4, 100), -np.inf, dtype=np.float32)
    assert not F.argmax(Tensor.from_numpy(hip_backend, x), 1, False).numpy().any()
    y = normal(37, 4 * 5000).astype(np.float32).reshape(4, 5000)
    y[0, 17] = np.nan          # a NaN that is not first never wins
    y[1, 0] = np.nan           # a NaN in position 0 is never displaced
    y[2, 4999] = np.nan
    Xh, Xo = both(hip_backend, oracle_backend, y)
    for fn in (F.argmax, F.argmin):
        assert np.array_equal(fn(Xh, 1).numpy(), fn(Xo, 1).numpy())


def test_argmax_transposed_view(hip_backend):
    x = randint(38, 4 * 5 * 6, 0, 100).astype(np.int32).reshape(4, 5, 6)
    X = Tensor.from_numpy(hip_backend, x)
    assert np.array_equal(F.argmax(X.transpose(), 0).numpy(), F.argmax(X, -1).numpy().transpose())


def test_error_statuses(hip_backend):
    from dlf_amd.hip_backend import DlfxError
    X = Tensor.from_numpy(hip_backend, np.zeros((4, 4), dtype=np.float32))
    with pytest.raises(DlfxError) as e:
        F.reduce("reduce_bogus", X, [1])
    assert e.value.status == -3
    Xi = Tensor.from_numpy(hip_backend, np.zeros((4, 4), dtype=np.int32))
    with pytest.raises(DlfxError) as e:
        F.reduce("reduce_log_sum_exp", Xi, [1])
    assert e.value.status == -2


def test_int64_mean_of_many_short_rows_truncates_exactly(hip_backend, oracle_backend):
    """The mean of int64 rows divides the (wrapping) sum by the row length, truncating toward
    zero.  Sums of every magnitude and sign, including the extremes, over row lengths from 1 to
    thousands."""
    from helpers import full_range_i64
    for n in (1, 2, 3, 7, 64, 1000, 4097):
        rows = 3000
        x = full_range_i64(300 + n, rows * n).reshape(rows, n)
        x[0] = 0
        x[0, 0] = np.iinfo(np.int64).min                                  # sum = INT64_MIN
        x[1] = 0
        x[1, 0] = np.iinfo(np.int64).max
        x[2] = -1
        x[3] = 1
        x[4] = 0
        x[4, 0] = -(n - 1) if n > 1 else -1                               # a quotient just above -1
        small = randint(301 + n, (rows - 5) * n // 2, -50, 50).astype(np.int64)
        x[5:5 + (rows - 5) // 2] = small[: ((rows - 5) // 2) * n].reshape(-1, n)      # quotients near zero, both signs
        got = F.reduce_mean(Tensor.from_numpy(hip_backend, x), [1]).numpy()
        want = F.reduce_mean(Tensor.from_numpy(oracle_backend, x), [1]).numpy()
        assert np.array_equal(got, want), n
        sums = [int(v) for v in x[5:50].astype(object).sum(axis=1)]
        wrapped = [((s + 2**63) % 2**64) - 2**63 for s in sums]
        exact = [abs(s) // n * (1 if s >= 0 else -1) for s in wrapped]
        assert got[5:50].tolist() == exact


@pytest.mark.parametrize("shape,axes", [((6, 40, 70, 65), [0, 2, 3]), ((5, 64, 9, 300, 20), [0, 2, 4]), ((3, 7, 4000, 17), [0, 2, 3]),
                                        ((2, 3, 40, 50, 20), [0, 2, 4]), ((20, 96, 56, 56), [0, 2, 3]), ((9, 3, 150, 151), [0, 2, 3]),
                                        ((3, 5, 20001), [0, 2]), ((2, 16, 8, 64, 64), [0, 2, 3, 4]), ((32, 7, 9, 56), [0, 3]),
                                        ((6, 50, 4, 128), [0, 3]), ((5, 33, 64, 16), [0, 2, 3])])
def test_long_rows_made_of_contiguous_runs(hip_backend, oracle_backend, shape, axes):
    # rows whose reduced dimensions end in a contiguous one (statistics per channel of an NCHW tensor): read
    # run by run; runs of 4550, 20, 68000, 20 and 3136 elements; then a few long runs a row, handed out in
    # pieces of 4096 elements (22650, 20001 and 32768 elements, the middle one off every boundary), and rows
    # of 1024 to 8192 elements made of runs (56, 128 and 1024 elements: whole cache lines or not)
    x = randint(190, int(np.prod(shape)), -100, 100).astype(np.int32).reshape(shape)
    Xh = Tensor.from_numpy(hip_backend, x)
    for name, fn in (("reduce_sum", np.sum), ("reduce_max", np.max), ("reduce_min", np.min)):
        got = F.reduce(name, Xh, axes).numpy()
        assert np.array_equal(got, fn(x.astype(np.int64), axis=tuple(axes)).astype(np.int32)), name
    y = (normal(191, int(np.prod(shape))) * 2).astype(np.float32).reshape(shape)
    Yh, Yo = both(hip_backend, oracle_backend, y)
    for name in ("reduce_sum", "reduce_mean", "reduce_max", "reduce_log_sum_exp", "reduce_sum_square", "reduce_nrm2"):
        check_float_reduce(name, Yh, Yo, axes)
    assert np.array_equal(F.count(Xh, np.int32(3), tuple(axes)).numpy(), (x == 3).sum(axis=tuple(axes)))


@pytest.mark.parametrize("shape,axis", [((8, 21, 64, 64), 1), ((64, 3, 50, 50), 1), ((5000, 2, 3), 1), ((3, 32, 5000), 1), ((2, 33, 5000), 1),
                                        ((17, 8000), 0), ((4, 5, 6, 700), 2),
                                        ((600, 50, 3, 17), 2), ((9000, 8, 20), 1), ((20000, 4, 16), 1), ((9000, 9, 20), 1), ((3000, 8, 47), 1), ((3000, 8, 48), 1)])
def test_short_axis_beside_many_columns_one_lane_per_column(hip_backend, oracle_backend, shape, axis):
    # a reduced axis of up to 32 elements that is not the innermost, beside thousands of columns: a lane
    # reduces a column on its own (33 elements: the kernel of four wavefronts per 64 columns); beside runs of
    # fewer than 48 columns an axis of up to 8 elements goes a lane a row through the strided-row kernel instead
    x = randint(192, int(np.prod(shape)), -9, 9).astype(np.int32).reshape(shape)       # ties: the first extremum counts
    Xh = Tensor.from_numpy(hip_backend, x)
    assert np.array_equal(F.reduce("reduce_sum", Xh, [axis]).numpy(), x.sum(axis=axis, dtype=np.int32))
    assert np.array_equal(F.reduce("reduce_max", Xh, [axis], True).numpy(), x.max(axis=axis, keepdims=True))
    assert np.array_equal(F.reduce("reduce_prod", Xh, [axis]).numpy(), np.prod(x, axis=axis, dtype=np.int32))
    assert np.array_equal(F.argmax(Xh, axis).numpy().reshape(-1), np.argmax(x, axis=axis).reshape(-1))
    assert np.array_equal(F.argmin(Xh, axis).numpy().reshape(-1), np.argmin(x, axis=axis).reshape(-1))
    assert np.array_equal(F.count(Xh, np.int32(0), (axis,)).numpy().reshape(-1), (x == 0).sum(axis=axis).reshape(-1))
    y = (normal(193, int(np.prod(shape))) * 2).astype(np.float32).reshape(shape)
    Yh, Yo = both(hip_backend, oracle_backend, y)
    for name in ("reduce_sum", "reduce_mean", "reduce_min", "reduce_log_sum_exp", "reduce_nrm2"):
        check_float_reduce(name, Yh, Yo, [axis])
    sl = Xh.slice([0], [shape[-1] - 1], [len(shape) - 1], [2])            # every other innermost element: the general kernels
    assert np.array_equal(F.reduce("reduce_sum", sl, [axis]).numpy(), x[..., 0:shape[-1] - 1:2].sum(axis=axis, dtype=np.int32))


@pytest.mark.parametrize("shape", [(40000, 56), (30000, 100), (100000, 7), (20000, 64), (70000, 16), (3000, 200), (9000, 31)])
def test_many_short_rows_whole_cache_lines_or_not(hip_backend, oracle_backend, shape):
    # rows of a few hundred bytes: a group of lanes a row; rows that are whole cache lines (from 512 bytes) are
    # loaded with the non-temporal hint, the others without - both for every element type here
    for dtype in (np.int32, np.int64, np.float16):
        x = randint(196, int(np.prod(shape)), -20, 20).astype(dtype).reshape(shape)
        Xh = Tensor.from_numpy(hip_backend, x)
        if dtype != np.float16:
            assert np.array_equal(F.reduce("reduce_sum", Xh, [1]).numpy(), x.sum(axis=1, dtype=dtype))
            assert np.array_equal(F.count(Xh, dtype(3), (1,)).numpy(), (x == 3).sum(axis=1))
        assert np.array_equal(F.reduce("reduce_max", Xh, [1]).numpy(), x.max(axis=1))
        assert np.array_equal(F.reduce("reduce_min", Xh, [1], True).numpy(), x.min(axis=1, keepdims=True))
        assert np.array_equal(F.argmax(Xh, 1, False).numpy(), np.argmax(x, axis=1))
        assert np.array_equal(F.argmin(Xh, 1, False).numpy(), np.argmin(x, axis=1))
        V = Xh.slice([1], [shape[1]], [1])                              # rows that start off every boundary
        assert np.array_equal(F.reduce("reduce_max", V, [1]).numpy(), x[:, 1:].max(axis=1))
    y = (normal(197, int(np.prod(shape))) * 2).astype(np.float32).reshape(shape)
    Yh, Yo = both(hip_backend, oracle_backend, y)
    for name in ("reduce_sum", "reduce_mean", "reduce_log_sum_exp", "reduce_nrm2"):
        check_float_reduce(name, Yh, Yo, [1])
