"""dlfx_logits_head: sum, max, argmax, log-sum-exp and the k best of every row in one launch.

Checked against the CPU oracle's results for the five separate operations on the same input
(max, argmax and the k best bit for bit; the two fp32 sums to the bound of the separate
reductions, |got - o64| <= 4 ulp(fp32) * log2(n) * scale) and against what the library's own
separate calls write.
"""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor, prepare_reduce
from helpers import normal, ulp_bound
from oracle import oracle as O
from oracle.oracle import OracleBackend

pytestmark = pytest.mark.gpu


def head(hip, x, k, row_stride=None, parts=("sum", "max", "argmax", "lse", "values", "indices")):
    m, n = x.shape
    stride = n if row_stride is None else row_stride
    padded = np.full((m, stride), np.float32(-7.0), dtype=np.float32)
    padded[:, :n] = x
    X = Tensor.from_numpy(hip, padded)
    out = {"sum": Tensor.empty(hip, [m], np.float32), "max": Tensor.empty(hip, [m], np.float32),
           "argmax": Tensor.empty(hip, [m], np.int32), "lse": Tensor.empty(hip, [m], np.float32),
           "values": Tensor.empty(hip, [m, max(k, 1)], np.float32), "indices": Tensor.empty(hip, [m, max(k, 1)], np.int32)}
    arg = {name: (out[name].storage if name in parts else None) for name in out}
    hip.logits_head(F.dtype_code(np.float32), m, n, X.storage, 0, stride, arg["sum"], arg["max"], arg["argmax"], arg["lse"], k,
                    arg["values"], arg["indices"])
    return {name: out[name].numpy() for name in parts}


def check(hip, x, k, row_stride=None):
    m, n = x.shape
    got = head(hip, x, k, row_stride)
    spec = OracleBackend(topk_mode=1)
    Xo = Tensor.from_numpy(spec, x)
    Xh = Tensor.from_numpy(hip, x)
    # order-based results: bit for bit the oracle's, and the separate calls'
    # (rows holding a NaN: the reference's comparisons leave their order open, so only the
    # library's own separate calls, which order NaNs by bit pattern, are the measure there)
    plain = ~np.isnan(x).any(axis=1)
    assert np.array_equal(got["max"][plain], F.reduce("reduce_max", Xo, [1]).numpy().reshape(-1)[plain])
    assert np.array_equal(got["max"].view(np.uint32), F.reduce("reduce_max", Xh, [1]).numpy().reshape(-1).view(np.uint32))
    assert np.array_equal(got["argmax"], F.argmax(Xo, 1).numpy().reshape(-1))
    assert np.array_equal(got["argmax"], F.argmax(Xh, 1).numpy().reshape(-1))
    if k:
        Ys, Is = F.top_k(Xo, k, 1, True)
        assert np.array_equal(got["values"].view(np.uint32)[plain], Ys.numpy().view(np.uint32)[plain])
        assert np.array_equal(got["indices"][plain], Is.numpy()[plain])
        Yh, Ih = F.top_k(Xh, k, 1, True)
        assert np.array_equal(got["values"].view(np.uint32), Yh.numpy().view(np.uint32))
        assert np.array_equal(got["indices"], Ih.numpy())
    # the sums: the bound of the separate fp32 reductions against the fp64 evaluation
    view, _, mm, nn = prepare_reduce(Xo.shape, [1], False)
    code = F.dtype_code(np.float32)
    finite = np.isfinite(x).all(axis=1)
    for name, mag_name, key in (("reduce_sum", "reduce_asum", "sum"), ("reduce_log_sum_exp", None, "lse")):
        want = O.reduce_f64(name, code, mm, nn, view, Xo.storage)
        scale = np.maximum(np.abs(want), O.reduce_f64(mag_name, code, mm, nn, view, Xo.storage) if mag_name else 1.0)
        separate = F.reduce(name, Xh, [1]).numpy().reshape(-1)
        sound = finite & np.isfinite(want)              # (an overflowing exp sum is +inf on every path)
        assert np.array_equal(got[key][~sound], separate[~sound], equal_nan=True), name
        assert np.array_equal(got[key][finite & ~sound].astype(np.float64), want[finite & ~sound]), name
        err = np.abs(got[key].astype(np.float64)[sound] - want[sound])
        assert (err <= ulp_bound(n, scale)[sound]).all(), name
        assert (np.abs(got[key].astype(np.float64)[sound] - separate[sound]) <= 2 * ulp_bound(n, scale)[sound]).all(), name


@pytest.mark.parametrize("n", [1, 2, 5, 63, 64, 65, 255, 256, 257, 511, 512, 513, 1000, 1024, 1025, 2047, 2048])
def test_row_lengths(hip_backend, n):
    x = normal(300 + n, 37 * n).astype(np.float32).reshape(37, n)
    for k in sorted({0, 1, min(n, 5), min(n, 8)}):
        check(hip_backend, x, k)


def test_logits_shape_with_ties_and_row_stride(hip_backend):
    x = (np.round(normal(301, 256 * 1000) * 8) / 8).astype(np.float32).reshape(256, 1000)      # many equal values
    check(hip_backend, x, 5)
    check(hip_backend, x, 8, row_stride=1003)
    check(hip_backend, x[:3], 1, row_stride=4096)


def test_zeros_infinities_and_nans(hip_backend):
    x = normal(302, 12 * 300).astype(np.float32).reshape(12, 300)
    x[0, :] = 0.0
    x[0, 5] = -0.0                      # one value with +0.0: index order decides, the sign is kept
    x[1, 7] = np.inf
    x[1, 200] = np.inf
    x[2, :] = -np.inf
    x[3, 11] = np.nan                   # a NaN elsewhere never wins argmax, and sorts above +inf among the best
    x[4, 0] = np.nan                    # a NaN in position 0 is never displaced
    x[5, :] = np.float32(-3.5)
    x[6, 299] = np.float32(1e30)
    check(hip_backend, x, 5)


def test_outputs_are_optional_and_limits_are_refused(hip_backend):
    x = normal(303, 9 * 100).astype(np.float32).reshape(9, 100)
    full = head(hip_backend, x, 3)
    only = head(hip_backend, x, 3, parts=("argmax", "indices"))
    assert np.array_equal(only["argmax"], full["argmax"]) and np.array_equal(only["indices"], full["indices"])
    only = head(hip_backend, x, 0, parts=("sum", "lse"))
    assert np.array_equal(only["sum"], full["sum"]) and np.array_equal(only["lse"], full["lse"])
    with pytest.raises(RuntimeError):
        head(hip_backend, normal(304, 2 * 2049).astype(np.float32).reshape(2, 2049), 1)      # row too long for a wavefront
    with pytest.raises(RuntimeError):
        head(hip_backend, x, 9)                                                             # more than the fused call orders
