"""ONNX node adapters on the HIP path vs the same nodes on the oracle: attribute defaults and
output order (dlf/include/predict.h:1078-1201, 1486-1510, 2031-2044)."""
import numpy as np
import pytest

from dlf_amd import onnx_ops
from dlf_amd.frontend import Tensor
from helpers import normal, randint

pytestmark = pytest.mark.gpu


def run(be, op, x, extra=(), attrs=None):
    return [None if t is None else t.numpy() for t in onnx_ops.evaluate(op, [Tensor.from_numpy(be, x), *extra], attrs)]


def same(a, b, exact):
    return np.array_equal(a, b) if exact else np.allclose(a, b, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("op", sorted(onnx_ops.REDUCERS))
def test_reductions(hip_backend, oracle_backend, op):
    x = (np.abs(normal(110, 4 * 5 * 60)) + 0.5).astype(np.float32).reshape(4, 5, 60)
    for attrs in (None, {"axes": [1]}, {"axes": [0, 2], "keepdims": 0}, {"axes": [-1], "keepdims": 1}):
        g, w = run(hip_backend, op, x, attrs=attrs), run(oracle_backend, op, x, attrs=attrs)
        assert g[0].shape == w[0].shape and same(g[0], w[0], op in ("ReduceMax", "ReduceMin")), (op, attrs)
    assert run(hip_backend, op, x)[0].shape == (1, 1, 1)          # keepdims defaults to 1


def test_arg_cumsum_topk_nonzero_softmax(hip_backend, oracle_backend):
    x = randint(111, 6 * 7 * 50, -9, 10).astype(np.float32).reshape(6, 7, 50)
    for op in ("ArgMax", "ArgMin"):
        for attrs in (None, {"axis": 2}, {"axis": 1, "keepdims": 0}):
            assert np.array_equal(run(hip_backend, op, x, attrs=attrs)[0], run(oracle_backend, op, x, attrs=attrs)[0])
    assert run(hip_backend, "ArgMax", x)[0].shape == (1, 7, 50)    # axis 0, keepdims 1
    for attrs in (None, {"exclusive": 1}, {"reverse": 1}, {"exclusive": 1, "reverse": 1}):
        assert np.array_equal(run(hip_backend, "CumSum", x, (1,), attrs)[0], run(oracle_backend, "CumSum", x, (1,), attrs)[0])
    for attrs in (None, {"axis": 1, "largest": 0}):
        g, w = run(hip_backend, "TopK", x, (3,), attrs), run(oracle_backend, "TopK", x, (3,), attrs)
        assert np.array_equal(g[0], w[0]) and np.array_equal(g[1], w[1])
    g = run(hip_backend, "NonZero", x)[0]
    assert g.shape[0] == 3 and np.array_equal(g, np.array(np.nonzero(x)))
    for op in ("Softmax", "LogSoftmax", "Hardmax"):
        for attrs in (None, {"axis": 2}, {"axis": 0}):
            g, w = run(hip_backend, op, x, attrs=attrs)[0], run(oracle_backend, op, x, attrs=attrs)[0]
            assert same(g, w, op == "Hardmax")
    with pytest.raises(KeyError):
        onnx_ops.evaluate("Conv", [Tensor.from_numpy(hip_backend, x)])
