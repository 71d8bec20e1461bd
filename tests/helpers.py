"""Shared helpers of the parity tests."""
import json
import os

import numpy as np

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from dlf_amd.shape import Shape

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden_cases():
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        return json.load(f)["cases"]


def case_input(backend, case):
    dtype = np.dtype(case["dtype"])
    shape = case["x_shape"]
    if "x" in case:
        x = np.array(case["x"], dtype=dtype).reshape(shape)
    else:
        x = (np.arange(int(np.prod(shape))) + case["x_range"]).astype(dtype).reshape(shape)
    X = Tensor.from_numpy(backend, x)
    if "as_strided" in case:
        X = X.view(Shape(case["as_strided"]["extents"], case["as_strided"]["strides"]))
    return X


def run_golden_case(backend, case):
    """Runs every call of one fixture through the front-end on `backend`; returns failures."""
    op = case["op"]
    X = case_input(backend, case)
    fails = []
    for call in case["calls"]:
        if op.startswith("reduce_"):
            got = F.reduce(op, X, call["axes"], call["keepdims"])
            outs = [(got, call["y_shape"], call["y"])]
        elif op in ("argmax", "argmin"):
            got = F.arg_reduce(op, X, call["axis"], call["keepdims"])
            outs = [(got, call["y_shape"], call["y"])]
        elif op in ("cumsum", "cumprod"):
            got = F.scan(op, X, call["axis"], call["exclusive"], call["reverse"])
            outs = [(got, case["x_shape"], call["y"])]
        elif op == "sort":
            got = F.sort(X, call["axis"])
            outs = [(got, case["x_shape"], call["y"])]
        elif op == "top_k":
            y, i = F.top_k(X, call["k"], call["axis"], call["largest"])
            outs = [(y, call["y_shape"], call["y"]), (i, call["y_shape"], call["i"])]
        elif op in ("softmax", "logsoftmax", "hardmax"):
            got = getattr(F, op)(X, call["axis"])
            outs = [(got, call["y_shape"], call["y"])]
        elif op == "count":
            got = F.count(X, call["value"], call["axes"], call["keepdims"])
            outs = [(got, call["y_shape"], call["y"])]
        elif op == "nonzero":
            got = F.nonzero(X, call["row_major"])
            outs = [(got, call["y_shape"], call["y"])]
        else:
            raise AssertionError("unknown op " + op)
        backend.synchronize()
        for t, shape, want in outs:
            g = t.numpy()
            w = np.array(want, dtype=g.dtype).reshape(shape)
            if list(g.shape) != list(shape):
                fails.append((call, "shape %s != %s" % (g.shape, shape)))
            elif "rtol" in case:
                if not np.allclose(g, w, rtol=case["rtol"], atol=0):
                    fails.append((call, g.tolist()))
            elif not np.array_equal(g, w):
                fails.append((call, g.tolist()))
    return fails


# ---------------------------------------------------------------- seeded synthetic data
_M64 = (1 << 64) - 1


def splitmix64(seed: int, index: np.ndarray) -> np.ndarray:
    """Counter-based generator: one 64-bit word per (seed, linear index)."""
    with np.errstate(over="ignore"):
        z = (index.astype(np.uint64) + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15) \
            + np.uint64((seed * 0xD1B54A32D192ED03) & _M64)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform01(seed, count, offset=0):
    r = splitmix64(seed, np.arange(offset, offset + count, dtype=np.uint64))
    return (r >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def normal(seed, count):
    """Box-Muller in fp64 from two decorrelated uniforms per element."""
    idx = np.arange(count, dtype=np.uint64)
    u1 = ((splitmix64(seed, 2 * idx) >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / (1 << 53))
    u2 = (splitmix64(seed, 2 * idx + 1) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def randint(seed, count, lo, hi):
    r = splitmix64(seed, np.arange(count, dtype=np.uint64))
    return (r % np.uint64(hi - lo)).astype(np.int64) + lo


def full_range_i64(seed, count):
    return splitmix64(seed, np.arange(count, dtype=np.uint64)).view(np.int64)


def ulp_bound(n, scale, ulps=4.0):
    """4 ulp x log2(n) of `scale` in fp32."""
    return ulps * max(1.0, np.log2(max(2, n))) * np.finfo(np.float32).eps * scale
