"""ONNX operator adapters over the front-ends: what dlf's interpreter does for the nodes that
land on the axis primitives (dlf/include/predict.h:1078-1201 Reduce*/ArgMax/ArgMin/CumSum,
:1486-1510 TopK, :2031-2044 NonZero, and the Softmax family), with the same attribute
defaults.  A node is given as its operator name, its input tensors and a dict of attributes;
tensor-valued inputs that the reference reads on the host (CumSum's axis, TopK's K) are
plain Python integers here.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

from . import frontend as F
from .frontend import Tensor

# ONNX reduction node -> reducer name (predict.h:1099-1137)
REDUCERS = {
    "ReduceMax": "reduce_max", "ReduceMin": "reduce_min", "ReduceSum": "reduce_sum",
    "ReduceSumSquare": "reduce_sum_square", "ReduceMean": "reduce_mean", "ReduceProd": "reduce_prod",
    "ReduceLogSum": "reduce_log_sum", "ReduceLogSumExp": "reduce_log_sum_exp",
    "ReduceL1": "reduce_asum", "ReduceL2": "reduce_nrm2",
}


def evaluate(op_type: str, inputs: Sequence, attrs: Dict = None) -> List[Tensor]:
    """Runs one node; returns its outputs in ONNX order."""
    a = dict(attrs or {})
    X = inputs[0]
    if op_type in REDUCERS:
        # axes default: all; keepdims default 1 (predict.h:1087-1089)
        return [F.reduce(REDUCERS[op_type], X, list(a.get("axes", [])), bool(a.get("keepdims", 1)))]
    if op_type in ("ArgMax", "ArgMin"):
        fn = F.argmax if op_type == "ArgMax" else F.argmin
        return [fn(X, int(a.get("axis", 0)), bool(a.get("keepdims", 1)))]
    if op_type == "CumSum":
        axis = int(inputs[1])                         # a rank-0 tensor read on the host (predict.h:1190-1193)
        return [F.cumsum(X, axis, bool(a.get("exclusive", 0)), bool(a.get("reverse", 0)))]
    if op_type == "TopK":
        k = int(inputs[1])
        values, indices = F.top_k(X, k, int(a.get("axis", -1)), bool(a.get("largest", 1)))
        return [values, indices]                      # always sorted, as the reference's device path
    if op_type == "NonZero":
        return [F.nonzero(X, True)]                   # [rank, n] (predict.h:2037)
    if op_type in ("Softmax", "LogSoftmax", "Hardmax"):
        fn = {"Softmax": F.softmax, "LogSoftmax": F.logsoftmax, "Hardmax": F.hardmax}[op_type]
        return [fn(X, int(a.get("axis", 1)))]
    raise KeyError("operator %r is not one of the axis primitives" % op_type)
