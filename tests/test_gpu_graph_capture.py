"""The boundary calls under HIP graph capture.

Every entry point only enqueues kernels on the stream it is given (no allocation, no
synchronisation, no memset nodes: state words are cleared by small kernels), so a caller may
record a sequence of calls into a graph and replay it.  Here a "logits head" sequence on
[256, 1000] plus a chained scan, a sort and a top_k over long rows is captured once and replayed
with new input contents; every replay is checked against the same calls issued eagerly, with
eager work and synchronisations between the replays."""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import normal, randint

pytestmark = pytest.mark.gpu


def sequence(X, L, Z):
    return [F.reduce("reduce_sum", X, (1,)), F.reduce("reduce_max", X, (1,)),
            F.reduce("reduce_log_sum_exp", X, (1,)), F.argmax(X, 1), *F.top_k(X, 5, 1),
            F.cumsum(L, 1), F.sort(L, 1), *F.argsort(L, 1, True, with_values=True),
            *F.top_k(Z, 50, 1), F.softmax(X, 1), F.count(Z, np.float32(0.0), (1,))]


def test_capture_and_replay_matches_eager(hip_backend):
    import torch
    x0 = normal(170, 256 * 1000).astype(np.float32).reshape(256, 1000)
    l0 = randint(171, 3 * 200000, 0, 100).astype(np.int32).reshape(3, 200000)
    z0 = np.round(normal(172, 8 * 40000).reshape(8, 40000) * 4).astype(np.float32)
    X, L, Z = (Tensor.from_numpy(hip_backend, a) for a in (x0, l0, z0))
    sequence(X, L, Z)                                   # warm-up: scratch is sized before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = sequence(X, L, Z)
    for r in range(3):
        # new contents in the captured input buffers, through ordinary eager work
        xr = np.roll(x0, r + 1, axis=1) * (r + 1)
        lr = np.roll(l0, 7 * r + 1, axis=1)
        zr = np.roll(z0, 3 * r + 2, axis=1) + r
        for T, a in ((X, xr), (L, lr), (Z, zr)):
            T.storage.copy_(torch.from_numpy(np.ascontiguousarray(a).reshape(-1)))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.numpy().copy() for o in outs]
        want = [o.numpy() for o in sequence(X, L, Z)]   # the same calls, eagerly, on the same inputs
        for i, (g, w) in enumerate(zip(got, want)):
            assert np.array_equal(g, w), (r, i)
        assert np.array_equal(got[6], np.cumsum(lr, axis=1, dtype=np.int32))
        assert np.array_equal(got[7], np.sort(lr, axis=1))
        assert np.array_equal(got[13], (zr == 0).sum(axis=1))


def test_reduce_static_records_and_replays(hip_backend):
    # dlfx_reduce_static is meant for callers under capture: once its first call on the device
    # has been made (outside any capture), recorded calls replay like any other launch and
    # allocate nothing (the caching allocator's count of allocations does not move across the
    # recording; a first recording that holds one fill kernel takes what torch itself sets up
    # once per process).
    import torch
    from dlf_amd.frontend import prepare_reduce
    x0 = normal(173, 3 * (1 << 20)).astype(np.float32).reshape(3, 1 << 20)
    X = Tensor.from_numpy(hip_backend, x0)
    view, out_dims, m, n = prepare_reduce(X.shape, [1], False)
    code = F.dtype_code(X.dtype)
    Y = Tensor.empty(hip_backend, out_dims, X.dtype)
    Ye = Tensor.empty(hip_backend, out_dims, X.dtype)
    hip_backend.reduce_static("reduce_sum", code, m, n, view, X.storage, Y.shape, Y.storage)     # the first call: eager
    torch.cuda.synchronize()
    def allocations():
        return torch.cuda.memory_stats(hip_backend.device)["allocation.all.allocated"]
    first = torch.cuda.CUDAGraph()
    with torch.cuda.graph(first):
        Ye.storage.zero_()
    before = allocations()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hip_backend.reduce_static("reduce_sum", code, m, n, view, X.storage, Y.shape, Y.storage)
        hip_backend.reduce_static("reduce_max", code, m, n, view, X.storage, Ye.shape, Ye.storage)
    assert allocations() == before
    for r in range(3):
        xr = np.roll(x0, 5 * r + 1, axis=1) * (r + 2)
        X.storage.copy_(torch.from_numpy(np.ascontiguousarray(xr).reshape(-1)))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_sum, got_max = Y.numpy().copy(), Ye.numpy().copy()
        want = F.reduce("reduce_sum", X, (1,)).numpy()                  # dlfx_reduce, eagerly, same input
        assert np.array_equal(got_sum, want), r
        assert np.array_equal(got_max, xr.max(axis=1)), r
