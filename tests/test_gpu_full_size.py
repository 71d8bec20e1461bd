"""The benchmark configurations at their full sizes, checked through properties that do not
need the CPU oracle: agreement with an independent device implementation where the result is
unique (sorted values, integer prefix sums, maxima), and otherwise sortedness, permutation,
stability, idempotence, prefix consistency of top_k, linearity of integer scans and sums of
partial sums.  The parity gates bench.py applies before timing are run here as well."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from dlf_amd.shape import Shape

pytestmark = pytest.mark.gpu

EPS32 = float(np.finfo(np.float32).eps)


def wrap(be, t):
    import torch
    np_of = {torch.float32: np.float32, torch.int32: np.int32, torch.int64: np.int64}
    return Tensor(be, Shape(list(t.shape)), t.reshape(-1), np_of[t.dtype])


def dev(T):
    return T.storage[:T.size].view(*T.shape.extents)


@pytest.mark.parametrize("config", ["c1", "c2", "c3", "c4", "c5", "n1", "n2", "n3"])
def test_bench_parity_gates(hip_backend, config):
    import torch
    import bench
    ops = bench.make_ops(hip_backend, config)
    assert ops
    for op in ops:
        if op.verify:
            op.verify()
    torch.cuda.synchronize()


def test_cumsum_int32_is_linear_and_ends_in_the_row_sum(hip_backend):
    import torch
    g = torch.Generator(device="cuda").manual_seed(11)
    a = torch.randint(-2**31, 2**31 - 1, (64, 1 << 20), dtype=torch.int64, device="cuda", generator=g).to(torch.int32)
    b = torch.randint(-1000, 1000, (64, 1 << 20), dtype=torch.int64, device="cuda", generator=g).to(torch.int32)
    ca, cb, cab = (dev(F.cumsum(wrap(hip_backend, t), 1)) for t in (a, b, a + b))       # int32 arithmetic wraps
    assert torch.equal(cab, ca + cb)
    assert torch.equal(ca[:, -1], a.sum(dim=1, dtype=torch.int64).to(torch.int32))
    assert torch.equal(ca[:, 1:] - ca[:, :-1], a[:, 1:]) and torch.equal(ca[:, 0], a[:, 0])
    rev = dev(F.cumsum(wrap(hip_backend, a), 1, False, True))
    assert torch.equal(rev, torch.flip(dev(F.cumsum(wrap(hip_backend, torch.flip(a, [1]).contiguous()), 1)), [1]))
    ex = dev(F.cumsum(wrap(hip_backend, a), 1, True, False))
    assert torch.equal(ex[:, 1:], ca[:, :-1]) and not bool(ex[:, 0].any())


def test_reduce_sum_of_2_30_elements_equals_the_sum_of_row_sums(hip_backend):
    import torch
    g = torch.Generator(device="cuda").manual_seed(12)
    x = torch.randn(1 << 30, device="cuda", generator=g)
    X = wrap(hip_backend, x)
    # fp32 sums are accumulated in fp64 and rounded once: the result is the rounded exact sum up
    # to the fp64 accumulation error, far inside the 4 * log2(n) ulp the interface promises
    total = float(F.reduce("reduce_sum", X, ()).storage[0])
    rows = dev(F.reduce("reduce_sum", wrap(hip_backend, x.view(1024, 1 << 20)), (1,)))
    exact = float(x.double().sum())
    mag = float(x.double().abs().sum())
    assert abs(total - exact) <= EPS32 * abs(exact) + 1e-12 * mag
    exact_rows = x.view(1024, 1 << 20).double().sum(dim=1)
    mag_rows = x.view(1024, 1 << 20).double().abs().sum(dim=1)
    assert bool(((rows.double() - exact_rows).abs() <= EPS32 * exact_rows.abs() + 1e-12 * mag_rows).all())
    assert abs(float(rows.double().sum()) - total) <= 1024 * EPS32 * float(exact_rows.abs().max()) + EPS32 * abs(total)
    mx = float(F.reduce("reduce_max", X, ()).storage[0])
    assert mx == float(x.max())


@pytest.mark.parametrize("dtype,rows,n", [("float32", 1024, 65536), ("int64", 256, 1 << 20)])
def test_sort_and_argsort_full_size(hip_backend, dtype, rows, n):
    import torch
    g = torch.Generator(device="cuda").manual_seed(13)
    if dtype == "float32":
        x = (torch.randn(rows, n, device="cuda", generator=g) * 64).round() / 8          # many ties
    else:
        x = torch.randint(-2**62, 2**62, (rows, n), dtype=torch.int64, device="cuda", generator=g)
        x[:, 0:n - 2:3] = x[:, 1:n - 1:3]                                                # ties
    X = wrap(hip_backend, x)
    for desc in (False, True):
        y = dev(F.sort(X, 1, desc))
        assert torch.equal(y, torch.sort(x, dim=1, descending=desc).values)
        assert torch.equal(dev(F.sort(wrap(hip_backend, y), 1, desc)), y)                # idempotent
        i = dev(F.argsort(X, 1, desc)).long()
        assert torch.equal(torch.gather(x, 1, i), y)
        # stable: where neighbours are equal the indices rise; and each row is a permutation
        same = y[:, 1:] == y[:, :-1]
        assert bool((i[:, 1:] > i[:, :-1])[same].all())
        assert torch.equal(torch.sort(i, dim=1).values, torch.arange(n, device="cuda").expand(rows, n))
        del y, i, same


def test_top_k_full_size_prefix_consistency(hip_backend):
    import torch
    g = torch.Generator(device="cuda").manual_seed(14)
    x = (torch.randn(4096, 32000, device="cuda", generator=g) * 256).round() / 256        # ties in every row
    X = wrap(hip_backend, x)
    order = torch.sort(x, dim=1, descending=True, stable=True)
    prev = None
    for k in (256, 50, 5, 1):
        Y, I = F.top_k(X, k, 1, True)
        y, i = dev(Y), dev(I).long()
        assert torch.equal(y, order.values[:, :k]) and torch.equal(i, order.indices[:, :k])
        if prev is not None:
            assert torch.equal(y, prev[0][:, :k]) and torch.equal(i, prev[1][:, :k])
        prev = (y, i)
    Y, I = F.top_k(X, 5, 1, False)
    up = torch.sort(x, dim=1, descending=False, stable=True)
    assert torch.equal(dev(Y), up.values[:, :5]) and torch.equal(dev(I).long(), up.indices[:, :5])


def test_nchw_reductions_full_size(hip_backend):
    import torch
    g = torch.Generator(device="cuda").manual_seed(15)
    x = torch.randn(32, 512, 56, 56, device="cuda", generator=g)
    x[:, 7] = x[:, 300]                                                                   # ties across channels
    X = wrap(hip_backend, x)
    assert torch.equal(dev(F.reduce("reduce_max", X, (1,))), x.amax(dim=1))
    am = dev(F.argmax(X, 1)).long().reshape(32, 56, 56)
    assert torch.equal(torch.gather(x, 1, am.unsqueeze(1)).squeeze(1), x.amax(dim=1))
    first = (x == x.amax(dim=1, keepdim=True)).to(torch.int32).argmax(dim=1)              # first maximum
    assert torch.equal(am, first)
    mean = dev(F.reduce("reduce_mean", X, (2, 3)))
    want = x.double().mean(dim=(2, 3))
    assert bool(((mean.double() - want).abs() <= 4 * 12 * EPS32 * x.double().abs().mean(dim=(2, 3))).all())
    cs = dev(F.cumsum(X, 1))
    want = torch.cumsum(x.double(), 1)
    mag = torch.cumsum(x.double().abs(), 1)
    assert bool(((cs.double() - want).abs() <= 4 * 9 * EPS32 * mag).all())


def test_tensors_of_more_than_2_32_elements(hip_backend):
    """Element offsets beyond 32 bits (HBM holds 2^36 fp32 elements): totals above 2^32 are
    served, single rows above 2^32 elements by reduce and scan; the routines whose results are
    32-bit positions or counts refuse such a row with the too-large status."""
    import torch
    from dlf_amd.hip_backend import DlfxError
    g = torch.Generator(device="cuda").manual_seed(16)
    N = 4_400_000_000
    x = torch.randint(-100, 100, (N,), dtype=torch.int32, device="cuda", generator=g)
    X = wrap(hip_backend, x)
    total = x.sum(dtype=torch.int64).to(torch.int32)
    assert int(F.reduce("reduce_sum", X, ()).storage[0]) == int(total)
    assert int(F.reduce("reduce_max", X, ()).storage[0]) == int(x.max())
    y = dev(F.cumsum(X, 0))
    for lo in (0, (1 << 31) - 5000, (1 << 32) - 5000, N - 6000):
        base = int(x[:lo].sum(dtype=torch.int64)) if lo else 0
        want = (torch.cumsum(x[lo:lo + 6000].long(), 0) + base).to(torch.int32)
        assert torch.equal(y[lo:lo + 6000], want), lo
    del y
    for call in (lambda: F.argmax(wrap(hip_backend, x.view(1, N)), 1), lambda: F.count(wrap(hip_backend, x.view(1, N)), np.int32(3), (1,)),
                 lambda: F.nonzero(X)):
        with pytest.raises(DlfxError, match="too large"):
            call()
    xr = x[:1025 * (1 << 22)].view(1025, 1 << 22)
    assert torch.equal(dev(F.cumsum(wrap(hip_backend, xr), 1))[-3:], torch.cumsum(xr[-3:], 1, dtype=torch.int32))
    assert torch.equal(dev(F.reduce("reduce_sum", wrap(hip_backend, xr), (1,))), xr.sum(dim=1, dtype=torch.int64).to(torch.int32))
    assert torch.equal(dev(F.reduce("reduce_sum", wrap(hip_backend, xr), (0,))), xr.sum(dim=0, dtype=torch.int64).to(torch.int32))
    am = dev(F.argmax(wrap(hip_backend, xr), 1)).long().reshape(-1)
    first = (xr == xr.amax(dim=1, keepdim=True)).to(torch.int8).argmax(dim=1)
    assert torch.equal(am, first)
    # columns that start up to 4.7 GB after the base (scan along the middle axis: lanes keep 64-bit offsets)
    xc = x[:70 * 64 * (1 << 18)].view(70, 64, 1 << 18)
    yc = dev(F.cumsum(wrap(hip_backend, xc), 1))
    for rows in (slice(0, 2), slice(-2, None)):
        assert torch.equal(yc[rows], torch.cumsum(xc[rows], 1, dtype=torch.int32))
    del yc
    xt = x[:135000 * 32000].view(135000, 32000)
    Y, I = F.top_k(wrap(hip_backend, xt), 5, 1, True)
    for rows in (slice(0, 32), slice(-32, None)):
        w = torch.sort(xt[rows], dim=1, descending=True, stable=True)
        assert torch.equal(dev(Y)[rows], w.values[:, :5]) and torch.equal(dev(I)[rows].long(), w.indices[:, :5])
    del Y, I, xt
    xs = x[:66000 * 65536].view(66000, 65536)
    ys = dev(F.sort(wrap(hip_backend, xs), 1))
    for rows in (slice(0, 8), slice(32768, 32776), slice(-8, None)):
        assert torch.equal(ys[rows], torch.sort(xs[rows], dim=1).values)


def test_one_row_of_2_26_elements(hip_backend):
    """A single long row (global sort / top-k / softmax over one vector): the routines that cut
    a row into tiles or segments, checked against an independent device implementation."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(17)
    n = 1 << 26
    x = (torch.randn(1, n, device="cuda", generator=g) * 1024).round() / 64            # ties
    X = wrap(hip_backend, x)
    want = torch.sort(x, dim=1, descending=True, stable=True)
    assert torch.equal(dev(F.sort(X, 1, True)), want.values)
    assert torch.equal(dev(F.argsort(X, 1, True)).long(), want.indices)
    for k in (1, 100, 1024):
        Y, I = F.top_k(X, k, 1, True)
        assert torch.equal(dev(Y), want.values[:, :k]) and torch.equal(dev(I).long(), want.indices[:, :k])
    Y, I = F.top_k(X, 7, 1, False, index_dtype=np.int64)
    up = torch.sort(x, dim=1, descending=False, stable=True)
    assert torch.equal(dev(Y), up.values[:, :7]) and torch.equal(dev(I), up.indices[:, :7])
    del want, up
    z = x / 16
    sm = dev(F.softmax(wrap(hip_backend, z), 1)).double()
    ref = torch.softmax(z.double(), 1)
    assert bool(((sm - ref).abs() <= 8 * 26 * EPS32 * ref + 1e-300).all())
    assert abs(float(sm.sum()) - 1.0) < 1e-5
    ls = dev(F.logsoftmax(wrap(hip_backend, z), 1)).double()
    refl = torch.log_softmax(z.double(), 1)
    assert bool(((ls - refl).abs() <= 8 * 26 * EPS32 * (1 + refl.abs())).all())
    hm = dev(F.hardmax(wrap(hip_backend, z), 1))
    assert float(hm.sum()) == 1.0 and int(hm.argmax()) == int((z == z.max()).to(torch.int8).argmax())
    xi = torch.randint(-1000, 1000, (1, n), dtype=torch.int32, device="cuda", generator=g)
    assert torch.equal(dev(F.cumsum(wrap(hip_backend, xi), 1)), torch.cumsum(xi, 1, dtype=torch.int32))
