"""scan: HIP path vs the CPU oracle on the same seeded inputs.

Integers are bit-exact (sums wrap).  fp32 prefixes are compared with the fp64
scan: |got - o64| <= 4 ulp(fp32) * log2(n) * max(|o64|, running sum of |x|).
cummax / cummin are exact for every dtype.
"""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import normal, randint, full_range_i64, ulp_bound
from oracle import oracle as O

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 63, 64, 65, 255, 256, 257, 1000, 1024, 1025, 4095, 4096, 4097, 8192, 12289, 16384, 16385, 20000, 32768, 32769, 100000]


def both(hip, orc, x):
    return Tensor.from_numpy(hip, x), Tensor.from_numpy(orc, x)


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_cumsum_rows_bit_exact(hip_backend, oracle_backend, n, dtype):
    x = randint(41 + n, 3 * n, 0, 100).astype(dtype).reshape(3, n)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for exclusive in (False, True):
        for reverse in (False, True):
            g = F.cumsum(Xh, 1, exclusive, reverse).numpy()
            w = F.cumsum(Xo, 1, exclusive, reverse).numpy()
            assert np.array_equal(g, w), (exclusive, reverse)


@pytest.mark.parametrize("shape,axis", [((5, 7, 300), 0), ((5, 7, 300), 1), ((5, 7, 300), 2),
                                        ((4, 33, 20, 20), 1), ((2, 5000, 3), 1), ((300, 40), 0),
                                        ((1000, 8), 1), ((70, 5000), 0), ((64, 2, 2), 1)])
@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float64])
def test_scan_any_axis(hip_backend, oracle_backend, shape, axis, dtype):
    x = randint(42, int(np.prod(shape)), -50, 50).astype(dtype).reshape(shape)   # exact in every dtype
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for exclusive in (False, True):
        for reverse in (False, True):
            g = F.cumsum(Xh, axis, exclusive, reverse).numpy()
            w = F.cumsum(Xo, axis, exclusive, reverse).numpy()
            assert np.array_equal(g, w), (exclusive, reverse)
    assert np.array_equal(F.cummax(Xh, axis).numpy(), F.cummax(Xo, axis).numpy())
    assert np.array_equal(F.cummin(Xh, axis, reverse=True).numpy(), F.cummin(Xo, axis, reverse=True).numpy())


def test_cumprod_int_and_wrap(hip_backend, oracle_backend):
    x = randint(43, 4 * 3000, 1, 4).astype(np.int64).reshape(4, 3000)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    assert np.array_equal(F.cumprod(Xh, 1).numpy(), F.cumprod(Xo, 1).numpy())
    y = full_range_i64(44, 2 * 100000).astype(np.int32).reshape(2, 100000)    # UniformTest.cpp:2188-2189 shape
    Yh, Yo = both(hip_backend, oracle_backend, y)
    assert np.array_equal(F.cumsum(Yh).numpy(), F.cumsum(Yo).numpy())
    assert np.array_equal(F.cumsum(Yh).numpy(), np.cumsum(y, axis=1, dtype=np.int32))


def test_in_place_and_views(hip_backend, oracle_backend):
    x = randint(45, 6 * 5000, -9, 9).astype(np.int32).reshape(6, 5000)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    F.cumsum(Xh, 1, out=Xh)
    F.cumsum(Xo, 1, out=Xo)
    assert np.array_equal(Xh.numpy(), Xo.numpy())
    # sliced / stepped / transposed inputs written to fresh outputs
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for args in (([1, 3], [5, 4999]), ([0, 4999], [6, 0], None, [2, -3])):
        for axis in (0, 1):
            g = F.cumsum(Xh.slice(*args), axis).numpy()
            w = F.cumsum(Xo.slice(*args), axis).numpy()
            assert np.array_equal(g, w)
    g = F.cumsum(Xh.transpose(), 0, True).numpy()
    assert np.array_equal(g, F.cumsum(Xo.transpose(), 0, True).numpy())


@pytest.mark.parametrize("shape,axis", [((4, 100000), 1), ((3, 4097), 1), ((8, 64, 30, 30), 1), ((2, 1 << 20), 1)])
def test_float_cumsum_tolerance(hip_backend, oracle_backend, shape, axis):
    x = normal(46, int(np.prod(shape))).astype(np.float32).reshape(shape)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for exclusive in (False, True):
        g = np.moveaxis(F.cumsum(Xh, axis, exclusive).numpy(), axis, -1).astype(np.float64)
        n = shape[axis]
        m = x.size // n
        xs = Xo.shape.moveaxis(axis, -1)
        want, mag = O.scan_f64("cumsum", 0, m, n, exclusive, xs, Xo.storage)
        g = g.reshape(m, n)
        bound = ulp_bound(n, np.maximum(np.abs(want), mag)) + 1e-30
        err = np.abs(g - want)
        assert (err <= bound).all(), "worst ratio %g" % (err / bound).max()
        # the reference-association restatement satisfies the same bound
        ref = np.moveaxis(F.cumsum(Xo, axis, exclusive).numpy(), axis, -1).reshape(m, n).astype(np.float64)
        assert (np.abs(ref - want) <= bound).all()


def test_float_cummax_exact_and_cumprod_close(hip_backend, oracle_backend):
    x = normal(47, 5 * 20000).astype(np.float32).reshape(5, 20000)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    assert np.array_equal(F.cummax(Xh, 1).numpy(), F.cummax(Xo, 1).numpy())
    assert np.array_equal(F.cummin(Xh, 1).numpy(), F.cummin(Xo, 1).numpy())
    y = (1.0 + 1e-3 * normal(48, 3 * 5000)).astype(np.float32).reshape(3, 5000)
    Yh, Yo = both(hip_backend, oracle_backend, y)
    np.testing.assert_allclose(F.cumprod(Yh, 1).numpy(), F.cumprod(Yo, 1).numpy(), rtol=2e-4)


def test_many_rows_of_one_tile_and_long_single_row(hip_backend, oracle_backend):
    x = randint(49, 3000 * 300, 0, 100).astype(np.int32).reshape(3000, 300)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    assert np.array_equal(F.cumsum(Xh, 1).numpy(), F.cumsum(Xo, 1).numpy())
    y = randint(50, 3_000_001, 0, 100).astype(np.int32).reshape(1, 3_000_001)
    Yh = Tensor.from_numpy(hip_backend, y)
    assert np.array_equal(F.cumsum(Yh, 1).numpy(), np.cumsum(y, axis=1, dtype=np.int32))


def test_tile_states_cleared_slice_by_slice(hip_backend):
    # Rows of 33 tiles: the tiles' states fill more than one slice of 1024 and a row straddles
    # the slice boundary, so its look-back reads states that two different workgroups cleared.
    # Twice over the same scratch: the second call meets the first call's states and must not
    # take them for its own.
    n = 33 * 32768
    x = randint(54, 40 * n, -100, 100).astype(np.int32).reshape(40, n)
    Xh = Tensor.from_numpy(hip_backend, x)
    want = np.cumsum(x, axis=1, dtype=np.int32)
    assert np.array_equal(F.cumsum(Xh, 1).numpy(), want)
    x2 = (x[::-1] * 3).astype(np.int32).copy()
    Xh2 = Tensor.from_numpy(hip_backend, x2)
    assert np.array_equal(F.cumsum(Xh2, 1).numpy(), np.cumsum(x2, axis=1, dtype=np.int32))
    y = normal(55, 40 * n).astype(np.float64).reshape(40, n)[:6]
    Yh = Tensor.from_numpy(hip_backend, y)
    assert np.array_equal(F.cummax(Yh, 1).numpy(), np.maximum.accumulate(y, axis=1))


def test_two_streams_with_stale_scratch(hip_backend):
    # Two chained scans at once on two streams, each with scratch of its own that is not clean:
    # all ones before the first round, afterwards whatever the round before left (the states and
    # slice words of an earlier call).  Every launch clears its own states while the other
    # stream's launch competes for the compute units, so workgroups need not start in index order.
    torch = hip_backend.torch
    lib = hip_backend.lib
    from dlf_amd.hip_backend import _arr, _check
    m, n = 64, 1 << 20
    a = randint(56, m * n, 0, 100).astype(np.int32).reshape(m, n)
    want = [np.cumsum(a, axis=1, dtype=np.int32), np.cumsum(a[::-1], axis=1, dtype=np.int32)]
    xs = [torch.from_numpy(a).to(hip_backend.device), torch.from_numpy(a[::-1].copy()).to(hip_backend.device)]
    ys = [torch.empty_like(x) for x in xs]
    nbytes = lib.dlfx_scan_scratch_bytes(2, m, n)
    scratch = [torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=hip_backend.device) for _ in range(2)]
    streams = [torch.cuda.Stream(device=hip_backend.device) for _ in range(2)]
    torch.cuda.synchronize(hip_backend.device)
    dims, strides = _arr([m, n]), _arr([n, 1])
    for it in range(24):
        for k in range(2):
            ys[k].zero_()
        torch.cuda.synchronize(hip_backend.device)
        for k in range(2):
            _check(lib.dlfx_scan(streams[k].cuda_stream, b"cumsum", 2, m, n, 0, 2, dims, xs[k].data_ptr(), 0, strides,
                                 ys[k].data_ptr(), 0, strides, scratch[k].data_ptr(), nbytes), "dlfx_scan")
        torch.cuda.synchronize(hip_backend.device)
        for k in range(2):
            assert np.array_equal(ys[k].cpu().numpy(), want[k]), (it, k)


def test_clearing_not_seen_in_time_folds_the_input(hip_backend):
    # With a poll limit of 0 a tile that has not seen its slice's word at its first look gives up
    # at once: it publishes nothing and folds every predecessor from the input; tiles behind it
    # time out on it the same way.  Dirty scratch, so that a state read by mistake would show.
    torch = hip_backend.torch
    lib = hip_backend.lib
    from dlf_amd.hip_backend import _arr, _check
    m, n = 6, 40 * 32768 + 77
    a = randint(57, m * n, -100, 100).astype(np.int32).reshape(m, n)
    x = torch.from_numpy(a).to(hip_backend.device)
    y = torch.empty_like(x)
    nbytes = lib.dlfx_scan_scratch_bytes(2, m, n)
    scratch = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=hip_backend.device)
    stream = torch.cuda.current_stream(hip_backend.device).cuda_stream
    hip_backend.set_tuning("scan_poll_limit", 0)
    try:
        for _ in range(3):
            _check(lib.dlfx_scan(stream, b"cumsum", 2, m, n, 0, 2, _arr([m, n]), x.data_ptr(), 0, _arr([n, 1]),
                                 y.data_ptr(), 0, _arr([n, 1]), scratch.data_ptr(), nbytes), "dlfx_scan")
            torch.cuda.synchronize(hip_backend.device)
            assert np.array_equal(y.cpu().numpy(), np.cumsum(a, axis=1, dtype=np.int32))
    finally:
        hip_backend.set_tuning("scan_poll_limit", 2048)


def test_bounded_wait_self_help_path(hip_backend, oracle_backend):
    # With a poll limit of 0 a tile never waits: whatever predecessor has not
    # published yet is folded from the input by the waiting tile itself.
    x = randint(51, 5 * 200000, -100, 100).astype(np.int32).reshape(5, 200000)
    y = randint(52, 3 * 70000, -10**9, 10**9).astype(np.int64).reshape(3, 70000)
    hip_backend.set_tuning("scan_poll_limit", 0)
    try:
        for a in (x, y):
            Xh, Xo = both(hip_backend, oracle_backend, a)
            for exclusive in (False, True):
                for reverse in (False, True):
                    g = F.cumsum(Xh, 1, exclusive, reverse).numpy()
                    assert np.array_equal(g, F.cumsum(Xo, 1, exclusive, reverse).numpy())
            assert np.array_equal(F.cummax(Xh, 1).numpy(), F.cummax(Xo, 1).numpy())
    finally:
        hip_backend.set_tuning("scan_poll_limit", 2048)


def test_in_place_long_rows_use_tickets(hip_backend, oracle_backend):
    x = randint(53, 4 * 300000, -100, 100).astype(np.int32).reshape(4, 300000)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    F.cumsum(Xh, 1, out=Xh)
    F.cumsum(Xo, 1, out=Xo)
    assert np.array_equal(Xh.numpy(), Xo.numpy())
    # ... and rows off a 16-byte boundary (an odd length), whose tiles start before the row
    for n in (300001, 70003):
        z = randint(54 + n, 5 * n, -100, 100).astype(np.int32).reshape(5, n)
        Z = Tensor.from_numpy(hip_backend, z)
        F.cumsum(Z, 1, out=Z)
        assert np.array_equal(Z.numpy(), np.cumsum(z, axis=1, dtype=np.int32))
    # In-place *exclusive* scans: the reference's CPU loop stores the running value
    # into y before it reads x (reduce_detail.h:183-187), so with y aliasing x it
    # loses the input it has yet to read.  That is a read-after-write slip, not a
    # specification; the HIP path must equal the out-of-place answer.
    Xh, Xo = both(hip_backend, oracle_backend, x)
    F.cumsum(Xh, 1, True, True, out=Xh)
    assert np.array_equal(Xh.numpy(), F.cumsum(Xo, 1, True, True).numpy())
    F.cumsum(Xo, 1, True, True, out=Xo)
    assert not np.array_equal(Xo.numpy(), Xh.numpy())     # the restated reference loop reproduces the slip


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 7, 8, 9, 13, 15, 16, 17, 63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257, 511, 512, 513, 767, 768, 769])
def test_short_rows_one_lane_group_per_row(hip_backend, oracle_backend, n):
    """Rows of up to 768 elements along a unit-stride axis are scanned by a group of 1, 4, 16 or
    64 lanes each.  Every size class; all four scans; exclusive and reversed; integer results are
    exact, floating ones within the usual bound of the fp64 evaluation."""
    m = 37 if n > 16 else 1037                       # several workgroups of thread- and quad-sized groups
    xi = randint(220 + n, m * n, -9, 10).astype(np.int32).reshape(m, n)
    Xi = Tensor.from_numpy(hip_backend, xi)
    for exclusive in (False, True):
        for reverse in (False, True):
            src = xi[:, ::-1] if reverse else xi
            want = np.cumsum(src, axis=1, dtype=np.int32)
            if exclusive:
                want = np.concatenate([np.zeros((m, 1), np.int32), want[:, :-1]], axis=1)
            want = want[:, ::-1] if reverse else want
            assert np.array_equal(F.cumsum(Xi, 1, exclusive, reverse).numpy(), want), (exclusive, reverse)
    assert np.array_equal(F.cummax(Xi, 1).numpy(), np.maximum.accumulate(xi, axis=1))
    assert np.array_equal(F.cummin(Xi, 1, True).numpy(), np.minimum.accumulate(xi[:, ::-1], axis=1)[:, ::-1])
    small = randint(221 + n, m * n, 1, 3).astype(np.int64).reshape(m, n)
    assert np.array_equal(F.cumprod(Tensor.from_numpy(hip_backend, small), 1).numpy(), np.cumprod(small, axis=1))   # wraps like numpy
    for dtype in (np.float32, np.float64, np.float16):
        xf = (normal(222 + n, m * n) * 0.5).astype(dtype).reshape(m, n)
        got = F.cumsum(Tensor.from_numpy(hip_backend, xf), 1).numpy().astype(np.float64)
        x64 = xf.astype(np.float64)
        want, mag = np.cumsum(x64, axis=1), np.cumsum(np.abs(x64), axis=1)
        eps = np.finfo(np.float32 if dtype == np.float16 else dtype).eps
        out_ulp = 2.0 ** -10 if dtype == np.float16 else 0.0
        assert (np.abs(got - want) <= 4 * max(1.0, np.log2(n)) * eps * mag + out_ulp * np.abs(want) + 1e-30).all(), dtype
    xc = ((normal(223 + n, m * n) + 1j * normal(224 + n, m * n)) * 0.5).astype(np.complex64).reshape(m, n)
    assert np.allclose(F.cumsum(Tensor.from_numpy(hip_backend, xc), 1, True).numpy()[:, 1:], np.cumsum(xc.astype(np.complex128), axis=1)[:, :-1], rtol=1e-5, atol=1e-5)
    # in place, and rows that are not 16-byte aligned (a sliced view)
    Z = Tensor.from_numpy(hip_backend, xi)
    F.cumsum(Z, 1, out=Z)
    assert np.array_equal(Z.numpy(), np.cumsum(xi, axis=1, dtype=np.int32))
    if n > 3:
        V = Xi.slice([1], [n], [1])
        assert np.array_equal(F.cumsum(V, 1).numpy(), np.cumsum(xi[:, 1:], axis=1, dtype=np.int32))
    # the same rows as columns of the transposed view: the axis is no longer unit-stride
    assert np.array_equal(F.cumsum(Xi.transpose(), 0).numpy(), np.cumsum(xi, axis=1, dtype=np.int32).T)


@pytest.mark.parametrize("n", [9, 70, 130, 190, 300, 601, 766, 1000, 5000, 16383, 16387, 40001, 150003])
def test_rows_off_a_vector_boundary(hip_backend, oracle_backend, n):
    """Unit-stride rows that do not start on a 16-byte boundary - odd row lengths, views cut one or
    two elements into a row - are laid out from the boundary before each row, so that their whole
    vectors still move as one access.  Input and output off the boundary by the same or by
    different amounts, every kernel size class, 4-, 8- and 2-byte elements, exclusive and reversed,
    and (long rows) with tiles that never wait for their predecessors."""
    m = 5
    for dtype in (np.int32, np.int64):
        x = randint(230 + n, m * (n + 3), -50, 50).astype(dtype).reshape(m, n + 3)
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for cut in (1, 2, 3):
            Vh, Vo = Xh.slice([cut], [cut + n], [1]), Xo.slice([cut], [cut + n], [1])
            for exclusive in (False, True):
                for reverse in (False, True):
                    assert np.array_equal(F.cumsum(Vh, 1, exclusive, reverse).numpy(), F.cumsum(Vo, 1, exclusive, reverse).numpy()), (dtype, cut, exclusive, reverse)
        # the output off the boundary by another amount than the input
        Yh = Tensor.from_numpy(hip_backend, np.zeros((m, n + 3), dtype))
        F.cumsum(Xh.slice([1], [1 + n], [1]), 1, out=Yh.slice([2], [2 + n], [1]))
        got = Yh.numpy()
        assert np.array_equal(got[:, 2: 2 + n], np.cumsum(x[:, 1: 1 + n], axis=1, dtype=dtype))
        assert not got[:, :2].any() and not got[:, 2 + n:].any()          # nothing written beside the rows
        assert np.array_equal(F.cummax(Xh.slice([3], [3 + n], [1]), 1).numpy(), np.maximum.accumulate(x[:, 3: 3 + n], axis=1))
    xh = (normal(231 + n, m * (n + 1)) * 0.25).astype(np.float16).reshape(m, n + 1)
    got = F.cumsum(Tensor.from_numpy(hip_backend, xh).slice([1], [1 + n], [1]), 1).numpy().astype(np.float64)
    x64 = xh[:, 1:].astype(np.float64)
    want, mag = np.cumsum(x64, axis=1), np.cumsum(np.abs(x64), axis=1)
    assert (np.abs(got - want) <= 4 * max(1.0, np.log2(n)) * np.finfo(np.float32).eps * mag + 2.0 ** -10 * np.abs(want) + 1e-30).all()
    if n > 20000:
        hip_backend.set_tuning("scan_poll_limit", 0)
        try:
            x = randint(232 + n, m * (n + 1), -50, 50).astype(np.int32).reshape(m, n + 1)
            Xh = Tensor.from_numpy(hip_backend, x)
            assert np.array_equal(F.cumsum(Xh.slice([1], [1 + n], [1]), 1).numpy(), np.cumsum(x[:, 1:], axis=1, dtype=np.int32))
        finally:
            hip_backend.set_tuning("scan_poll_limit", 2048)


@pytest.mark.parametrize("n", [8, 64, 200, 512, 776, 1024, 4096, 16384, 40000, 150008, 1 << 20])
def test_rows_walked_backwards_move_whole_vectors(hip_backend, oracle_backend, n):
    """A reversed scan walks a unit-stride row with stride -1; rows that end on a 16-byte boundary
    load and store whole vectors, last element first.  Input and output reversed together (the
    reverse scans), only one of them (a flipped view scanned into a forward result and the other
    way round), in place, 2-, 4- and 8-byte elements, every kernel size class; rows that end off
    the boundary (views cut short by one to three elements) take the element-wise path in the
    same launch."""
    m = 5 if n < 100000 else 2
    for dtype in (np.int32, np.int64):
        x = randint(260 + n, m * n, -50, 50).astype(dtype).reshape(m, n)
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for exclusive in (False, True):
            assert np.array_equal(F.cumsum(Xh, 1, exclusive, True).numpy(), F.cumsum(Xo, 1, exclusive, True).numpy()), (dtype, exclusive)
        want = np.cumsum(x[:, ::-1], axis=1, dtype=dtype)
        assert np.array_equal(F.cumsum(Xh.flip([1]), 1).numpy(), want), dtype                 # reversed in, forward out
        Yh = Tensor.from_numpy(hip_backend, np.zeros((m, n), dtype))
        F.cumsum(Xh, 1, out=Yh.flip([1]))                                                     # forward in, reversed out
        assert np.array_equal(Yh.numpy(), np.cumsum(x, axis=1, dtype=dtype)[:, ::-1]), dtype
        assert np.array_equal(F.cummax(Xh, 1, True).numpy(), np.maximum.accumulate(x[:, ::-1], axis=1)[:, ::-1]), dtype
        assert np.array_equal(F.cumprod(Xh, 1, False, True).numpy(), F.cumprod(Xo, 1, False, True).numpy()), dtype
        for cut in (1, 2, 3):
            if n > cut:
                Vh, Vo = Xh.slice([0], [n - cut], [1]), Xo.slice([0], [n - cut], [1])
                assert np.array_equal(F.cumsum(Vh, 1, False, True).numpy(), F.cumsum(Vo, 1, False, True).numpy()), (dtype, cut)
        Zh = Tensor.from_numpy(hip_backend, x)
        F.cumsum(Zh, 1, False, True, out=Zh)                                                  # in place
        assert np.array_equal(Zh.numpy(), np.cumsum(x[:, ::-1], axis=1, dtype=dtype)[:, ::-1]), dtype
    xh = (normal(261 + n, m * n) * 0.25).astype(np.float16).reshape(m, n)
    got = F.cumsum(Tensor.from_numpy(hip_backend, xh), 1, False, True).numpy().astype(np.float64)
    x64 = xh[:, ::-1].astype(np.float64)
    want, mag = np.cumsum(x64, axis=1)[:, ::-1], np.cumsum(np.abs(x64), axis=1)[:, ::-1]
    assert (np.abs(got - want) <= 4 * max(1.0, np.log2(n)) * np.finfo(np.float32).eps * mag + 2.0 ** -10 * np.abs(want) + 1e-30).all()
    xb = (randint(262 + n, m * n, 0, 3) == 0)
    xb = xb.reshape(m, n)
    assert np.array_equal(F.cumsum(Tensor.from_numpy(hip_backend, xb.astype(np.int64)), 1, True, True).numpy(),
                          (np.cumsum(xb[:, ::-1], axis=1, dtype=np.int64) - xb[:, ::-1])[:, ::-1])


@pytest.mark.parametrize("shape,axis", [((40000, 64), 0), ((100000, 17), 0), ((3, 9000, 100), 1), ((2050, 1000), 0), ((262144, 8), 0), ((5000, 7), 0)])
def test_long_axis_beside_few_columns_is_cut_into_segments(hip_backend, shape, axis):
    # an axis that is not the innermost, long, with too few columns beside it to fill the device:
    # workgroups take segments of the axis and start from the totals of the segments before them
    # (the last shape has too few columns for that kernel and keeps the strided rows)
    x = randint(480, int(np.prod(shape)), -50, 50).astype(np.int32).reshape(shape)
    Xh = Tensor.from_numpy(hip_backend, x)
    assert np.array_equal(F.cumsum(Xh, axis).numpy(), np.cumsum(x, axis=axis, dtype=np.int32))
    ex = np.cumsum(x, axis=axis, dtype=np.int32) - x
    assert np.array_equal(F.cumsum(Xh, axis, True).numpy(), ex)
    rev = np.flip(np.cumsum(np.flip(x, axis), axis=axis, dtype=np.int32), axis)
    assert np.array_equal(F.cumsum(Xh, axis, False, True).numpy(), rev)
    assert np.array_equal(F.cummax(Xh, axis).numpy(), np.maximum.accumulate(x, axis=axis))
    assert np.array_equal(F.cummin(Xh, axis).numpy(), np.minimum.accumulate(x, axis=axis))
    y = (normal(481, int(np.prod(shape))) * 3).astype(np.float32).reshape(shape)
    Yh = Tensor.from_numpy(hip_backend, y)
    got = F.cumsum(Yh, axis).numpy().astype(np.float64)
    want = np.cumsum(y.astype(np.float64), axis=axis)
    mag = np.cumsum(np.abs(y.astype(np.float64)), axis=axis)
    n = shape[axis]
    assert np.all(np.abs(got - want) <= 4 * np.log2(n) * np.finfo(np.float32).eps * np.maximum(np.abs(want), mag))
    F.cumsum(Xh, axis, out=Xh)                                          # in place
    assert np.array_equal(Xh.numpy(), np.cumsum(x, axis=axis, dtype=np.int32))


@pytest.mark.parametrize("shape,axis", [((8, 21, 64, 64), 1), ((4, 100, 30, 30), 1), ((4096, 128), 0), ((3, 5000, 66), 1), ((5000, 67), 0),
                                        ((64, 3, 25, 25), 1), ((2, 40, 6, 10, 12), 1), ((70000, 6), 0)])
def test_two_byte_columns_go_two_to_a_lane(hip_backend, shape, axis):
    """Half elements along an axis that is not the innermost: a lane takes two columns that lie
    side by side (one 4-byte access) where every such pair starts on a 4-byte boundary - an even
    number of columns in the innermost run, even strides, an aligned base - and one column
    otherwise (odd extents, views that start at an odd element).  Running maxima and minima are
    exact, running sums held to the fp32 bound; short axes, long axes cut into segments, views,
    in place, exclusive and reversed."""
    x = (normal(500, int(np.prod(shape))) * 2).astype(np.float16).reshape(shape)
    Xh = Tensor.from_numpy(hip_backend, x)
    n = shape[axis]

    def check_sum(got, src, ax, exclusive=False, reverse=False):
        s64 = src.astype(np.float64)
        if reverse:
            s64 = np.flip(s64, ax)
        want, mag = np.cumsum(s64, axis=ax), np.cumsum(np.abs(s64), axis=ax)
        if exclusive:
            want, mag = want - s64, mag
        if reverse:
            want, mag = np.flip(want, ax), np.flip(mag, ax)
        err = np.abs(got.astype(np.float64) - want)
        assert (err <= 4 * max(1.0, np.log2(n)) * np.finfo(np.float32).eps * mag + 2.0 ** -10 * np.abs(want) + 1e-30).all()

    assert np.array_equal(F.cummax(Xh, axis).numpy(), np.maximum.accumulate(x, axis=axis))
    assert np.array_equal(F.cummin(Xh, axis).numpy(), np.minimum.accumulate(x, axis=axis))
    assert np.array_equal(F.cummax(Xh, axis, True).numpy(), np.flip(np.maximum.accumulate(np.flip(x, axis), axis=axis), axis))
    check_sum(F.cumsum(Xh, axis).numpy(), x, axis)
    check_sum(F.cumsum(Xh, axis, True).numpy(), x, axis, exclusive=True)
    check_sum(F.cumsum(Xh, axis, False, True).numpy(), x, axis, reverse=True)
    # views of the innermost dimension: an even start keeps the pairs, an odd start or an odd length does not
    last = len(shape) - 1
    w = shape[last]
    for lo, hi in ((2, w), (1, w - 1), (0, w - 1), (2, w - 2)):
        if hi - lo < 1:
            continue
        Vh = Xh.slice([lo], [hi], [last])
        v = x[..., lo:hi]
        assert np.array_equal(F.cummax(Vh, axis).numpy(), np.maximum.accumulate(v, axis=axis)), (lo, hi)
        check_sum(F.cumsum(Vh, axis).numpy(), v, axis)
        # into a view of a larger result: nothing is written beside it
        Yh = Tensor.from_numpy(hip_backend, np.full(shape, 7, np.float16))
        F.cummin(Vh, axis, out=Yh.slice([lo], [hi], [last]))
        got = Yh.numpy()
        assert np.array_equal(got[..., lo:hi], np.minimum.accumulate(v, axis=axis)), (lo, hi)
        assert (got[..., :lo] == 7).all() and (got[..., hi:] == 7).all(), (lo, hi)
    # every other column (stride 2 in the innermost dimension: no neighbours to pair)
    Sh = Xh.slice([0], [w], [last], [2])
    assert np.array_equal(F.cummax(Sh, axis).numpy(), np.maximum.accumulate(x[..., ::2], axis=axis))
    # the columns walked backwards
    assert np.array_equal(F.cummax(Xh.flip([last]), axis).numpy(), np.maximum.accumulate(x[..., ::-1], axis=axis))
    Zh = Tensor.from_numpy(hip_backend, x)
    F.cummax(Zh, axis, out=Zh)                                           # in place
    assert np.array_equal(Zh.numpy(), np.maximum.accumulate(x, axis=axis))
    # one column a lane gives the same, sums included (the same additions in the same order)
    pairs = F.cumsum(Xh, axis).numpy()
    hip_backend.set_tuning("scan_cols_per_lane", 1)
    try:
        singles = F.cumsum(Xh, axis).numpy()
    finally:
        hip_backend.set_tuning("scan_cols_per_lane", 0)
    assert np.array_equal(pairs.view(np.uint16), singles.view(np.uint16))


@pytest.mark.parametrize("shape,axis", [((8, 21, 64, 64), 1), ((64, 3, 50, 50), 1), ((5000, 2, 3), 1), ((3, 32, 5000), 1), ((2, 33, 5000), 1),
                                        ((17, 8000), 0), ((4, 5, 6, 700), 2)])
def test_short_axis_beside_many_columns_one_lane_per_column(hip_backend, shape, axis):
    # an axis of up to 32 positions that is not the innermost, beside thousands of columns: every lane
    # scans a column in registers (33 positions: the kernel of four wavefronts a round)
    x = randint(490, int(np.prod(shape)), -50, 50).astype(np.int32).reshape(shape)
    Xh = Tensor.from_numpy(hip_backend, x)
    inc = np.cumsum(x, axis=axis, dtype=np.int32)
    assert np.array_equal(F.cumsum(Xh, axis).numpy(), inc)
    assert np.array_equal(F.cumsum(Xh, axis, True).numpy(), inc - x)
    assert np.array_equal(F.cumsum(Xh, axis, True, True).numpy(), np.flip(np.cumsum(np.flip(x, axis), axis=axis, dtype=np.int32), axis) - x)
    assert np.array_equal(F.cummax(Xh, axis).numpy(), np.maximum.accumulate(x, axis=axis))
    assert np.array_equal(F.cumprod(Xh, axis).numpy(), np.cumprod(x, axis=axis, dtype=np.int32))
    y = (normal(491, int(np.prod(shape))) * 3).astype(np.float64).reshape(shape)
    Yh = Tensor.from_numpy(hip_backend, y)
    assert np.allclose(F.cumsum(Yh, axis).numpy(), np.cumsum(y, axis=axis), rtol=1e-12, atol=1e-12)
    sl = Xh.slice([0], [shape[-1] - 1], [len(shape) - 1], [2])            # every other innermost element: columns with a step
    assert np.array_equal(F.cumsum(sl, axis).numpy(), np.cumsum(x[..., 0:shape[-1] - 1:2], axis=axis, dtype=np.int32))
    F.cumsum(Xh, axis, out=Xh)
    assert np.array_equal(Xh.numpy(), inc)
