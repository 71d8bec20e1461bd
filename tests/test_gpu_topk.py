"""top_k: HIP path vs the CPU oracle, bit-exact.

Values must equal what the reference's heap algorithm returns (restated in the
oracle, mode 0).  Indices must equal the specification order -- first `limit`
entries of a stable sort, so the lowest index wins ties (oracle mode 1; the
reference's own tie order is implementation-defined and its test concedes the
indices may differ) -- and gather(X, I) must reproduce the values.
"""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import normal, randint, full_range_i64
from oracle.oracle import OracleBackend

pytestmark = pytest.mark.gpu


def check(hip, x, k, axis=-1, largest=True, index_dtype=np.int32):
    spec, heap = OracleBackend(topk_mode=1), OracleBackend(topk_mode=0)
    Yh, Ih = F.top_k(Tensor.from_numpy(hip, x), k, axis, largest, index_dtype)
    Ys, Is = F.top_k(Tensor.from_numpy(spec, x), k, axis, largest, index_dtype)
    Yr, _ = F.top_k(Tensor.from_numpy(heap, x), k, axis, largest, index_dtype)
    yh, ih = Yh.numpy(), Ih.numpy()
    assert ih.dtype == np.dtype(index_dtype)
    assert np.array_equal(yh, Ys.numpy()) and np.array_equal(yh, Yr.numpy())
    assert np.array_equal(ih, Is.numpy())
    assert np.array_equal(F.gather_elements(x, ih, axis), yh)


def quantised(seed, shape):
    return (np.round(normal(seed, int(np.prod(shape))) * 2 * 256) / 256).astype(np.float32).reshape(shape)


@pytest.mark.parametrize("k", [1, 5, 50, 256])
@pytest.mark.parametrize("largest", [True, False])
def test_quantised_rows_with_ties(hip_backend, k, largest):
    check(hip_backend, quantised(70, (24, 32000)), k, -1, largest)           # benchmark row shape
    check(hip_backend, quantised(71, (40, 1000)), k, -1, largest, np.int64)  # logits-head shape


@pytest.mark.parametrize("n", [1, 2, 10, 255, 256, 257, 1000, 1024, 1025, 2048, 4097, 8192, 10000, 16385, 32769, 65536])
def test_row_lengths(hip_backend, n):
    x = randint(72 + n, 3 * n, 0, 50).astype(np.int32).reshape(3, n)       # heavy ties
    for k in sorted({1, min(n, 7), min(n, 200), min(n, 1024)}):
        check(hip_backend, x, k, -1, True)
        check(hip_backend, x, k, -1, False)


@pytest.mark.parametrize("n", [1027, 4099, 8191, 8193, 8199, 16381, 16387, 32765, 32771, 50257, 65533, 65535])
def test_rows_off_a_vector_boundary(hip_backend, oracle_backend, n):
    """Contiguous rows of an odd length start at every offset within a 16-byte vector; beyond 8192
    elements they are read as whole vectors from the boundary before each row, which makes a
    row up to a vector less one element longer (a longer size class just below a class limit;
    no change where that would take the row past what one workgroup holds, or from the rows
    that finish in one launch into those that may spill).  Ties across the padding on either
    side of a row, the row's first and last elements among the winners, a view that starts
    mid-buffer, all element widths."""
    for dtype in (np.float32, np.int64, np.float16, np.int16, np.float64):
        x = (normal(300 + n, 6 * n) * 300).astype(dtype).reshape(6, n)
        x[1, 0] = x[1].max() + 1                       # the first element wins
        x[2, n - 1] = x[2].max() + 1                   # ... the last
        x[3] = x[3, 0]                                 # all equal: the lowest indices win
        x[4, ::3] = x[4].min()                         # a third of the row ties at the bottom
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for k in (1, 5, 40, 300):
            for largest in (True, False):
                Yh, Ih = F.top_k(Xh, k, -1, largest)
                Yo, Io = F.top_k(Xo, k, -1, largest)
                assert np.array_equal(Ih.numpy(), Io.numpy()), (dtype, k, largest)
                assert np.array_equal(Yh.numpy().view(np.uint8), Yo.numpy().view(np.uint8)), (dtype, k, largest)
        Vh, Vo = Xh.slice([1], [6], [0]), Xo.slice([1], [6], [0])      # the rows from the second on
        Yh, Ih = F.top_k(Vh, 7, -1, True)
        Yo, Io = F.top_k(Vo, 7, -1, True)
        assert np.array_equal(Ih.numpy(), Io.numpy()) and np.array_equal(Yh.numpy().view(np.uint8), Yo.numpy().view(np.uint8))


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_dtypes_and_axes(hip_backend, dtype):
    if np.dtype(dtype).kind == "f":
        x = (normal(73, 6 * 40 * 30) * 100).astype(dtype).reshape(6, 40, 30)
    else:
        x = full_range_i64(73, 6 * 40 * 30).astype(dtype).reshape(6, 40, 30)
    for axis in (0, 1, 2):
        check(hip_backend, x, 5, axis, True)
        check(hip_backend, x, 3, axis, False, np.int64)


def test_reference_test_shapes(hip_backend):
    # UniformTest.cpp:2494-2535: [2, n] ints, k = 10 / 200 / 500 / 1000
    for n in (10, 500, 1000):
        check(hip_backend, randint(74 + n, 2 * n, 0, 10000).astype(np.int32).reshape(2, n), 10)
    for n in (1000, 5000, 10000):
        x = randint(75 + n, 2 * n, 0, 100000).astype(np.int32).reshape(2, n)
        for k in (200, 500, 1000):
            check(hip_backend, x, k)


def test_all_equal_rows_and_k_equals_n(hip_backend):
    x = np.full((4, 3000), 7, dtype=np.int64)
    Y, I = F.top_k(Tensor.from_numpy(hip_backend, x), 100)
    assert np.array_equal(I.numpy(), np.tile(np.arange(100, dtype=np.int32), (4, 1)))
    assert (Y.numpy() == 7).all()
    y = randint(76, 5 * 300, -5, 5).astype(np.int32).reshape(5, 300)
    check(hip_backend, y, 300)
    check(hip_backend, y, 1000)          # limit clamps to the extent


def test_long_rows_and_large_limits_take_the_sort_path(hip_backend):
    check(hip_backend, quantised(77, (3, 100000)), 50)
    check(hip_backend, randint(78, 2 * 20000, 0, 1000).astype(np.int32).reshape(2, 20000), 3000, -1, False)
    check(hip_backend, full_range_i64(79, 2 * 40000).reshape(2, 40000), 10, -1, True, np.int64)


def test_signed_zeros_and_infinities(hip_backend):
    x = np.array([[0.0, -0.0, -1.0, -0.0, np.inf, -np.inf, 0.0, 3.0]], dtype=np.float32)
    Y, I = F.top_k(Tensor.from_numpy(hip_backend, x), 5)
    assert I.numpy().tolist() == [[4, 7, 0, 1, 3]]
    assert np.array_equal(np.signbit(Y.numpy()[0]), np.signbit(x[0][I.numpy()[0]]))
    Y, I = F.top_k(Tensor.from_numpy(hip_backend, x), 4, largest=False)
    assert I.numpy().tolist() == [[5, 2, 0, 1]]


def test_strided_views(hip_backend):
    x = randint(80, 40 * 700, 0, 30).astype(np.int32).reshape(40, 700)
    X = Tensor.from_numpy(hip_backend, x)
    from oracle.oracle import OracleBackend as OB
    Xo = Tensor.from_numpy(OB(1), x)
    for args in (([3, 5], [37, 690]), ([0, 699], [40, 0], None, [3, -2])):
        Yh, Ih = F.top_k(X.slice(*args), 9, -1)
        Yo, Io = F.top_k(Xo.slice(*args), 9, -1)
        assert np.array_equal(Yh.numpy(), Yo.numpy()) and np.array_equal(Ih.numpy(), Io.numpy())
        Yh, Ih = F.top_k(X.slice(*args), 4, 0, False)
        Yo, Io = F.top_k(Xo.slice(*args), 4, 0, False)
        assert np.array_equal(Yh.numpy(), Yo.numpy()) and np.array_equal(Ih.numpy(), Io.numpy())


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
@pytest.mark.parametrize("n,k", [(700, 5), (5000, 50), (32000, 5), (32000, 256), (40000, 17)])
def test_top_k_with_nans_agrees_with_the_sort(hip_backend, dtype, n, k):
    """The reference leaves the place of NaNs open (its comparisons are not an order on them).
    Here they are ordered by their bit pattern everywhere - positive NaNs above +inf, negative
    ones below -inf - so top_k must return the head of the stable argsort, bit for bit, whatever
    path selects the row."""
    x = (normal(190 + n + k, 4 * n) * 3).astype(dtype).reshape(4, n)
    bits = {np.float32: np.uint32, np.float64: np.uint64, np.float16: np.uint16}[dtype]
    pos_nan = np.array([np.nan], dtype=dtype)
    neg_nan = (pos_nan.view(bits) | (bits(1) << bits(8 * dtype().itemsize - 1))).view(dtype)
    x[0, [3, n // 2, n - 1]] = pos_nan[0]
    x[1, [0, n // 3]] = neg_nan[0]
    x[1, [5, n - 2]] = pos_nan[0]
    x[2, n // 7] = np.inf
    x[2, n // 5] = -np.inf                       # infinities of both signs, no NaN
    X = Tensor.from_numpy(hip_backend, x)
    for largest in (True, False):
        Y, I = F.top_k(X, k, -1, largest)
        SV, SI = F.argsort(X, -1, largest, with_values=True)
        assert np.array_equal(I.numpy(), SI.numpy()[:, :k]), largest
        assert np.array_equal(Y.numpy().view(bits), SV.numpy()[:, :k].view(bits)), largest
    top = F.top_k(X, 3, -1, True)[0].numpy()
    assert np.isnan(top[0]).all() and np.isnan(top[1][:2]).all() and top[2, 0] == np.inf


@pytest.mark.parametrize("n", [1, 5, 63, 64, 65, 128, 129, 255, 256, 257, 1000, 1024, 1025, 1300, 2048, 2049, 2300, 3000, 4096])
def test_short_rows_one_wave_per_row(hip_backend, oracle_backend, n):
    """Rows of up to 1024 elements with limits up to 32, and rows of up to 256 elements with any
    limit (the wave then orders the whole row), are selected by one wavefront each; beyond
    (rows of up to 4096 elements, larger limits) a workgroup of 256 or 1024 threads per row
    pre-filters with a bound from its full waves' maxima (a row that does not fill the
    workgroup leaves its last waves empty, and a limit above the number of full ones must not
    take its bound from them) and selects from its registers when too many survive.
    Every size class, limits up to the cap, both directions, all element types, and the rows
    that defeat the bound (all equal, few distinct values, sorted either way)."""
    for dtype in (np.float32, np.int32, np.float64, np.int64, np.float16, np.int16):
        x = (normal(210 + n, 7 * n) * 40).astype(dtype).reshape(7, n)
        x[1] = 3                                               # all equal: every element reaches the bound
        x[2] = randint(211 + n, n, 0, 3).astype(dtype)         # three distinct values
        x[3] = np.sort(x[3])
        x[4] = np.sort(x[4])[::-1]
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for k in sorted({1, min(n, 5), min(n, 9), min(n, 16), min(n, 17), min(n, 32), min(n, 33), min(n, 64), min(n, 65), min(n, 200), min(n, 256), min(n, 257), min(n, 700)}):
            for largest in (True, False):
                Yh, Ih = F.top_k(Xh, k, -1, largest)
                Yo, Io = F.top_k(Xo, k, -1, largest)
                assert np.array_equal(Ih.numpy(), Io.numpy()), (dtype, k, largest)
                assert np.array_equal(Yh.numpy().view(np.uint8), Yo.numpy().view(np.uint8))
    # 64-bit indices and a strided view
    a = (normal(212, 33 * 5 * max(n, 2)) * 9).astype(np.float32).reshape(33, 5, max(n, 2))
    T, O = Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(oracle_backend, a)
    k = min(3, a.shape[2])
    Yh, Ih = F.top_k(T.flip([2]), k, 2, True, index_dtype=np.int64)
    Yo, Io = F.top_k(O.flip([2]), k, 2, True)
    assert Ih.numpy().dtype == np.int64 and np.array_equal(Ih.numpy(), Io.numpy()) and np.array_equal(Yh.numpy(), Yo.numpy())
    Yh, Ih = F.top_k(T, min(4, a.shape[0]), 0, False)
    Yo, Io = F.top_k(O, min(4, a.shape[0]), 0, False)
    assert np.array_equal(Ih.numpy(), Io.numpy()) and np.array_equal(Yh.numpy(), Yo.numpy())


@pytest.mark.parametrize("n", [1, 2, 7, 63, 64, 100, 511, 512, 700])
def test_rows_side_by_side_in_memory(hip_backend, oracle_backend, n):
    """top_k along an outer axis with a limit of at most 16: one thread per row, several waves
    per row segment.  Every list length, both directions, all element types, rows that are all
    ties, row counts that leave lanes idle, and a middle axis."""
    cols = 16400 + n % 50
    for dtype in (np.float32, np.int32, np.float64, np.int64, np.float16, np.int16):
        x = (normal(230 + n, n * cols) * 40).astype(dtype).reshape(n, cols)
        x[:, 1] = 3                                                   # all equal
        x[:, 2] = randint(231 + n, n, 0, 3).astype(dtype)             # three distinct values
        x[:, 3] = np.sort(x[:, 3], kind="stable")
        x[:, 4] = np.sort(x[:, 4], kind="stable")[::-1]
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for k in sorted({1, min(n, 2), min(n, 3), min(n, 4), min(n, 5), min(n, 8), min(n, 9), min(n, 16)}):
            for largest in (True, False):
                Yh, Ih = F.top_k(Xh, k, 0, largest)
                Yo, Io = F.top_k(Xo, k, 0, largest)
                assert np.array_equal(Ih.numpy(), Io.numpy()), (dtype, k, largest)
                assert np.array_equal(Yh.numpy().view(np.uint8), Yo.numpy().view(np.uint8))
    a = (normal(232, 3 * n * 6000) * 9).astype(np.float32).reshape(3, n, 6000)
    a[1, :, 17] = np.nan                                              # ordered by bit pattern, as in the sort
    a[2, n // 2, :] = -0.0
    a[2, 0, :] = 0.0
    T, O = Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(oracle_backend, a)
    k = min(5, n)
    Yh, Ih = F.top_k(T, k, 1, True, index_dtype=np.int64)
    SV, SI = F.argsort(T, 1, True, with_values=True)
    assert Ih.numpy().dtype == np.int64 and np.array_equal(Ih.numpy(), SI.numpy()[:, :k, :])
    assert np.array_equal(Yh.numpy().view(np.uint32), SV.numpy()[:, :k, :].view(np.uint32))
    Yh, Ih = F.top_k(T.flip([1]), k, 1, False)
    Yo, Io = F.top_k(O.flip([1]), k, 1, False)
    ok = ~np.isnan(Yo.numpy())
    assert np.array_equal(Ih.numpy()[ok], Io.numpy()[ok]) and np.array_equal(Yh.numpy()[ok], Yo.numpy()[ok])


@pytest.mark.parametrize("n", [64, 200, 513])
def test_rows_side_by_side_any_number_of_waves(hip_backend, oracle_backend, n):
    """The wavefronts that share a block of 64 neighbouring rows each take a piece of the axis and
    merge their lists: one, four and eight of them give what the oracle gives, for every list
    length, with ties (lower index first) inside a piece and across pieces."""
    cols = 16384 + 70
    for dtype, spread in ((np.float32, 3), (np.int64, 2), (np.int16, 40), (np.float64, 1000)):
        x = np.round(normal(240 + n, n * cols) * spread).astype(dtype).reshape(n, cols)
        x[:, 5] = 1                                                    # one value: the first `limit` positions win
        x[n // 2:, 6] = x[: n - n // 2, 6]                             # every value twice, in different pieces
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for k in (1, 2, 3, 5, 6, 7, 8):
            for largest in (True, False):
                Yo, Io = F.top_k(Xo, k, 0, largest)
                for waves in (1, 4, 8, 0):
                    hip_backend.set_tuning("topk_cols_waves", waves)
                    try:
                        Yh, Ih = F.top_k(Xh, k, 0, largest)
                    finally:
                        hip_backend.set_tuning("topk_cols_waves", 0)
                    assert np.array_equal(Ih.numpy(), Io.numpy()), (dtype, k, largest, waves)
                    assert np.array_equal(Yh.numpy(), Yo.numpy()), (dtype, k, largest, waves)


@pytest.mark.parametrize("n", [17, 33, 63, 64])
def test_short_rows_side_by_side_with_a_long_list(hip_backend, oracle_backend, n):
    """top_k along an outer axis of at most 64 elements with a limit beyond the register lists:
    tiles of 64 neighbouring rows, one wavefront orders a row whole.  Every element type, both
    directions, tied columns, a row count that leaves the last tile ragged, a middle axis."""
    cols = 4096 + 37
    for dtype in (np.float32, np.int32, np.float64, np.int64, np.float16, np.int16):
        x = (normal(250 + n, n * cols) * 40).astype(dtype).reshape(n, cols)
        x[:, 1] = 3
        x[:, 2] = randint(251 + n, n, 0, 3).astype(dtype)
        x[:, cols - 1] = np.sort(x[:, cols - 1], kind="stable")
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for k in sorted({17, min(n, 20), n}):
            for largest in (True, False):
                Yh, Ih = F.top_k(Xh, k, 0, largest)
                Yo, Io = F.top_k(Xo, k, 0, largest)
                assert np.array_equal(Ih.numpy(), Io.numpy()), (dtype, k, largest)
                assert np.array_equal(Yh.numpy().view(np.uint8), Yo.numpy().view(np.uint8))
    a = (normal(252, 2 * n * 2100) * 9).astype(np.float32).reshape(2, n, 2100)
    a[1, n // 2, :] = -0.0
    a[1, 0, :] = 0.0
    T, O = Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(oracle_backend, a)
    Yh, Ih = F.top_k(T, 17, 1, True, index_dtype=np.int64)
    Yo, Io = F.top_k(O, 17, 1, True, index_dtype=np.int64)
    assert np.array_equal(Ih.numpy(), Io.numpy()) and np.array_equal(Yh.numpy().view(np.uint32), Yo.numpy().view(np.uint32))


def test_many_rows_side_by_side_one_wave_per_block(hip_backend, oracle_backend):
    x = (normal(240, 64 * 524291) * 5).astype(np.float32).reshape(64, 524291)
    Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
    for k, largest in ((5, True), (8, False)):
        Yh, Ih = F.top_k(Xh, k, 0, largest)
        Yo, Io = F.top_k(Xo, k, 0, largest)
        assert np.array_equal(Ih.numpy(), Io.numpy()) and np.array_equal(Yh.numpy(), Yo.numpy())


@pytest.mark.parametrize("n", [1, 5, 31, 32, 33, 64, 100, 257, 1000, 1024])
def test_many_short_rows_one_thread_per_row(hip_backend, oracle_backend, n):
    """At least 16384 contiguous rows of up to 1024 elements with a limit of at most 8: a thread
    per row behind a coalesced, LDS-transposed load.  Piece boundaries (32 elements), row counts
    that leave lanes and waves idle, every list length, ties, all element types, a row pitch
    above the row length."""
    hip_backend.set_tuning("topk_thread_rows", 2048)          # by default only rows of up to 256 (8-byte keys: 128) go this way
    try:
        _many_short_rows(hip_backend, oracle_backend, n)
    finally:
        hip_backend.set_tuning("topk_thread_rows", 256)
    if n <= 100:
        _many_short_rows(hip_backend, oracle_backend, n, dtypes=(np.float32, np.int64))


def _many_short_rows(hip_backend, oracle_backend, n, dtypes=None):
    rows = 16384 + 70 + n % 7
    dtypes = dtypes or ((np.float32, np.int32, np.float64, np.int64, np.float16, np.int16) if n <= 100 else (np.float32, np.int64))
    for dtype in dtypes:
        x = (normal(250 + n, rows * n) * 40).astype(dtype).reshape(rows, n)
        x[1] = 3                                                      # all equal
        x[2] = randint(251 + n, n, 0, 3).astype(dtype)                # three distinct values
        x[3] = np.sort(x[3], kind="stable")
        x[4] = np.sort(x[4], kind="stable")[::-1]
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for k in sorted({1, min(n, 2), min(n, 3), min(n, 5), min(n, 8)}):
            for largest in (True, False):
                Yh, Ih = F.top_k(Xh, k, -1, largest)
                Yo, Io = F.top_k(Xo, k, -1, largest)
                assert np.array_equal(Ih.numpy(), Io.numpy()), (dtype, k, largest)
                assert np.array_equal(Yh.numpy().view(np.uint8), Yo.numpy().view(np.uint8))
    if n >= 5:
        a = (normal(252, rows * n) * 9).astype(np.float32).reshape(rows, n)
        a[7, 1] = np.nan
        a[9, :] = 0.0
        a[9, n // 2] = -0.0
        T = Tensor.from_numpy(hip_backend, a).slice([0, 1], [rows, n - 1])      # pitch n, rows of n - 2
        k = min(4, n - 2)
        Yh, Ih = F.top_k(T, k, 1, True, index_dtype=np.int64)
        SV, SI = F.argsort(T, 1, True, with_values=True)
        assert Ih.numpy().dtype == np.int64 and np.array_equal(Ih.numpy(), SI.numpy()[:, :k])
        assert np.array_equal(Yh.numpy().view(np.uint32), SV.numpy()[:, :k].view(np.uint32))


@pytest.mark.parametrize("shape,axis", [((1, 200000), 1), ((3, 70001), 1), ((2, 1 << 20), 1), ((70001, 3), 0), ((2, 65537), 1),
                                        ((1, 5_000_000), 1)])
def test_rows_longer_than_the_selection_kernel_takes(hip_backend, shape, axis):
    """Rows of more than 65536 (8-byte keys: 32768) elements: selection within segments, then
    among the segments' winners (and again, when those are still too many), places turned back
    into row indices.  Ties across segment boundaries, every element type, both directions,
    64-bit indices, a strided axis, NaNs by bit pattern."""
    n = shape[axis]
    x = quantised(270 + n, shape)                               # ties everywhere, also across segments
    ks = (1, 5, 100, 1024) if n < 1_000_000 else (5, 1000)
    for k in ks:
        check(hip_backend, x, k, axis, True)
    check(hip_backend, x, 7, axis, False, np.int64)
    if n <= 200000:
        for dtype in (np.int64, np.float64, np.float16, np.int16, np.int32):
            xd = (normal(271 + n, int(np.prod(shape))) * 300).astype(dtype).reshape(shape)
            check(hip_backend, xd, 33, axis, True)
            check(hip_backend, xd, 2, axis, False)
        xn = (normal(272 + n, int(np.prod(shape))) * 3).astype(np.float32).reshape(shape)
        flat = np.moveaxis(xn, axis, -1)
        flat[0, [3, n // 2, n - 1]] = np.nan
        flat[0, 70000 if n > 70000 else 11] = np.inf
        X = Tensor.from_numpy(hip_backend, xn)
        for largest in (True, False):
            Y, I = F.top_k(X, 6, axis, largest)
            SV, SI = F.argsort(X, axis, largest, with_values=True)
            take = [slice(None)] * 2
            take[axis] = slice(0, 6)
            assert np.array_equal(I.numpy(), SI.numpy()[tuple(take)]), largest
            assert np.array_equal(Y.numpy().view(np.uint32), SV.numpy()[tuple(take)].view(np.uint32)), largest
