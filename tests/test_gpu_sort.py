"""sort / argsort: HIP path vs the CPU oracle, bit-exact.

Values must equal the restated reference merge sort; argsort indices must equal
the stable order (lowest source index first among equal keys, both directions),
which no reference test pins -- it is pinned against numpy's stable argsort in
the CPU suite -- and gather(X, I) must reproduce the sorted values.
"""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import normal, randint, full_range_i64, uniform01

pytestmark = pytest.mark.gpu


def both(hip, orc, x):
    return Tensor.from_numpy(hip, x), Tensor.from_numpy(orc, x)


def make(dtype, seed, count, dup):
    if dup:
        return randint(seed, count, -6, 6).astype(dtype)
    if np.dtype(dtype) == np.int64:
        return full_range_i64(seed, count)
    if np.dtype(dtype) == np.int32:
        return full_range_i64(seed, count).astype(np.int32)
    return (normal(seed, count) * 1e3).astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.int64, np.float64])
@pytest.mark.parametrize("n", [2, 3, 10, 100, 1000, 4095, 4096, 4097, 10000, 70001])
def test_sort_rows_sizes(hip_backend, oracle_backend, dtype, n):
    for dup in (False, True):
        x = make(dtype, 60 + n, 2 * n, dup).reshape(2, n)
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for desc in (False, True):
            g = F.sort(Xh, -1, desc).numpy()
            assert np.array_equal(g, F.sort(Xo, -1, desc).numpy()), (desc, dup)


@pytest.mark.parametrize("dtype", [np.float32, np.int64])
@pytest.mark.parametrize("axis", [0, 1, 2])
def test_sort_any_axis_and_in_place(hip_backend, oracle_backend, dtype, axis):
    x = make(dtype, 61, 6 * 50 * 40, True).reshape(6, 50, 40)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for desc in (False, True):
        assert np.array_equal(F.sort(Xh, axis, desc).numpy(), F.sort(Xo, axis, desc).numpy())
    F.sort(Xh, axis, out=Xh)
    assert np.array_equal(Xh.numpy(), np.sort(x, axis=axis))


@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.int64, np.float64])
@pytest.mark.parametrize("n", [2, 10, 257, 1000, 4096, 4097, 10000, 70001])
def test_argsort_stable_both_directions(hip_backend, oracle_backend, dtype, n):
    for dup in (True, False):
        x = make(dtype, 62 + n, 2 * n, dup).reshape(2, n)
        Xh, Xo = both(hip_backend, oracle_backend, x)
        for desc in (False, True):
            Ih = F.argsort(Xh, -1, desc).numpy()
            Io = F.argsort(Xo, -1, desc).numpy()
            assert Ih.dtype == np.int32 and np.array_equal(Ih, Io), (desc, dup)
            Yh, Ih2 = F.argsort(Xh, -1, desc, with_values=True)
            Yo, _ = F.argsort(Xo, -1, desc, with_values=True)
            assert np.array_equal(Ih2.numpy(), Io)
            assert np.array_equal(Yh.numpy(), Yo.numpy())
            assert np.array_equal(F.gather_elements(x, Ih, -1), Yo.numpy())


@pytest.mark.parametrize("axis", [0, 1, 2])
def test_argsort_axes_int64_indices_and_in_place_values(hip_backend, oracle_backend, axis):
    x = make(np.int32, 63, 5 * 30 * 20, True).reshape(5, 30, 20)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    I64 = F.argsort(Xh, axis, index_dtype=np.int64).numpy()
    assert I64.dtype == np.int64 and np.array_equal(I64, F.argsort(Xo, axis).numpy())
    # values written over the input (UniformTest.cpp:2419: argsort(Y, Y, I, axis))
    Yh, Ih = F.argsort(Xh, axis, values=Xh)
    assert np.array_equal(Yh.numpy(), np.sort(x, axis=axis))
    assert np.array_equal(F.gather_elements(x, Ih.numpy(), axis), np.sort(x, axis=axis))


def test_argsort_signed_zeros_are_one_key(hip_backend):
    x = np.array([[0.0, -0.0, 1.0, -0.0, 0.0, -1.0, -0.0]], dtype=np.float32)
    X = Tensor.from_numpy(hip_backend, x)
    Y, I = F.argsort(X, -1, with_values=True)
    assert I.numpy().tolist() == [[5, 0, 1, 3, 4, 6, 2]]
    assert np.array_equal(np.signbit(Y.numpy()), np.signbit(x[0][I.numpy()[0]])[None, :])
    Y, I = F.argsort(X, -1, True, with_values=True)
    assert I.numpy().tolist() == [[2, 0, 1, 3, 4, 6, 5]]


def test_extent_one_axis_copies(hip_backend):
    x = make(np.float32, 64, 7, False).reshape(7, 1)
    X = Tensor.from_numpy(hip_backend, x)
    assert np.array_equal(F.sort(X, 1).numpy(), x)
    Y, I = F.argsort(X, 1, with_values=True)
    assert np.array_equal(Y.numpy(), x) and not I.numpy().any()


def test_quantised_heavy_duplicates_and_full_range(hip_backend, oracle_backend):
    # the two benchmark input families at reduced size
    x = (np.floor(uniform01(65, 8 * 65536) * 4096) / 4096).astype(np.float32).reshape(8, 65536)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for desc in (False, True):
        assert np.array_equal(F.sort(Xh, -1, desc).numpy(), F.sort(Xo, -1, desc).numpy())
        assert np.array_equal(F.argsort(Xh, -1, desc).numpy(), F.argsort(Xo, -1, desc).numpy())
    y = full_range_i64(66, 2 * (1 << 18)).reshape(2, 1 << 18)
    Yh, Yo = both(hip_backend, oracle_backend, y)
    for desc in (False, True):
        assert np.array_equal(F.sort(Yh, -1, desc).numpy(), F.sort(Yo, -1, desc).numpy())
        assert np.array_equal(F.argsort(Yh, -1, desc).numpy(), F.argsort(Yo, -1, desc).numpy())


def test_bounded_wait_self_help_path(hip_backend, oracle_backend):
    x = make(np.int32, 67, 3 * 50000, True).reshape(3, 50000)
    y = full_range_i64(68, 2 * 30000).reshape(2, 30000)
    hip_backend.set_tuning("sort_poll_limit", 0)
    try:
        for a in (x, y):
            Xh, Xo = both(hip_backend, oracle_backend, a)
            assert np.array_equal(F.sort(Xh, -1, True).numpy(), F.sort(Xo, -1, True).numpy())
            assert np.array_equal(F.argsort(Xh, -1).numpy(), F.argsort(Xo, -1).numpy())
    finally:
        hip_backend.set_tuning("sort_poll_limit", 2048)


def test_many_short_rows(hip_backend, oracle_backend):
    x = make(np.float32, 69, 3000 * 17, True).reshape(3000, 17)
    Xh, Xo = both(hip_backend, oracle_backend, x)
    assert np.array_equal(F.sort(Xh, -1).numpy(), F.sort(Xo, -1).numpy())
    assert np.array_equal(F.argsort(Xh, 0).numpy(), F.argsort(Xo, 0).numpy())


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
def test_rows_leave_out_passes_that_move_nothing(hip_backend, oracle_backend, dtype):
    # digits that are the same in a whole row are not sorted on; rows decide independently, so
    # neighbouring rows take different routes through the scratch buffers
    n = 10000
    small = randint(70, n, 0, 200).astype(dtype)                      # only the lowest digit varies
    medium = randint(71, n, 0, 50000).astype(dtype)                   # two digits vary
    constant = np.full(n, 7, dtype=dtype)                             # nothing varies: one pass, input -> output
    if np.dtype(dtype).kind == "i":
        wide = full_range_i64(72, n).astype(dtype)
    else:
        wide = (normal(72, n) * 1e3).astype(dtype)
    x = np.stack([small, wide, constant, medium, small[::-1].copy(), constant])
    Xh, Xo = both(hip_backend, oracle_backend, x)
    for desc in (False, True):
        assert np.array_equal(F.sort(Xh, -1, desc).numpy(), F.sort(Xo, -1, desc).numpy()), desc
        Yh, Ih = F.argsort(Xh, -1, desc, with_values=True)
        Yo, Io = F.argsort(Xo, -1, desc, with_values=True)
        assert np.array_equal(Ih.numpy(), Io.numpy()), desc
        assert np.array_equal(Yh.numpy(), Yo.numpy()), desc
    # written over the input: every pass runs, none may read the input while it is overwritten
    F.sort(Xh, -1, out=Xh)
    assert np.array_equal(Xh.numpy(), np.sort(x, axis=-1))
    Xh = Tensor.from_numpy(hip_backend, x)
    Yh, Ih = F.argsort(Xh, -1, values=Xh)
    assert np.array_equal(Yh.numpy(), np.sort(x, axis=-1))
    assert np.array_equal(Ih.numpy(), np.argsort(x, axis=-1, kind="stable"))


@pytest.mark.parametrize("dtype", [np.int64, np.float32, np.int32, np.float64])
@pytest.mark.parametrize("n", [5000, 9000, 17000, 40000, 150000, 300000, 600000, 1 << 20])
def test_long_rows_cut_into_buckets(hip_backend, dtype, n):
    """Rows longer than one workgroup sorts are cut into buckets of equal depth by value and
    each bucket is finished on chip.  Checked against numpy's stable sort and against the
    least-significant-digit-first passes (the same call with the bucket route switched off)."""
    if np.dtype(dtype).kind == "i":
        wide = full_range_i64(300, n).astype(dtype)                   # even leading digit
        lopsided = (full_range_i64(301, n) >> 40).astype(dtype)       # (int64) three digits vary, the top one in two values
        narrow = randint(302, n, 0, 60000).astype(dtype)              # two low digits vary: leading digit of those spreads evenly
    else:
        wide = np.ldexp(uniform01(300, n) + 1.0, randint(303, n, -100, 100).astype(np.int32)).astype(dtype) * np.where(randint(304, n, 0, 2) > 0, 1, -1).astype(dtype)
        lopsided = (normal(301, n) * 1e3).astype(dtype)               # the sign and exponent byte takes few values
        narrow = (1.0 + randint(302, n, 0, 60000) / 65536.0).astype(dtype)
    ties = wide.copy()
    ties[1::2] = ties[0::2][: ties[1::2].size]                        # every key twice: the order of equals shows
    one_digit = randint(305, n, 0, 200).astype(dtype)
    # every key beside one that differs from it in its low 20 bits only: the leading digits of a
    # run do not settle the order
    close = wide.copy()
    bits = close.view(np.uint64 if close.itemsize == 8 else np.uint32)
    bits[1::2] = bits[0::2][: bits[1::2].size] ^ randint(306, bits[1::2].size, 0, 1 << 20).astype(bits.dtype)
    # the same for one key in 64 (a few per run, which move within the run without the lower
    # digits being sorted), and groups of 4 and of 6 such keys
    few = wide.copy()
    bits = few.view(np.uint64 if few.itemsize == 8 else np.uint32)
    for group, step in ((2, 64), (4, 1000), (6, 1777)):
        for j in range(1, group):
            at = np.arange(0, n - group, step) + j
            bits[at] = bits[at - j] ^ randint(307 + j, at.size, 0, 1 << 20).astype(bits.dtype)
    # rows whose order is not random: sorted, a sawtooth of sorted runs, and one value with a few
    # strays at both ends (the sample reads evenly spaced places; the strays must not stretch
    # the range the buckets divide)
    in_order = np.sort(wide)
    sawtooth = np.sort(narrow.reshape(-1, 250) if n % 250 == 0 else narrow[: n // 250 * 250].reshape(-1, 250), axis=1).reshape(-1)
    sawtooth = np.concatenate([sawtooth, narrow[sawtooth.size:]])
    strays = np.full(n, narrow[0])
    strays[[1, n // 3, n - 2]] = [wide.min(), wide.max(), wide.min()]
    strays[n // 2: n // 2 + 300] = narrow[:300]
    x = np.stack([wide, lopsided, ties, one_digit, narrow, wide[::-1].copy(), close, few, in_order, sawtooth, strays])
    Xh = Tensor.from_numpy(hip_backend, x)
    want = np.sort(x, axis=-1, kind="stable")
    order = np.argsort(x, axis=-1, kind="stable")
    assert np.array_equal(F.sort(Xh, -1).numpy().view(np.uint8), want.view(np.uint8))
    Yh, Ih = F.argsort(Xh, -1, False, with_values=True, index_dtype=np.int64)
    assert np.array_equal(Ih.numpy(), order) and np.array_equal(Yh.numpy().view(np.uint8), want.view(np.uint8))
    got = {}
    for route in (1, 0):
        hip_backend.set_tuning("sort_buckets", route)
        try:
            Yd, Id = F.argsort(Xh, -1, True, with_values=True)
            got[route] = (F.sort(Xh, -1, True).numpy(), Yd.numpy(), Id.numpy(), F.argsort(Xh, -1).numpy())
        finally:
            hip_backend.set_tuning("sort_buckets", 1)
    for a, b in zip(got[1], got[0]):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    assert np.array_equal(got[1][0].view(np.uint8), np.ascontiguousarray(want[:, ::-1]).view(np.uint8))
    assert np.array_equal(np.take_along_axis(x, got[1][2].astype(np.int64), -1).view(np.uint8), got[1][1].view(np.uint8))
    assert np.array_equal(got[1][3], order)
    # strided outputs (a transposed destination) and an input view with a step
    Zh = Tensor.from_numpy(hip_backend, np.zeros((n // 2, x.shape[0]), dtype=dtype)).transpose([1, 0])
    F.sort(Xh.slice([0], [n], [1], [2]).flip([1]), -1, out=Zh)
    assert np.array_equal(np.ascontiguousarray(Zh.numpy()).view(np.uint8), np.sort(x[:, 0:n:2], axis=-1).view(np.uint8))


@pytest.mark.parametrize("dtype", [np.int64, np.float64, np.int32, np.float32])
@pytest.mark.parametrize("n", [9000, 17000, 40000, 300000])
def test_buckets_ranked_by_comparison_or_by_digit_passes(hip_backend, dtype, n):
    """A bucket whose counting bins are crowded (many equal or clustered keys) is finished by the
    stable digit passes - for argsort first by index, then by key - instead of by comparing the
    entries of a bin.  Forcing that for every bucket ("sort_compare_max" 0), and allowing bins of
    any size to be compared (4096), gives the same values and indices, and both match numpy."""
    spread = full_range_i64(320, 3 * n).reshape(3, n)
    spread[1, 1::2] = spread[1, 0::2][: spread[1, 1::2].size]                   # every key twice
    spread[2] = np.repeat(spread[2, : (n + 99) // 100], 100)[:n]                # runs of 100 equal keys
    clustered = (full_range_i64(321, 2 * n).reshape(2, n) >> 40)
    clustered[1] = clustered[1] // 1000 * 1000                                  # few distinct values
    raw = np.concatenate([spread, clustered])
    if np.dtype(dtype).itemsize == 4:
        raw = (raw >> 32).astype(np.int32)
    if np.dtype(dtype).kind == "f":
        x = raw.view(dtype).copy()
        x[np.isnan(x)] = 0.0
    else:
        x = raw.astype(dtype)
    Xh = Tensor.from_numpy(hip_backend, x)
    order = np.argsort(x, axis=-1, kind="stable")
    want = np.take_along_axis(x, order, -1)
    for limit in (0, 32, 96, 4096):
        hip_backend.set_tuning("sort_compare_max", limit)
        try:
            Yh, Ih = F.argsort(Xh, -1, False, with_values=True)
            Id = F.argsort(Xh, -1, True).numpy().astype(np.int64)
            Sh = F.sort(Xh, -1).numpy()
        finally:
            hip_backend.set_tuning("sort_compare_max", 32)
        assert np.array_equal(Ih.numpy(), order) and np.array_equal(Yh.numpy().view(np.uint8), want.view(np.uint8)), limit
        assert np.array_equal(np.sort(x, axis=-1).view(np.uint8), Sh.view(np.uint8)), limit
        got = np.take_along_axis(x, Id, -1)
        assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(want[:, ::-1]).view(np.uint8)), limit
        same = got[:, 1:] == got[:, :-1]
        assert np.all(Id[:, 1:][same] > Id[:, :-1][same]), limit


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [70000, 1 << 20])
def test_float_rows_spread_by_value_or_by_image(hip_backend, dtype, n):
    """Float rows choose how their range is spread over the fine bins: evenly over the values
    (bell-shaped data on both sides of zero, uniform data) or over the key images (magnitudes over
    many binades).  Either way the order is exact, with infinities, NaNs and zeros of both signs
    in the row, ascending and descending."""
    bell = normal(350, 2 * n).astype(dtype).reshape(2, n)
    bell[1] = bell[1] * dtype(1e-3) + dtype(5.0)                       # a narrow bell far from zero
    decades = np.exp(normal(351, n).astype(np.float64) * 12.0).astype(dtype).reshape(1, n)      # magnitudes over many binades
    decades[0, ::2] *= dtype(-1.0)
    mixed = normal(352, n).astype(dtype).reshape(1, n)
    mixed[0, 5:2000:7] = np.inf
    mixed[0, 6:2000:7] = -np.inf
    mixed[0, 7:3000:11] = np.nan
    mixed[0, 100:200] = 0.0
    mixed[0, 150:250:2] = -0.0
    flat = np.full((1, n), dtype(2.5))
    flat[0, n // 2] = dtype(-1.0)
    x = np.concatenate([bell, decades, mixed, flat])
    Xh = Tensor.from_numpy(hip_backend, x)
    want = np.sort(x, axis=-1)
    got = F.sort(Xh, -1).numpy()
    assert np.array_equal(got, want, equal_nan=True)
    assert np.array_equal(F.sort(Xh, -1, True).numpy(), want[:, ::-1], equal_nan=True)
    plain = [0, 1, 2, 4]                                                # rows without NaNs: the stable order is numpy's
    order = np.argsort(x[plain], axis=-1, kind="stable")
    Ih = F.argsort(Tensor.from_numpy(hip_backend, x[plain]), -1, False)
    assert np.array_equal(Ih.numpy(), order)
    Yh, Jh = F.argsort(Xh, -1, True, with_values=True)
    assert np.array_equal(np.take_along_axis(x, Jh.numpy().astype(np.int64), -1).view(np.uint8), Yh.numpy().view(np.uint8))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [30720, 31000, 65536, 131072])
def test_float_rows_either_side_of_zero_close_the_gap_between_their_images(hip_backend, dtype, n):
    """Float rows of 30 720 to 131 072 elements with values on both sides of zero leave the images
    between their smallest negative and positive magnitudes out of the fine bins.  Rows where that
    applies (bell-shaped, with a few zeros, with one stray tiny value a side), rows where it does
    not (half zeros, tiny values all over, one sign only, magnitudes over many binades) and rows
    with infinities and NaNs, ascending and descending, against numpy."""
    rows = normal(360, 8 * n).astype(dtype).reshape(8, n)
    rows[1, ::97] = 0.0
    rows[1, 5::97] = -0.0
    rows[2, 17] = dtype(1e-30)
    rows[2, 4711] = dtype(-1e-30)
    rows[3, rows[3] < 0] = 0.0                                            # half the row zeros
    rows[4, ::3] *= dtype(1e-20)                                          # a third of the row tiny, both signs
    rows[5] = np.abs(rows[5]) + dtype(0.25)                               # one sign only
    rows[6] = (np.exp(normal(361, n).astype(np.float64) * 10.0) * np.sign(rows[6])).astype(dtype)
    rows[7, 5:2000:7] = np.inf
    rows[7, 6:2000:7] = -np.inf
    rows[7, 7:3000:11] = np.nan
    rows[7, 8:3000:11] = -np.nan
    Xh = Tensor.from_numpy(hip_backend, rows)
    want = np.sort(rows, axis=-1)
    got = F.sort(Xh, -1).numpy()
    assert np.array_equal(got[:7], want[:7])
    nans = np.isnan(got[7])                                               # negative NaNs first, positive ones last; numpy: all last
    assert nans.sum() == np.isnan(rows[7]).sum()
    assert np.array_equal(got[7][~nans], want[7][: (~nans).sum()])
    assert np.array_equal(F.sort(Tensor.from_numpy(hip_backend, rows[:7]), -1, True).numpy(), want[:7, ::-1])
    order = np.argsort(rows[:7], axis=-1, kind="stable")
    Yh, Ih = F.argsort(Tensor.from_numpy(hip_backend, rows[:7]), -1, False, with_values=True)
    assert np.array_equal(Ih.numpy(), order)
    assert np.array_equal(Yh.numpy().view(np.uint8), np.take_along_axis(rows[:7], order, -1).view(np.uint8))
    Yd, Jd = F.argsort(Xh, -1, True, with_values=True)
    assert np.array_equal(np.take_along_axis(rows, Jd.numpy().astype(np.int64), -1).view(np.uint8), Yd.numpy().view(np.uint8))
    d = Yd.numpy()[:7]
    assert bool((d[:, 1:] <= d[:, :-1]).all())


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.int64])
def test_buckets_of_narrow_and_of_wide_keys_in_turn(hip_backend, dtype):
    """A bucket whose keys differ in fewer bits than the finishing workgroup has counting bins uses
    (scans, clears) only the first of them; buckets of full-width keys use all.  Rows that mix
    the two kinds - so that one workgroup meets them in turn - and rows of every width from one
    bit up, keys only and with indices, against numpy."""
    n = 60000
    widths = [1, 3, 5, 8, 11, 12, 13, 20]
    rows = np.stack([randint(370 + w, n, 0, 1 << w) for w in widths]).astype(np.int64)
    wide = full_range_i64(371, 3 * n).reshape(3, n) >> (33 if np.dtype(dtype).itemsize == 4 else 1)
    mixed = wide.copy()
    mixed[0, ::2] = randint(372, n // 2, 0, 50)                          # every other key one of 50 values
    mixed[1, : n // 2] = randint(373, n // 2, 1000, 1004)                # half the row four values, the rest wide
    mixed[2, n // 3:] = (mixed[2, n // 3:] >> 12) << 12                  # low bits all zero in two thirds
    raw = np.concatenate([rows, mixed, wide[:1]])
    x = raw.astype(dtype)
    Xh = Tensor.from_numpy(hip_backend, x)
    want = np.sort(x, axis=-1)
    for _ in range(2):                                                    # a second call over the same scratch
        assert np.array_equal(F.sort(Xh, -1).numpy(), want)
        assert np.array_equal(F.sort(Xh, -1, True).numpy(), want[:, ::-1])
    order = np.argsort(x, axis=-1, kind="stable")
    Yh, Ih = F.argsort(Xh, -1, False, with_values=True)
    assert np.array_equal(Ih.numpy(), order)
    assert np.array_equal(Yh.numpy(), want)


@pytest.mark.parametrize("dtype", [np.int64, np.float32])
def test_rows_beyond_a_million_keys_take_the_largest_buckets(hip_backend, dtype):
    """Rows longer than 1.1 M keys are cut into buckets of up to 10240 keys, finished by workgroups
    of sixteen wavefronts (up to 2 359 296 keys a row; longer rows keep the digit passes)."""
    for n in (1_500_000, 2_359_296, 2_359_297, 2_700_001):
        raw = full_range_i64(340 + n % 7, 2 * n).reshape(2, n)
        x = raw.astype(dtype) if np.dtype(dtype).kind == "i" else (raw >> 40).astype(np.float32) / np.float32(64.0)
        Xh = Tensor.from_numpy(hip_backend, x)
        order = np.argsort(x, axis=-1, kind="stable")
        Yh, Ih = F.argsort(Xh, -1, False, with_values=True)
        assert np.array_equal(Ih.numpy(), order)
        assert np.array_equal(Yh.numpy(), np.take_along_axis(x, order, -1))
        assert np.array_equal(F.sort(Xh, -1, True).numpy(), np.sort(x, axis=-1)[:, ::-1])


@pytest.mark.parametrize("dtype", [np.int64, np.float32, np.float64])
@pytest.mark.parametrize("n", [1_800_000, 2_100_000, 2_350_000])
def test_long_rows_whose_bins_are_packed_bucket_by_bucket(hip_backend, dtype, n):
    """Near the longest rows the route takes, buckets of (capacity - largest fine bin) are more
    than 256: the fine bins are packed into buckets one after the other instead.  Evenly spread
    keys, bell-shaped and sharply peaked values (whose largest bin is several times the mean)."""
    if np.dtype(dtype).kind == "i":
        kinds = [full_range_i64(400, n), full_range_i64(401, n) >> 20, (normal(402, n) * 1e15).astype(np.int64)]
    else:
        g = normal(403, n)
        kinds = [g, np.sign(g) * g * g, uniform01(404, n) * 1000.0]
    x = np.stack(kinds).astype(dtype)
    Xh = Tensor.from_numpy(hip_backend, x)
    want = np.sort(x, axis=-1, kind="stable")
    assert np.array_equal(F.sort(Xh, -1).numpy(), want)
    order = np.argsort(x, axis=-1, kind="stable")
    Yh, Ih = F.argsort(Xh, -1, False, with_values=True)
    assert np.array_equal(Ih.numpy(), order)
    assert np.array_equal(Yh.numpy().view(np.uint8), want.view(np.uint8))
    assert np.array_equal(F.argsort(Xh, -1, True).numpy(), np.argsort(-x if np.dtype(dtype).kind == "f" else ~x, axis=-1, kind="stable"))


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_rows_with_oversized_buckets_beside_rows_that_cut_evenly(hip_backend, dtype):
    """Rows that do not cut into buckets a workgroup holds (one value repeated, a handful of
    values: a fine bin fuller than a bucket) get buckets of their own size, finished by one
    workgroup each, in the same call that sorts its other rows the usual way; several calls in
    a row over one scratch buffer."""
    n = 70000
    x = (full_range_i64(330, 9 * n).reshape(9, n) >> (40 if np.dtype(dtype).itemsize == 8 else 36)).astype(dtype)
    x[1, :] = 7                                   # one value
    x[4, :] = x[4, :] % 5                         # five values
    x[6, : n // 2] = -3                           # half the row one value
    Xh = Tensor.from_numpy(hip_backend, x)
    order = np.argsort(x, axis=-1, kind="stable")
    for _ in range(2):
        Yh, Ih = F.argsort(Xh, -1, False, with_values=True)
        Sh = F.sort(Xh, -1, True)
        assert np.array_equal(Ih.numpy(), order)
        assert np.array_equal(Yh.numpy(), np.take_along_axis(x, order, -1))
        assert np.array_equal(Sh.numpy(), np.sort(x, axis=-1)[:, ::-1])


def oversized_rows(dtype, n, seed):
    """Rows whose keys defeat cutting by value: repeated values, and distinct values packed more
    tightly than the fine bins of the row's range resolve."""
    dt = np.dtype(dtype)
    if dt.kind == "i":
        wide = full_range_i64(seed, n).astype(dtype)
        cluster = wide.copy()                                         # nine keys in ten within 1000 of one another
        near = randint(seed + 1, n, 0, 1000).astype(dtype) + dtype(12345)
        pick = randint(seed + 2, n, 0, 10) > 0
        cluster[pick] = near[pick]
        pair = (randint(seed + 3, n, 0, 2) + 40).astype(dtype)        # two neighbouring values
        pair[:: 97] = wide[:: 97]
    else:
        wide = (normal(seed, n) * 1e3).astype(dtype)
        cluster = wide.copy()
        eps = np.finfo(dtype).eps
        near = (dtype(3.25) * (1 + randint(seed + 1, n, 0, 1000).astype(dtype) * eps)).astype(dtype)
        pick = randint(seed + 2, n, 0, 10) > 0
        cluster[pick] = near[pick]
        pair = np.where(randint(seed + 3, n, 0, 2) > 0, dtype(0.0), dtype(-0.0)).astype(dtype)       # the two zeros: one key for a stable argsort
        pair[:: 97] = wide[:: 97]
    constant = np.full(n, wide[0], dtype=dtype)
    few = wide[randint(seed + 4, n, 0, 5)]                            # five values
    many = np.sort(wide[:300])[randint(seed + 5, n, 0, 300)]          # 300 values: more heavy bins than buckets
    half = wide.copy()
    half[randint(seed + 6, n, 0, 2) > 0] = wide[1]
    return np.stack([constant, cluster, few, wide, pair, many, half])


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
@pytest.mark.parametrize("n", [20000, 70000, 300000, 1 << 20])
def test_buckets_larger_than_a_workgroup_holds(hip_backend, dtype, n):
    x = oversized_rows(dtype, n, 340)
    Xh = Tensor.from_numpy(hip_backend, x)
    want = np.sort(x, axis=-1, kind="stable")
    for desc in (False, True):
        key = -x if (desc and np.dtype(dtype).kind == "f") else x
        order = np.argsort(key, axis=-1, kind="stable") if not desc or np.dtype(dtype).kind == "f" else np.argsort(~x, axis=-1, kind="stable")
        got = F.sort(Xh, -1, desc).numpy()
        ref = want[:, ::-1] if desc else want
        assert np.array_equal(got, ref), desc                              # (== : the two zeros are one value)
        Ih = F.argsort(Xh, -1, desc)                                       # indices alone: keys of the far side come from the input
        assert np.array_equal(Ih.numpy(), order), desc
        Yh, I64 = F.argsort(Xh, -1, desc, with_values=True, index_dtype=np.int64)
        assert np.array_equal(I64.numpy(), order), desc
        assert np.array_equal(Yh.numpy().view(np.uint8), np.take_along_axis(x, order, -1).view(np.uint8)), desc
    # in place, and onto a transposed destination
    Zh = Tensor.from_numpy(hip_backend, x)
    F.sort(Zh, -1, out=Zh)
    assert np.array_equal(Zh.numpy(), want)
    xp = x + dtype(0) if np.dtype(dtype).kind == "f" else x               # (-0.0 + 0.0 = +0.0: written over the input, the two zeros order by sign)
    Zh = Tensor.from_numpy(hip_backend, xp)
    Yh, Ih = F.argsort(Zh, -1, values=Zh)
    assert np.array_equal(Ih.numpy(), np.argsort(xp, axis=-1, kind="stable"))
    assert np.array_equal(Yh.numpy(), want)
    Th = Tensor.from_numpy(hip_backend, np.zeros((n, x.shape[0]), dtype=dtype)).transpose([1, 0])
    F.sort(Xh, -1, out=Th)
    assert np.array_equal(np.ascontiguousarray(Th.numpy()), want)


@pytest.mark.parametrize("dtype", [np.float32, np.int32])
@pytest.mark.parametrize("n", [17000, 40000, 70000, 131072])
def test_many_rows_each_planned_and_moved_by_one_workgroup(hip_backend, dtype, n):
    # calls of at least 512 rows of 4-byte keys of up to 131072 elements: one workgroup takes a
    # row from its sample to its scatter; rows that cut evenly beside rows with oversized buckets
    m = 530
    kinds = oversized_rows(dtype, n, 360)                               # 7 kinds of awkward rows
    if np.dtype(dtype).kind == "f":
        wide = (normal(361, m * n) * 3).astype(dtype).reshape(m, n)
        wide[::3] = np.floor(uniform01(362, ((m + 2) // 3) * n) * 4096).astype(dtype).reshape(-1, n) / dtype(4096)      # the benchmark's quantised rows
    else:
        wide = (full_range_i64(361, m * n) >> 33).astype(dtype).reshape(m, n)
    x = wide
    x[5::40] = kinds[np.arange(x[5::40].shape[0]) % kinds.shape[0]]
    Xh = Tensor.from_numpy(hip_backend, x)
    want = np.sort(x, axis=-1, kind="stable")
    assert np.array_equal(F.sort(Xh, -1).numpy(), want)
    order = np.argsort(x, axis=-1, kind="stable")
    assert np.array_equal(F.argsort(Xh, -1).numpy(), order)
    Yh, Ih = F.argsort(Xh, -1, True, with_values=True)
    rev = np.argsort(-x if np.dtype(dtype).kind == "f" else ~x, axis=-1, kind="stable")
    assert np.array_equal(Ih.numpy(), rev)
    assert np.array_equal(Yh.numpy().view(np.uint8), np.take_along_axis(x, rev, -1).view(np.uint8))
    F.sort(Xh, -1, True, out=Xh)                                        # in place
    assert np.array_equal(Xh.numpy(), want[:, ::-1])


def clustered_rows(dtype, n, seed):
    """Rows whose distinct keys crowd parts of their range: the evenly spaced fine bins of the
    bucket route cannot cut them, a map made from the quantiles of a sample can."""
    dt = np.dtype(dtype)
    u = uniform01(seed, n)
    g = normal(seed + 1, n)
    if dt.kind == "i":
        top = float(np.iinfo(dtype).max)
        zipf = np.minimum(np.floor(1.0 / np.maximum(u, 1e-12) ** 1.3), top / 2).astype(dtype)      # most keys small, a long tail
        two = np.where(randint(seed + 2, n, 0, 2) > 0, 1000 + randint(seed + 3, n, 0, 5000), int(top / 3) + randint(seed + 4, n, 0, 5000)).astype(dtype)
        tail = np.where(randint(seed + 5, n, 0, 20) > 0, randint(seed + 6, n, -3000, 3000), (g * top / 8).astype(np.int64)).astype(dtype)
        steps = (np.floor(u * 64).astype(np.int64) * int(top / 80) + randint(seed + 7, n, 0, 300)).astype(dtype)     # 64 narrow clusters
    else:
        zipf = np.exp(g * 6).astype(dtype)                                                # log-normal: twenty binades
        two = np.where(randint(seed + 2, n, 0, 2) > 0, 1.0 + g * 1e-5, -250.0 + g * 1e-4).astype(dtype)
        tail = np.where(randint(seed + 5, n, 0, 20) > 0, g * 1e-3, g * 1e6).astype(dtype)
        steps = (np.floor(u * 64) * 1000 + g * 1e-2).astype(dtype)
    return np.stack([zipf, two, tail, steps, np.sort(zipf), np.sort(two)[::-1]])


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
@pytest.mark.parametrize("n", [30000, 131072, 1 << 20, 2300000])
def test_rows_whose_keys_cluster(hip_backend, dtype, n):
    x = clustered_rows(dtype, n, 370)
    Xh = Tensor.from_numpy(hip_backend, x)
    want = np.sort(x, axis=-1, kind="stable")
    assert np.array_equal(F.sort(Xh, -1).numpy(), want)
    order = np.argsort(x, axis=-1, kind="stable")
    assert np.array_equal(F.argsort(Xh, -1).numpy(), order)
    Yh, Ih = F.argsort(Xh, -1, True, with_values=True)
    rev = np.argsort(-x if np.dtype(dtype).kind == "f" else ~x, axis=-1, kind="stable")
    assert np.array_equal(Ih.numpy(), rev)
    assert np.array_equal(Yh.numpy().view(np.uint8), np.take_along_axis(x, rev, -1).view(np.uint8))
    one = Tensor.from_numpy(hip_backend, x[2:3])                         # a single row: every workgroup on it
    assert np.array_equal(F.sort(one, -1).numpy(), want[2:3])
    F.sort(Xh, -1, out=Xh)                                              # in place: nothing goes straight to the outputs
    assert np.array_equal(Xh.numpy(), want)


@pytest.mark.parametrize("dtype", [np.int32, np.float32])
def test_many_rows_whose_keys_cluster(hip_backend, dtype):
    # the calls of many short rows (one workgroup plans and moves a row): clustered rows among plain ones
    m, n = 600, 40000
    kinds = clustered_rows(dtype, n, 380)
    if np.dtype(dtype).kind == "f":
        x = normal(381, m * n).astype(dtype).reshape(m, n)
    else:
        x = (full_range_i64(381, m * n) >> 34).astype(dtype).reshape(m, n)
    x[3::7] = kinds[np.arange(x[3::7].shape[0]) % kinds.shape[0]]
    Xh = Tensor.from_numpy(hip_backend, x)
    assert np.array_equal(F.sort(Xh, -1).numpy(), np.sort(x, axis=-1))
    order = np.argsort(x, axis=-1, kind="stable")
    Yh, Ih = F.argsort(Xh, -1, with_values=True)
    assert np.array_equal(Ih.numpy(), order)
    assert np.array_equal(Yh.numpy().view(np.uint8), np.take_along_axis(x, order, -1).view(np.uint8))


@pytest.mark.parametrize("dtype", [np.int32, np.float64])
def test_repeated_and_clustered_keys_on_strided_views(hip_backend, dtype):
    # the rows of the two tests above read through a view with a step, backwards, and written to
    # transposed outputs: the stable pass writes oversized buckets straight to such outputs, and an
    # index-only argsort reads its keys back from such an input
    n = 80000
    x2 = np.concatenate([oversized_rows(dtype, 2 * n, 390), clustered_rows(dtype, 2 * n, 391)])
    m = x2.shape[0]
    view = x2[:, ::2][:, ::-1]
    Xh = Tensor.from_numpy(hip_backend, x2).slice([0], [2 * n], [1], [2]).flip([1])
    assert np.array_equal(Xh.numpy().view(np.uint8), np.ascontiguousarray(view).view(np.uint8))
    from dlf_amd.frontend import dtype_code

    def argsort_into(desc, Y, I):                       # the boundary call, with outputs that are views
        hip_backend.argsort(int(desc), dtype_code(Xh.dtype), dtype_code(I.dtype), Xh.shape, Xh.storage,
                            Y.shape if Y is not None else None, Y.storage if Y is not None else None, I.shape, I.storage)

    for desc in (False, True):
        key = view if not desc else (-view if np.dtype(dtype).kind == "f" else ~view)
        order = np.argsort(key, axis=-1, kind="stable")
        Ih = Tensor.from_numpy(hip_backend, np.zeros((n, m), dtype=np.int64)).transpose([1, 0])
        argsort_into(desc, None, Ih)
        assert np.array_equal(np.ascontiguousarray(Ih.numpy()), order), desc
        Yh = Tensor.from_numpy(hip_backend, np.zeros((n, m), dtype=dtype)).transpose([1, 0])
        I32 = Tensor.from_numpy(hip_backend, np.zeros((n, m), dtype=np.int32)).transpose([1, 0])
        argsort_into(desc, Yh, I32)
        assert np.array_equal(np.ascontiguousarray(I32.numpy()), order), desc
        assert np.array_equal(np.ascontiguousarray(Yh.numpy()).view(np.uint8), np.ascontiguousarray(np.take_along_axis(view, order, -1)).view(np.uint8)), desc
        Zh = Tensor.from_numpy(hip_backend, np.zeros((n, m), dtype=dtype)).transpose([1, 0])
        F.sort(Xh, -1, desc, out=Zh)
        want = np.sort(view, axis=-1)
        assert np.array_equal(np.ascontiguousarray(Zh.numpy()), want[:, ::-1] if desc else want), desc


@pytest.mark.parametrize("n", [70000, 300000])
def test_index_only_argsort_written_over_its_input(hip_backend, n):
    # argsort(X, X) of int32 (UniformTest.cpp:2461-2466 does this with short rows): there is no value
    # output and the input is gone once indices are written, so an oversized bucket of several
    # values is sorted where it lies
    from dlf_amd.frontend import dtype_code
    x = oversized_rows(np.int32, n, 350)
    Xh = Tensor.from_numpy(hip_backend, x)
    hip_backend.argsort(0, dtype_code(np.int32), dtype_code(np.int32), Xh.shape, Xh.storage, None, None, Xh.shape, Xh.storage)
    assert np.array_equal(Xh.numpy(), np.argsort(x, axis=-1, kind="stable"))


@pytest.mark.parametrize("dtype", [np.int64, np.float64])
@pytest.mark.parametrize("n", [100, 700, 2048, 4096, 5000, 6144, 8192])
def test_wide_keys_in_short_rows_settle_on_their_leading_digits_or_run_every_digit(hip_backend, dtype, n):
    """Rows sorted whole on chip order 8-byte keys by as many leading digits as their count needs
    and run the lower digits only when two neighbours still agree.  Rows where they never do,
    rows where every key has a neighbour differing in low bits only, exact duplicates, and keys
    that differ in the lowest digit alone, against numpy's stable sort."""
    m = 24
    spread = full_range_i64(310, m * n).reshape(m, n)
    near = spread.copy()
    near[:, 1::2] = near[:, 0::2][:, : near[:, 1::2].shape[1]] ^ randint(311, m * (n // 2), 0, 1 << 24).reshape(m, n // 2)
    twice = spread.copy()
    twice[:, 1::2] = twice[:, 0::2][:, : twice[:, 1::2].shape[1]]
    low = (spread & ~np.int64(0xff)) [:, :1] | randint(312, m * n, 0, 256).reshape(m, n)
    # a few groups of 2 to 4 keys that differ in their low 16 bits (they find their places among
    # themselves), and the same with groups of 6 (too long for that: every digit runs)
    some, long_runs = spread.copy(), spread.copy()
    for rows, sizes in ((some, (2, 3, 4)), (long_runs, (2, 6))):
        for g, group in enumerate(sizes):
            for j in range(1, group):
                at = np.arange(7 * g, n - group, 97) + j
                rows[:, at] = rows[:, at - j] ^ randint(313 + j, m * at.size, 0, 1 << 16).reshape(m, at.size)
    raw = np.concatenate([spread, near, twice, low, some, long_runs])
    if np.dtype(dtype).kind == "f":
        x = raw.view(np.float64).copy()
        x[np.isnan(x)] = 0.0
    else:
        x = raw
    Xh = Tensor.from_numpy(hip_backend, x)
    for descending in (False, True):
        want = np.sort(x, axis=-1, kind="stable")
        order = np.argsort(x, axis=-1, kind="stable")
        if descending:
            want = np.ascontiguousarray(want[:, ::-1])
        assert np.array_equal(F.sort(Xh, -1, descending).numpy().view(np.uint8), want.view(np.uint8))
        Yh, Ih = F.argsort(Xh, -1, descending, with_values=True)
        assert np.array_equal(Yh.numpy().view(np.uint8), want.view(np.uint8))
        got = Ih.numpy().astype(np.int64)
        assert np.array_equal(np.take_along_axis(x, got, -1).view(np.uint8), want.view(np.uint8))
        # equal keys keep their source order in both directions
        same = np.take_along_axis(x, got, -1)[:, 1:] == np.take_along_axis(x, got, -1)[:, :-1]
        assert np.all(got[:, 1:][same] > got[:, :-1][same])
        if not descending:
            assert np.array_equal(got, order)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_nans_take_the_place_of_their_bit_pattern(hip_backend, dtype):
    """The reference's comparisons do not order NaNs (std::sort on them is undefined).  The radix
    key places them by bit pattern: negative NaNs first, positive NaNs last, ascending."""
    bits = {np.float32: np.uint32, np.float64: np.uint64, np.float16: np.uint16}[dtype]
    pos = np.array([np.nan], dtype=dtype)
    neg = (pos.view(bits) | (bits(1) << bits(8 * dtype().itemsize - 1))).view(dtype)
    row = np.array([1.5, pos[0], -np.inf, neg[0], np.inf, -2.0, pos[0], 0.0], dtype=dtype)
    x = np.tile(row, (3, 200))                      # rows of 1600 elements
    X = Tensor.from_numpy(hip_backend, x)
    asc = F.sort(X, -1).numpy()
    assert np.signbit(asc[:, :200]).all() and np.isnan(asc[:, :200]).all()          # negative NaNs
    assert np.isnan(asc[:, -400:]).all() and not np.signbit(asc[:, -400:]).any()    # positive NaNs
    mid = asc[:, 200:-400]
    assert not np.isnan(mid).any() and (mid[:, 1:] >= mid[:, :-1]).all()
    desc = F.sort(X, -1, True).numpy()
    assert np.array_equal(desc.view(bits), asc[:, ::-1].view(bits))
    idx = F.argsort(X, -1).numpy()
    assert np.array_equal(np.take_along_axis(x, idx, 1).view(bits), asc.view(bits))
    assert (np.diff(idx[:, :200], axis=1) > 0).all()                                # equal keys keep their order


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 63, 64, 65, 100, 127, 128, 129, 255, 256, 257, 300, 511, 512, 513, 1023, 1024, 1025, 1535, 1536, 1537, 2047, 2048, 2049, 2560, 2561, 3072, 3073, 3584, 3585,
                               4095, 4096, 4097, 5119, 5120, 5121, 6144, 6145, 8191, 8192, 8193, 10240, 10241, 12288, 12289, 14336, 14337, 16383, 16384, 16385])
def test_rows_around_the_one_workgroup_limits(hip_backend, oracle_backend, n):
    """Rows of up to 64, 128, 256 (512 for values only or 8-byte keys) elements are sorted by one
    wavefront in registers, rows of up to 4096 elements - 8192 for 8-byte keys, 16384 for 4-byte
    keys - by one workgroup on chip (512 to 16384 slots); longer rows take the tiled passes or the
    bucket route.  Every boundary, all key widths, both directions, values, indices (32- and
    64-bit) and in place."""
    for dtype in (np.float32, np.int64, np.float64, np.int16, np.float16, np.int32):
        x = (normal(200 + n, 5 * n) * 50).astype(dtype).reshape(5, n)
        x[1] = x[1, 0]                                   # a constant row: no pass runs
        x[2] = np.sort(x[2])[::-1]
        if n > 4:
            x[3, : n // 2] = x[3, n // 2: 2 * (n // 2)]  # every key twice: stability matters
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for desc in (False, True):
            want = np.sort(x, axis=1, kind="stable")
            want = want[:, ::-1] if desc else want
            assert np.array_equal(F.sort(Xh, -1, desc).numpy(), want)
            Y, I = F.argsort(Xh, -1, desc, with_values=True)
            Yo, Io = F.argsort(Xo, -1, desc, with_values=True)
            assert np.array_equal(I.numpy(), Io.numpy()) and np.array_equal(Y.numpy(), Yo.numpy())
            I64 = F.argsort(Xh, -1, desc, index_dtype=np.int64)
            assert I64.numpy().dtype == np.int64 and np.array_equal(I64.numpy(), Io.numpy())
        Z = Tensor.from_numpy(hip_backend, x)
        F.sort(Z, -1, False, out=Z)                      # in place
        assert np.array_equal(Z.numpy(), np.sort(x, axis=1, kind="stable"))


def test_short_rows_on_strided_views(hip_backend, oracle_backend):
    a = (normal(201, 40 * 9 * 300) * 20).astype(np.float32).reshape(40, 9, 300)
    T, O = Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(oracle_backend, a)
    for V, W, v in ((T.transpose(), O.transpose(), a.transpose()),
                    (T.slice([0, 1, 3], [40, 9, 300], None, [3, 2, 7]), O.slice([0, 1, 3], [40, 9, 300], None, [3, 2, 7]), a[::3, 1::2, 3::7]),
                    (T.flip([2]), O.flip([2]), a[:, :, ::-1])):
        for axis in range(3):
            assert np.array_equal(F.sort(V, axis).numpy(), np.sort(v, axis=axis, kind="stable"))
            assert np.array_equal(F.argsort(V, axis, True).numpy(), F.argsort(W, axis, True).numpy())
    # sorted into a strided output view
    out = Tensor.from_numpy(hip_backend, np.zeros((300, 9, 40), dtype=np.float32))
    F.sort(T, 2, False, out=out.transpose())
    assert np.array_equal(out.numpy(), np.sort(a, axis=2).transpose())
    # zeros of both signs in a short row: values keep their sign, equal keys keep their order
    z = np.array([[0.0, -0.0, 1.0, -0.0, 0.0, -1.0]], dtype=np.float32)
    Y, I = F.argsort(Tensor.from_numpy(hip_backend, z), -1, with_values=True)
    assert I.numpy().tolist() == [[5, 0, 1, 3, 4, 2]]
    assert np.array_equal(np.signbit(Y.numpy()), np.signbit(z[0][I.numpy()[0]])[None, :])


@pytest.mark.parametrize("n", [65, 128, 200, 256, 400, 512])
def test_short_rows_sorted_by_one_workgroup_when_the_wave_sort_is_switched_off(hip_backend, oracle_backend, n):
    """The one-workgroup kernel still serves rows of 65 to 512 elements when the knob that bounds
    the wave sort says so (and always for 4-byte keys with indices above 256)."""
    hip_backend.set_tuning("sort_wave_rows", 64)
    try:
        for dtype in (np.float32, np.int64, np.int16):
            x = (normal(220 + n, 300 * n) * 50).astype(dtype).reshape(300, n)
            x[3, : n // 2] = x[3, n // 2: 2 * (n // 2)]
            Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
            for desc in (False, True):
                Y, I = F.argsort(Xh, -1, desc, with_values=True)
                Yo, Io = F.argsort(Xo, -1, desc, with_values=True)
                assert np.array_equal(I.numpy(), Io.numpy()) and np.array_equal(Y.numpy(), Yo.numpy())
                assert np.array_equal(F.sort(Xh, -1, desc).numpy(), Yo.numpy())
    finally:
        hip_backend.set_tuning("sort_wave_rows", 512)


@pytest.mark.parametrize("n", [1, 2, 7, 33, 63, 64])
def test_short_rows_side_by_side_in_memory(hip_backend, oracle_backend, n):
    """sort / argsort along an outer axis of at most 64 elements with thousands of rows side by
    side: tiles of 64 rows pass through LDS.  All key widths, both directions, 64-bit indices,
    a middle axis, a row count that leaves part of the last tile empty, in place, signed zeros."""
    for dtype in (np.float32, np.int64, np.float64, np.int16, np.float16, np.int32):
        x = (normal(280 + n, n * 5003) * 50).astype(dtype).reshape(n, 5003)
        x[:, 1] = x[0, 1]
        if n > 4:
            x[: n // 2, 3] = x[n // 2: 2 * (n // 2), 3]            # every key twice: stability matters
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for desc in (False, True):
            want = np.sort(x, axis=0, kind="stable")
            want = want[::-1] if desc else want
            assert np.array_equal(F.sort(Xh, 0, desc).numpy(), want)
            Y, I = F.argsort(Xh, 0, desc, with_values=True)
            Yo, Io = F.argsort(Xo, 0, desc, with_values=True)
            assert np.array_equal(I.numpy(), Io.numpy()) and np.array_equal(Y.numpy(), Yo.numpy())
        I64 = F.argsort(Xh, 0, False, index_dtype=np.int64)
        assert I64.numpy().dtype == np.int64 and np.array_equal(I64.numpy(), F.argsort(Xo, 0).numpy())
        Z = Tensor.from_numpy(hip_backend, x)
        F.sort(Z, 0, False, out=Z)
        assert np.array_equal(Z.numpy(), np.sort(x, axis=0, kind="stable"))
    a = (normal(281 + n, 3 * n * 2100) * 9).astype(np.float32).reshape(3, n, 2100)
    a[1, 0, :] = 0.0
    if n > 1:
        a[1, n - 1, :] = -0.0
    T, O = Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(oracle_backend, a)
    Y, I = F.argsort(T, 1, True, with_values=True)
    Yo, Io = F.argsort(O, 1, True, with_values=True)
    assert np.array_equal(I.numpy(), Io.numpy()) and np.array_equal(Y.numpy().view(np.uint32), Yo.numpy().view(np.uint32))


@pytest.mark.parametrize("n", [65, 100, 128, 129, 161, 200, 255, 256, 257])
def test_rows_of_up_to_256_keys_side_by_side_in_memory(hip_backend, oracle_backend, n):
    """sort along an outer axis of 65 to 256 elements with thousands of rows side by side: 4-byte
    keys (8-byte keys up to 128 elements) pass through LDS in tiles of 16 rows (129 to 160
    elements and every argsort keep a wavefront per row).  Both directions, a row count that leaves the last tile ragged, a middle
    axis whose innermost run is shorter than a tile, in place, signed zeros and NaNs, a view
    that steps over every other row; the other key widths and argsort beside it."""
    cols = 4099
    for dtype in (np.float32, np.int32, np.int64, np.float64, np.float16):
        x = (normal(290 + n, n * cols) * 50).astype(dtype).reshape(n, cols)
        x[:, 1] = x[0, 1]
        x[: n // 2, 3] = x[n // 2: 2 * (n // 2), 3]
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        for desc in (False, True):
            want = np.sort(x, axis=0, kind="stable")
            want = want[::-1] if desc else want
            assert np.array_equal(F.sort(Xh, 0, desc).numpy(), want), (dtype, desc)
            I, Io = F.argsort(Xh, 0, desc), F.argsort(Xo, 0, desc)
            assert np.array_equal(I.numpy(), Io.numpy()), (dtype, desc)
        Z = Tensor.from_numpy(hip_backend, x)
        F.sort(Z, 0, False, out=Z)                                     # in place
        assert np.array_equal(Z.numpy(), np.sort(x, axis=0, kind="stable"))
        V = Xh.slice([0], [cols], [1], [2])                            # every other row
        assert np.array_equal(F.sort(V, 0).numpy(), np.sort(x[:, ::2], axis=0, kind="stable"))
    a = (normal(291 + n, 5 * n * 900) * 9).astype(np.float32).reshape(5, n, 900)
    a[1, 0, :] = 0.0
    a[1, n - 1, :] = -0.0
    a[2, 5, ::7] = np.nan
    # (comparisons do not order NaNs, nor -0.0 against +0.0: the keys' order-preserving images do - negative NaNs
    # first, -0.0 before +0.0, positive NaNs last -, and descending is that order reversed)
    bits = a.view(np.uint32)
    image = np.where(bits >> 31 != 0, ~bits, bits | np.uint32(0x80000000))
    by_image = np.take_along_axis(a, np.argsort(image, axis=1, kind="stable"), 1)
    T = Tensor.from_numpy(hip_backend, a)
    assert np.array_equal(F.sort(T, 1).numpy().view(np.uint32), by_image.view(np.uint32))
    assert np.array_equal(F.sort(T, 1, True).numpy().view(np.uint32), by_image[:, ::-1].view(np.uint32))
    b = (normal(292 + n, 700 * n * 6) * 9).astype(np.float32).reshape(700, n, 6)       # innermost runs of 6 rows
    assert np.array_equal(F.sort(Tensor.from_numpy(hip_backend, b), 1).numpy(), np.sort(b, axis=1, kind="stable"))
