"""softmax / logsoftmax / hardmax: HIP path vs the CPU oracle (the reference's row loops).

hardmax is exact.  softmax and logsoftmax: the reference sums a row serially in the element
type, which for long fp32 rows is itself several hundred ulp away from the exact value, so
fp32 results are held to |got - exact| <= 4 * log2(n) * eps32 * |exact| (softmax: all terms
are non-negative, no cancellation; logsoftmax: scaled by max(1, |exact|)) against an fp64
evaluation of the same formula, and the oracle is checked to lie within its own serial-sum
error of that value.  fp64 results are compared with the oracle within
(4 * log2(n) + sqrt(n)) * eps64."""
import numpy as np
import pytest
from scipy.special import log_softmax as sp_log_softmax, softmax as sp_softmax

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import normal, randint

pytestmark = pytest.mark.gpu


def check_rows(hip, orc, x, axis):
    Xh, Xo = Tensor.from_numpy(hip, x), Tensor.from_numpy(orc, x)
    m = int(np.prod(x.shape[:axis]))
    n = x.size // m
    eps = float(np.finfo(x.dtype).eps)
    tiny = float(np.finfo(x.dtype).tiny)
    gs = F.softmax(Xh, axis).numpy().astype(np.float64).reshape(m, n)
    gl = F.logsoftmax(Xh, axis).numpy().astype(np.float64).reshape(m, n)
    ws = F.softmax(Xo, axis).numpy().astype(np.float64).reshape(m, n)
    wl = F.logsoftmax(Xo, axis).numpy().astype(np.float64).reshape(m, n)
    if x.dtype == np.float32:
        flat = x.reshape(m, n).astype(np.float64)
        es, el = sp_softmax(flat, axis=1), sp_log_softmax(flat, axis=1)
        bound = 4 * max(1.0, np.log2(n)) * eps
        assert (np.abs(gs - es) <= bound * np.maximum(es, tiny)).all()
        assert (np.abs(gl - el) <= bound * np.maximum(1.0, np.abs(el))).all()
        serial = (n + 8) * eps                          # what a serial fp32 sum may be off by
        assert (np.abs(ws - es) <= serial * np.maximum(es, tiny)).all()
        assert (np.abs(wl - el) <= serial * np.maximum(1.0, np.abs(el))).all()
    else:
        bound = (4 * max(1.0, np.log2(n)) + np.sqrt(n)) * eps
        assert (np.abs(gs - ws) <= bound * np.maximum(ws, tiny)).all()
        assert (np.abs(gl - wl) <= bound * np.maximum(1.0, np.abs(wl))).all()
    assert np.array_equal(F.hardmax(Xh, axis).numpy(), F.hardmax(Xo, axis).numpy())


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [1, 2, 7, 64, 65, 256, 1000, 1023, 2048, 2049, 8191, 16384, 32000, 32768, 40000, 100003])
def test_rows_of_every_size_class(hip_backend, oracle_backend, dtype, n):
    x = (normal(100 + n, 5 * n) * 4).astype(dtype).reshape(5, n)
    check_rows(hip_backend, oracle_backend, x, 1)


def test_axes_views_and_special_values(hip_backend, oracle_backend):
    x = (normal(101, 6 * 10 * 33) * 2).astype(np.float32).reshape(6, 10, 33)
    for axis in (0, 1, 2):
        check_rows(hip_backend, oracle_backend, x, axis)
    Xh, Xo = Tensor.from_numpy(hip_backend, x).transpose([1, 0, 2]), Tensor.from_numpy(oracle_backend, x).transpose([1, 0, 2])
    assert np.allclose(F.softmax(Xh, 2).numpy(), F.softmax(Xo, 2).numpy(), rtol=1e-5, atol=1e-9)
    # large magnitudes do not overflow (the row maximum is subtracted), -inf entries get weight 0
    s = np.array([[10000.0, 10001.0, -np.inf, 10003.0], [-5.0, -np.inf, -np.inf, -5.0]], dtype=np.float32)
    g = F.softmax(Tensor.from_numpy(hip_backend, s), 1).numpy()
    w = F.softmax(Tensor.from_numpy(oracle_backend, s), 1).numpy()
    assert np.allclose(g, w, rtol=1e-6) and g[0, 2] == 0 and np.allclose(g[1], [0.5, 0, 0, 0.5])
    # rows far from zero: x - max must be formed before log(sum) is subtracted
    big = (normal(103, 4 * 1000) * 2 + 30000).astype(np.float32).reshape(4, 1000)
    check_rows(hip_backend, oracle_backend, big, 1)
    # ties: the first maximum is the hot one (DNNTest.cpp:848-858); long rows of equal values too
    t = np.full((3, 5000), 2.5, dtype=np.float32)
    h = F.hardmax(Tensor.from_numpy(hip_backend, t), 1).numpy()
    assert (h[:, 0] == 1).all() and h.sum() == 3


def test_large_matrix_property(hip_backend):
    # the benchmark shape at reduced height: rows sum to one, order is preserved
    x = (normal(102, 64 * 32000) * 2).astype(np.float32).reshape(64, 32000)
    y = F.softmax(Tensor.from_numpy(hip_backend, x), 1).numpy().astype(np.float64)
    assert np.allclose(y.sum(axis=1), 1.0, atol=1e-5)
    assert np.array_equal(np.argmax(y, axis=1), np.argmax(x, axis=1))


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
@pytest.mark.parametrize("n", [1, 9, 300, 5000, 20000, 40000])
def test_hardmax_of_integer_rows(hip_backend, oracle_backend, dtype, n):
    # the reference instantiates hardmax (only) for int32 / int64 as well (gdnn.cpp:1897-1902)
    x = randint(150 + n, 6 * n, -40, 40).astype(dtype).reshape(6, n)
    x[3] = np.iinfo(dtype).min                      # a row of the lowest value: the first element is hot
    got = F.hardmax(Tensor.from_numpy(hip_backend, x), 1).numpy()
    assert got.dtype == dtype
    assert np.array_equal(got, F.hardmax(Tensor.from_numpy(oracle_backend, x), 1).numpy())
    want = np.zeros_like(x)
    want[np.arange(6), x.argmax(axis=1)] = 1
    assert np.array_equal(got, want)
    with pytest.raises(Exception):
        F.softmax(Tensor.from_numpy(hip_backend, x), 1)


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 8, 10, 15, 16, 17, 31, 32, 33, 61, 63, 64, 65, 66, 125, 128, 129, 189, 192, 193, 253, 255, 257, 509, 512, 513, 765, 768, 769, 1021, 1025, 1533, 1536, 1537,
                               2045, 2047, 2051, 3069, 3072, 3073, 4095, 4096, 4097, 6141, 6144, 6145, 8189, 8193, 12285, 12289, 16381, 16385, 24573, 24577, 32765])
def test_row_lengths_around_the_team_sizes(hip_backend, oracle_backend, n):
    """One lane per row up to 4 (fp32) / 2 (fp64) / 8 (half) elements, four lanes up to four times
    that, sixteen lanes per row up to 128 (fp32) elements, a wavefront up to 2048, a workgroup of
    256 threads up to 6144 and of 1024 threads up to 32768: the boundaries of each class.  Rows that do not start on a 16-byte
    boundary (odd lengths) are laid out from the boundary before them, which moves those
    boundaries down by up to a vector less one element; the output rows here start on other
    boundaries than the input rows (a view that begins one row into its buffer)."""
    m = 700 if n <= 16 else 70 if n < 1000 else 9     # several workgroups of one- and four-lane teams
    for dtype in (np.float32, np.float64, np.float16):
        x = (normal(230 + n, m * n) * 2).astype(dtype).reshape(m, n)
        x[1] = x[1, 0]                                   # a constant row
        if n > 2:
            x[2, n // 2] = np.nan                        # a NaN that is not in position 0 is skipped
        Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
        x64 = np.delete(x, 2, axis=0).astype(np.float64) if n > 2 else x.astype(np.float64)
        keep = [r for r in range(m) if not (n > 2 and r == 2)]
        eps = np.finfo(np.float32 if dtype == np.float16 else dtype).eps
        out_ulp = 2.0 ** -10 if dtype == np.float16 else 0.0
        slack = 8 * max(1.0, np.log2(n)) * eps + out_ulp
        got = F.softmax(Xh).numpy().astype(np.float64)[keep]
        assert (np.abs(got - sp_softmax(x64, axis=1)) <= sp_softmax(x64, axis=1) * slack + 1e-30 + (2.0 ** -24 if dtype == np.float16 else 0)).all(), dtype
        got = F.logsoftmax(Xh).numpy().astype(np.float64)[keep]
        want = sp_log_softmax(x64, axis=1)
        assert (np.abs(got - want) <= slack * (1 + np.abs(want)) + out_ulp * np.abs(want)).all(), dtype
        assert np.array_equal(F.hardmax(Xh).numpy(), F.hardmax(Xo).numpy()), dtype
        if dtype == np.float32 and n > 1:
            Vh, Vo = Xh.slice([1], [m], [0]), Xo.slice([1], [m], [0])          # the same rows from the second on
            assert np.array_equal(F.softmax(Vh).numpy(), F.softmax(Xh).numpy()[1:], equal_nan=True)
            assert np.array_equal(F.hardmax(Vh).numpy(), F.hardmax(Vo).numpy())


@pytest.mark.parametrize("n,dtype", [(32769, np.float32), (40957, np.float32), (40960, np.float32), (49153, np.float32), (50257, np.float32),
                                     (57344, np.float32), (65533, np.float32), (65536, np.float32), (65537, np.float32), (50257, np.float16),
                                     (65536, np.float16), (16385, np.float64), (24577, np.float64), (32765, np.float64), (32768, np.float64)])
def test_many_long_rows_are_held_in_registers(hip_backend, oracle_backend, n, dtype):
    """With at least 256 rows, rows of up to 65536 4-byte (32768 8-byte) elements are held in the
    registers of one workgroup, 40 to 64 a thread, and read once; longer ones are streamed.
    All three kinds, rows that start off a 16-byte boundary, a NaN in position 0 and elsewhere,
    -inf entries, a constant row."""
    m = 257
    x = (normal(280 + n, m * n) * 3).astype(dtype).reshape(m, n)
    x[0, n // 3] = -np.inf
    x[1, 0] = np.nan
    x[2, n - 5] = np.nan
    x[3] = 2.5
    Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
    eps = float(np.finfo(np.float32 if dtype == np.float16 else dtype).eps)
    out_ulp = 2.0 ** -10 if dtype == np.float16 else 0.0
    slack = 8 * np.log2(n) * eps + out_ulp
    clean = [r for r in range(m) if r not in (1, 2)]
    x64 = x[clean].astype(np.float64)
    got = F.softmax(Xh).numpy().astype(np.float64)
    want = sp_softmax(x64, axis=1)
    assert (np.abs(got[clean] - want) <= want * slack + 1e-30 + (2.0 ** -24 if dtype == np.float16 else 0)).all()
    assert np.isnan(got[1]).all() and np.isnan(got[2]).all()
    got = F.logsoftmax(Xh).numpy().astype(np.float64)
    want = sp_log_softmax(x64, axis=1)
    fin = np.isfinite(want)
    assert (np.abs(got[clean][fin] - want[fin]) <= slack * (1 + np.abs(want[fin])) + out_ulp * np.abs(want[fin])).all()
    assert np.array_equal(np.isneginf(got[clean]), np.isneginf(want))
    assert np.array_equal(F.hardmax(Xh).numpy(), F.hardmax(Xo).numpy())


@pytest.mark.parametrize("m,n,dtype", [(1, 200000, np.float32), (3, 70001, np.float32), (7, 40000, np.float64), (2, 32769, np.float32),
                                       (5, 16385, np.float64), (2, 100000, np.float16), (200, 33000, np.float32)])
def test_few_long_rows_are_cut_into_tiles(hip_backend, oracle_backend, m, n, dtype):
    """Fewer than 256 rows that are too long for one workgroup's registers: every row is cut
    into tiles that the whole device works on (two kernels, one record per tile in scratch).
    All three kinds, in place and out of place, a NaN in position 0 and elsewhere, -inf entries,
    an all -inf row, and the same call without scratch (one workgroup per row)."""
    import ctypes
    x = (normal(260 + n, m * n) * 3).astype(dtype).reshape(m, n)
    x[0, n // 3] = -np.inf
    if m > 1:
        x[1, 0] = np.nan                                 # the reference's maximum: the whole row becomes NaN
    if m > 2:
        x[2, n - 5] = np.nan                             # poisons the sum, not the maximum
    if m > 4:
        x[4] = -np.inf
    Xh, Xo = Tensor.from_numpy(hip_backend, x), Tensor.from_numpy(oracle_backend, x)
    eps = float(np.finfo(np.float32 if dtype == np.float16 else dtype).eps)
    out_ulp = 2.0 ** -10 if dtype == np.float16 else 0.0
    slack = 8 * np.log2(n) * eps + out_ulp
    clean = [r for r in range(m) if r not in (1, 2, 4)]
    x64 = x[clean].astype(np.float64)
    results = {}
    for name, fn, want in (("softmax", F.softmax, sp_softmax(x64, axis=1)), ("logsoftmax", F.logsoftmax, sp_log_softmax(x64, axis=1))):
        got = fn(Xh).numpy().astype(np.float64)
        results[name] = got
        if name == "softmax":
            assert (np.abs(got[clean] - want) <= want * slack + 1e-30 + (2.0 ** -24 if dtype == np.float16 else 0)).all()
        else:
            fin = np.isfinite(want)
            assert (np.abs(got[clean][fin] - want[fin]) <= slack * (1 + np.abs(want[fin])) + out_ulp * np.abs(want[fin])).all()
            assert (got[clean][~fin] == -np.inf).all()
        ref = fn(Xo).numpy().astype(np.float64)
        for r in (1, 2, 4):                              # NaN rows and the all -inf row: the same non-finite pattern as the reference's loop
            if r < m:
                assert np.array_equal(np.isnan(got[r]), np.isnan(ref[r])), (name, r)
    assert np.array_equal(F.hardmax(Xh).numpy(), F.hardmax(Xo).numpy())
    # in place (the reference's calling convention)
    Z = Tensor.from_numpy(hip_backend, x)
    hip_backend.softmax("softmax", F.dtype_code(Z.dtype), m, n, Z.storage, 0, Z.storage, 0)
    assert np.array_equal(np.nan_to_num(Z.numpy().astype(np.float64), nan=-7.0), np.nan_to_num(results["softmax"], nan=-7.0))
    # no scratch given: one workgroup per row, the same values up to the order of the sums
    lib = hip_backend.lib
    assert lib.dlfx_softmax_scratch_bytes(F.dtype_code(x.dtype), m, n) > 0
    Y = Tensor.empty(hip_backend, [m, n], x.dtype)
    import torch
    st = lib.dlfx_softmax(torch.cuda.current_stream().cuda_stream, b"softmax", F.dtype_code(x.dtype), m, n,
                          Xh.storage.data_ptr(), 0, Y.storage.data_ptr(), 0, None, 0)
    assert st == 0
    a, b = Y.numpy().astype(np.float64)[clean], results["softmax"][clean]
    assert (np.abs(a - b) <= b * 2 * slack + 1e-30 + (2.0 ** -23 if dtype == np.float16 else 0)).all()


@pytest.mark.parametrize("n", [3000, 3001, 5001, 20000, 20003, 32766, 32768, 50257])
def test_hardmax_in_place_with_a_leading_nan(hip_backend, n):
    """In place (the reference's routine, gdnn.h:253-264, only works in place) on rows held by a
    workgroup of 256 or 1024 threads, rows off a 16-byte boundary among them (odd lengths: the
    first and last vectors of a row are then shared with its neighbours, which other workgroups
    rewrite at the same time): a row that starts with a NaN keeps position 0 hot (nothing compares
    larger than a NaN in the serial loop, dnn_detail.h:334-346), and exactly one element is hot,
    whichever wave stores element 0 first."""
    x = (normal(171 + n, 64 * n) * 3).astype(np.float32).reshape(64, n)
    x[::2, 0] = np.nan
    x[1::2, n - 1] = 50.0
    X = Tensor.from_numpy(hip_backend, x)
    for _ in range(3):
        X.storage.copy_(Tensor.from_numpy(hip_backend, x).storage)
        hip_backend.softmax("hardmax", F.dtype_code(np.float32), 64, n, X.storage, 0, X.storage, 0)
        y = X.numpy()
        assert (y.sum(axis=1) == 1).all()
        assert (y[::2, 0] == 1).all() and (y[1::2, n - 1] == 1).all()
    # softmax in place agrees with softmax out of place
    x[::2, 0] = 0.5
    X.storage.copy_(Tensor.from_numpy(hip_backend, x).storage)
    want = F.softmax(Tensor.from_numpy(hip_backend, x)).numpy()
    hip_backend.softmax("softmax", F.dtype_code(np.float32), 64, n, X.storage, 0, X.storage, 0)
    assert np.array_equal(X.numpy(), want)
