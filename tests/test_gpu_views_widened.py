"""The widened operations (count, nonzero, merge, 16-bit and complex element types) on views that
do not walk memory in order: transposed, sliced with steps, flipped.  Expected values come from
numpy on the same view (and the oracle where numpy has no stable equivalent)."""
import numpy as np
import pytest

from dlf_amd import frontend as F
from dlf_amd.frontend import Tensor
from helpers import normal, randint

pytestmark = pytest.mark.gpu


def views(T, a):
    """(tensor view, numpy view) pairs of one 3-d tensor."""
    yield T, a
    yield T.transpose(), a.transpose()
    yield T.transpose([1, 2, 0]), a.transpose(1, 2, 0)
    yield T.slice([1, 0, 2], [a.shape[0], a.shape[1], a.shape[2]], None, [2, 3, 1]), a[1::2, ::3, 2:]
    yield T.flip([2]), a[:, :, ::-1]
    yield T.flip([0, 1]).transpose([2, 0, 1]), a[::-1, ::-1, :].transpose(2, 0, 1)


def test_count_and_nonzero_on_views(hip_backend):
    a = randint(180, 9 * 14 * 40, 0, 3).astype(np.float32).reshape(9, 14, 40)
    T = Tensor.from_numpy(hip_backend, a)
    for V, v in views(T, a):
        for axes in ((), (0,), (2,), (0, 1)):
            want = (v == 1).sum(axis=axes if axes else None)
            assert np.array_equal(F.count(V, np.float32(1), axes).numpy().reshape(-1), np.asarray(want).reshape(-1))
        assert np.array_equal(F.nonzero(V).numpy(), np.argwhere(v != 0))
        assert np.array_equal(F.nonzero(V, True).numpy(), np.array(np.nonzero(v)))


def test_merge_on_views(hip_backend, oracle_backend):
    a = np.sort(randint(181, 6 * 5 * 300, -50, 50).astype(np.int32).reshape(6, 5, 300), axis=2)
    b = np.sort(randint(182, 6 * 5 * 170, -50, 50).astype(np.int32).reshape(6, 5, 170), axis=2)
    A, B = Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(hip_backend, b)
    want = np.sort(np.concatenate([a, b], axis=2), axis=2)
    assert np.array_equal(F.merge(A, B).numpy(), want)
    # descending inputs as flipped views of the same storage
    got = F.merge(A.flip([2]), B.flip([2]), -1, True).numpy()
    assert np.array_equal(got, want[:, :, ::-1])
    # rows taken with a step, merged along the last axis
    got = F.merge(A.slice([0], [6], [0], [2]), B.slice([0], [6], [0], [2])).numpy()
    assert np.array_equal(got, want[::2])
    # merge along a middle axis: both inputs sorted along axis 1
    a1, b1 = np.sort(a, axis=1), np.sort(b[:, :, :300] if b.shape[2] >= 300 else np.resize(b, (6, 5, 300)), axis=1)
    got = F.merge(Tensor.from_numpy(hip_backend, a1), Tensor.from_numpy(hip_backend, b1), 1).numpy()
    assert np.array_equal(got, np.sort(np.concatenate([a1, b1], axis=1), axis=1))


@pytest.mark.parametrize("dtype", [np.float16, np.int16])
def test_sixteen_bit_sort_family_on_views(hip_backend, oracle_backend, dtype):
    a = (normal(183, 8 * 12 * 50) * 30).astype(dtype).reshape(8, 12, 50)
    T, O = Tensor.from_numpy(hip_backend, a), Tensor.from_numpy(oracle_backend, a)
    for (V, v), (W, _) in zip(views(T, a), views(O, a)):
        for axis in range(3):
            assert np.array_equal(F.sort(V, axis).numpy(), np.sort(v, axis=axis, kind="stable"))
            assert np.array_equal(F.argsort(V, axis, True).numpy(), F.argsort(W, axis, True).numpy())
            assert np.array_equal(F.argmax(V, axis).numpy(), F.argmax(W, axis).numpy())
            k = min(3, v.shape[axis])
            Yh, Ih = F.top_k(V, k, axis)
            Yo, Io = F.top_k(W, k, axis)
            assert np.array_equal(Ih.numpy(), Io.numpy()) and np.array_equal(Yh.numpy(), Yo.numpy())


@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
def test_complex_on_views(hip_backend, dtype):
    a = ((normal(184, 7 * 9 * 33) + 1j * normal(185, 7 * 9 * 33)) * 0.5).astype(dtype).reshape(7, 9, 33)
    T = Tensor.from_numpy(hip_backend, a)
    tol = dict(rtol=200 * np.finfo(dtype).eps, atol=200 * np.finfo(dtype).eps)
    for V, v in views(T, a):
        v128 = v.astype(np.complex128)
        for axes in ((), (1,), (0, 2)):
            got = F.reduce("reduce_sum", V, axes).numpy()
            assert np.allclose(got.reshape(-1), np.asarray(v128.sum(axis=axes if axes else None)).reshape(-1), **tol)
        for axis in range(3):
            assert np.allclose(F.cumsum(V, axis).numpy(), np.cumsum(v128, axis=axis), **tol)
            assert np.allclose(F.cumsum(V, axis, True, True).numpy()[(slice(None),) * axis + (slice(0, -1),)],
                               np.cumsum(v128[(slice(None),) * axis + (slice(None, None, -1),)], axis=axis)[(slice(None),) * axis + (slice(None, None, -1),)][(slice(None),) * axis + (slice(1, None),)], **tol)
        assert np.array_equal(F.count(V, dtype(a[0, 0, 0]), (2,)).numpy(), (v == a[0, 0, 0]).sum(axis=2))


def test_half_scans_and_softmax_on_views(hip_backend):
    a = (normal(186, 6 * 10 * 64) * 0.5).astype(np.float16).reshape(6, 10, 64)
    T = Tensor.from_numpy(hip_backend, a)
    for V, v in views(T, a):
        v64 = v.astype(np.float64)
        for axis in range(3):
            got = F.cumsum(V, axis).numpy().astype(np.float64)
            want = np.cumsum(v64, axis=axis)
            mag = np.cumsum(np.abs(v64), axis=axis)
            assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -10 + 1e-5 * mag + 2.0 ** -24).all()
            assert np.array_equal(F.cummax(V, axis).numpy(), np.maximum.accumulate(v, axis=axis))
        got = F.reduce("reduce_max", V, (1,)).numpy()
        assert np.array_equal(got, v.max(axis=1))


def test_contiguous_copy_of_views(hip_backend):
    """Tensor.contiguous(): transposed, sliced, broadcast and flipped views come back in
    row-major order in storage of their own (the layout copy softmax makes of a view)."""
    a = randint(211, 5 * 7 * 9, -1000, 1000).astype(np.int32).reshape(5, 7, 9)
    T = Tensor.from_numpy(hip_backend, a)
    for view, want in ((T.transpose([2, 0, 1]), a.transpose(2, 0, 1)),
                       (T.transpose([1, 0, 2]), a.transpose(1, 0, 2)),
                       (T.flip([1]), a[:, ::-1, :]),
                       (T, a)):
        C = view.contiguous()
        assert C.shape.is_contiguous() and C.storage is not view.storage
        assert (C.numpy() == want).all()
    before = T.numpy().copy()
    C = T.contiguous()
    C.storage.zero_()
    assert (T.numpy() == before).all()


@pytest.mark.parametrize("dtype", [np.int16, np.float32, np.int64, np.complex128, np.bool_])
def test_copy_and_fill_over_views(hip_backend, dtype):
    """dlfx_copy / dlfx_fill (gdnn.h:14-26): strided view to strided view, every element width."""
    rng = np.random.default_rng(212)
    a = rng.integers(0, 2 if dtype == np.bool_ else 1000, size=(6, 5, 8, 3)).astype(dtype)
    T = Tensor.from_numpy(hip_backend, a)
    for view, want in ((T.transpose([3, 1, 0, 2]), a.transpose(3, 1, 0, 2)),
                       (T.flip([0, 2]), a[::-1, :, ::-1, :]),
                       (T.slice([1, 2], [5, 7], [0, 2], [2, 3]), a[1:5:2, :, 2:7:3, :]),
                       (T.transpose([1, 0, 2, 3]).slice([0], [1], [3]), a.transpose(1, 0, 2, 3)[:, :, :, 0:1])):
        assert np.array_equal(view.contiguous().numpy(), want)
    # into a strided destination: the transposed view of a second tensor
    D = Tensor.from_numpy(hip_backend, np.zeros((8, 6), dtype=dtype))
    src = Tensor.from_numpy(hip_backend, a[:, 0, :, 0].copy())             # [6, 8]
    dv = D.transpose([1, 0])
    hip_backend.copy(F.dtype_code(dtype), src.shape.extents, src.storage, 0, src.shape.strides,
                     D.storage, dv.shape.offset, dv.shape.strides)
    assert np.array_equal(D.numpy(), a[:, 0, :, 0].T)
    # a stride of 0 on the source repeats it
    row = Tensor.from_numpy(hip_backend, a[0, 0, :, 0].copy())             # [8]
    hip_backend.copy(F.dtype_code(dtype), [6, 8], row.storage, 0, [0, 1], src.storage, 0, [8, 1])
    assert np.array_equal(src.numpy(), np.broadcast_to(a[0, 0, :, 0], (6, 8)))
    # fill of every other column
    value = a.reshape(-1)[7]
    hip_backend.fill(F.dtype_code(dtype), [6, 4], [8, 2], src.storage, 1, value)
    got = src.numpy()
    assert (got[:, 1::2] == value).all() and np.array_equal(got[:, 0::2], np.broadcast_to(a[0, 0, 0::2, 0], (6, 4)))
