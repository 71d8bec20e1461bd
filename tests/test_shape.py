"""Host view algebra (mirror of dlf's Shape, moveaxis, flip, prepare_reduce)."""
import numpy as np
import pytest

from dlf_amd.frontend import prepare_reduce
from dlf_amd.shape import Shape, ShapeError, norm_axes, norm_axis


def gather(shape, base):
    return np.array([base[shape.linear_offset(i)] for i in range(shape.size)]).reshape(shape.extents)


def test_row_major_strides_and_contiguity():
    s = Shape([2, 3, 4])
    assert s.strides == (12, 4, 1) and s.size == 24 and s.is_contiguous()
    assert not s.transpose().is_contiguous()


def test_transpose_and_moveaxis_match_numpy():
    base = np.arange(2 * 3 * 4 * 5)
    a = base.reshape(2, 3, 4, 5)
    s = Shape([2, 3, 4, 5])
    assert np.array_equal(gather(s.transpose([2, 0, 3, 1]), base), a.transpose(2, 0, 3, 1))
    for src, dst in [(0, -1), (1, -1), (3, 0), (-1, 1), (2, 2)]:
        assert np.array_equal(gather(s.moveaxis(src, dst), base), np.moveaxis(a, src, dst))


def test_slice_and_flip_match_numpy():
    base = np.arange(6 * 7)
    a = base.reshape(6, 7)
    s = Shape([6, 7])
    assert np.array_equal(gather(s.slice([1, 2], [5, 7]), base), a[1:5, 2:7])
    assert np.array_equal(gather(s.slice([5], [0], [0], [-2]), base), a[5:0:-2])
    assert np.array_equal(gather(s.flip([1]), base), a[:, ::-1])
    assert np.array_equal(gather(s.flip(), base), a[::-1, ::-1])
    assert s.flip([1]).strides == (7, -1) and s.flip([1]).offset == 6


def test_rank1_transpose_adds_unit_axis():
    assert Shape([5]).transpose().extents == (5, 1)


def test_axis_errors():
    with pytest.raises(ShapeError):
        norm_axis(3, 3)
    with pytest.raises(ShapeError):
        norm_axes(3, [0, 0])
    assert norm_axes(3, [-1, 0]) == [2, 0]
    with pytest.raises(ShapeError):
        Shape([2, 3]).transpose([0, 0])


def test_prepare_reduce_nchw_views():
    # kept axes first (original order), then reduced axes; m, n their products
    s = Shape([32, 512, 56, 56])
    v, out, m, n = prepare_reduce(s, [2, 3], False)
    assert v.strides == s.strides and out == [32, 512] and (m, n) == (16384, 3136)
    v, out, m, n = prepare_reduce(s, [1], True)
    assert v.extents == (32, 56, 56, 512) and v.strides == (1605632, 56, 1, 3136)
    assert out == [32, 1, 56, 56] and (m, n) == (100352, 512)
    v, out, m, n = prepare_reduce(s, [], False)
    assert out == [] and (m, n) == (1, s.size)
