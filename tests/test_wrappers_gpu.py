"""Thin wrappers on the sort path: sort_complex, partition, argpartition
(cupynumeric/_module/ssc_sorting.py:124-268, tests/integration/test_sort_complex.py,
test_partition.py)."""
from __future__ import annotations

import numpy as np
import pytest
from conftest import ALL_REAL_DTYPES, make_input

import cupynumeric_amd as num

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ALL_REAL_DTYPES + [np.complex64, np.complex128])
def test_sort_complex_matches_numpy(dtype):
    for shape in [(12,), (3, 4), (2, 2, 3), (0,), (1,)]:
        x = make_input(dtype, shape, seed=3, special=False)
        if np.dtype(dtype).kind == "f":
            x = np.round(x * 4) / 4
        got = num.sort_complex(num.array(x))
        want = np.sort_complex(x)
        assert got.dtype == want.dtype, (dtype, got.dtype, want.dtype)
        assert got.shape == want.shape
        assert np.array_equal(np.asarray(got), want)


def partition_property(part: np.ndarray, original: np.ndarray, kth: int, axis: int) -> None:
    """tests/integration/test_partition.py:23-47: everything left of kth is <=, right is >=; and
    the element at kth is the one a full sort puts there."""
    p = np.moveaxis(part, axis, -1)
    s = np.moveaxis(np.sort(original, axis=axis, kind="stable"), axis, -1)
    assert np.array_equal(p[..., kth], s[..., kth])
    if kth > 0:
        assert (p[..., :kth].max(axis=-1) <= p[..., kth]).all()
    assert (p[..., kth:].min(axis=-1) >= p[..., kth]).all()
    assert np.array_equal(np.sort(p, axis=-1), s)  # same multiset per row


@pytest.mark.parametrize("dtype", [np.uint32, np.int8, np.float32, np.float64])
def test_partition_and_argpartition(dtype):
    for shape in [(30,), (7, 11), (3, 4, 5)]:
        x = make_input(dtype, shape, seed=9, special=False)
        a = num.array(x)
        for axis in range(-len(shape), len(shape)):
            for kth in (0, shape[axis] // 2, shape[axis] - 1):
                partition_property(np.asarray(num.partition(a, kth, axis=axis)), x, kth, axis)
                idx = np.asarray(num.argpartition(a, kth, axis=axis))
                assert idx.dtype == np.int64 and idx.shape == x.shape
                partition_property(np.take_along_axis(x, idx, axis=axis), x, kth, axis)
                assert np.array_equal(np.asarray(a.argpartition(kth, axis=axis)), idx)
                b = num.array(x)
                b.partition(kth, axis=axis)
                partition_property(np.asarray(b), x, kth, axis)
    flat = num.partition(num.array(make_input(np.int32, (4, 5), seed=1)), 3, axis=None)
    assert flat.shape == (20,)


def test_partition_validation():
    a = num.array(np.arange(6).reshape(2, 3))
    with pytest.raises(ValueError, match="invalid axis"):
        num.partition(a, 1, axis=2)
    with pytest.raises(NotImplementedError):
        num.argpartition(a, 1, order="x")
