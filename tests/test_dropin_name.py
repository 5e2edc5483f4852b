"""The reference's own name for the package: `import cupynumeric as np` must resolve to the sort
path built here, and the reference's sort example (examples/sort.py:24-89: seeded random input,
`np.sort(a, axis)` / `np.argsort(a, axis)`, `--check` against numpy.sort) must run on it."""
from __future__ import annotations

import numpy
import pytest


def test_cupynumeric_is_the_sort_package():
    import cupynumeric
    import cupynumeric.random  # noqa: F401
    import cupynumeric_amd

    for name in cupynumeric_amd.__all__:
        assert getattr(cupynumeric, name) is getattr(cupynumeric_amd, name), name
    assert cupynumeric.random is cupynumeric_amd.random
    assert cupynumeric.ndarray.sort is cupynumeric_amd.ndarray.sort


def run_sort(np, shape, axis, argsort, datatype, lower=None, upper=None):
    # examples/sort.py:37-89 (`np` is the array module under test, as there)
    np.random.seed(42)
    newtype = numpy.dtype(datatype).type
    n = int(numpy.prod(shape))
    if numpy.issubdtype(newtype, numpy.integer):
        lower = numpy.iinfo(newtype).min if lower is None else lower
        upper = numpy.iinfo(newtype).max if upper is None else upper
        a = np.random.randint(low=lower, high=upper, size=n).astype(newtype)
        a = a.reshape(shape)
    else:
        a = np.random.random(shape).astype(newtype)
    return a, (np.argsort(a, axis) if argsort else np.sort(a, axis))


@pytest.mark.gpu
@pytest.mark.parametrize("datatype", ["int32", "uint8", "float32", "float64"])
@pytest.mark.parametrize("shape,axis", [((100000,), -1), ((300, 257), -1), ((300, 257), 0), ((7, 50, 33), 1)])
def test_sort_example_check(datatype, shape, axis):
    import cupynumeric as np

    a, a_sorted = run_sort(np, shape, axis, False, datatype)
    # check_sorted (examples/sort.py:24-34): numpy.sort of the same input
    a_numpy = numpy.asarray(a)
    assert a_numpy.dtype == numpy.dtype(datatype) and a_numpy.shape == tuple(shape)
    assert numpy.allclose(numpy.sort(a_numpy, axis), numpy.asarray(a_sorted))
    assert numpy.array_equal(numpy.sort(a_numpy, axis, kind="stable"), numpy.asarray(a_sorted))
    a2, order = run_sort(np, shape, axis, True, datatype)
    assert numpy.array_equal(numpy.asarray(a2), a_numpy)  # same seed, same input
    assert numpy.array_equal(numpy.asarray(order), numpy.argsort(a_numpy, axis, kind="stable"))
