"""MI355X-native sort / argsort behind the cuPyNumeric API.

    import cupynumeric_amd as num
    a = num.array(host_array)
    num.sort(a, axis=0); num.argsort(a, kind="stable"); a.sort()

Only the sort path of cuPyNumeric is provided (`cupynumeric/_module/ssc_sorting.py:29-121`,
`cupynumeric/_array/array.py:3773-3824`).  Every sort runs in hand-written HIP kernels of
`libcpnsort.so`; there is no CPU fallback.
"""
from __future__ import annotations

from typing import Any

import numpy as np

from . import random  # noqa: F401
from ._array import convert_to_ndarray, ndarray
from ._thunk import SUPPORTED_DTYPES, DeviceArray, check_dtype

__all__ = [
    "ndarray", "array", "asarray", "sort", "argsort", "sort_complex", "partition", "argpartition", "lexsort", "searchsorted", "unique", "take_along_axis",
    "quantile", "percentile", "median", "nanquantile", "nanpercentile", "nanmedian",
    "random",
    "SUPPORTED_DTYPES",
]

__version__ = "0.1.0"


def array(obj: Any, dtype: Any = None, copy: bool = True) -> ndarray:
    """Create an array from an array-like (host data is uploaded on first device use)."""
    if isinstance(obj, ndarray) and dtype is None and not copy:
        return obj
    host = np.array(obj, dtype=dtype, copy=True)
    check_dtype(host.dtype)
    return ndarray(host.shape, host.dtype, thunk=DeviceArray.from_numpy(host))


def asarray(obj: Any, dtype: Any = None) -> ndarray:
    if isinstance(obj, ndarray) and (dtype is None or np.dtype(dtype) == obj.dtype):
        return obj
    return array(obj, dtype=dtype)


def argsort(a: Any, axis: int | None = -1, kind: str = "quicksort", order: Any = None) -> ndarray:
    """Indices that would sort `a` (`cupynumeric/_module/ssc_sorting.py:29-74`).

    `kind` is 'quicksort', 'mergesort', 'heapsort' or 'stable'; every kind is served by the same
    stable kernels.  `order` is not supported.  The result is int64, of `a.shape`, or flat when
    `axis` is None.
    """
    a = convert_to_ndarray(a)
    if axis is None:
        result = ndarray((a.size,), np.int64)
    else:
        result = ndarray(a.shape, np.int64)
    result._thunk.sort(rhs=a._thunk, argsort=True, axis=axis, kind=kind, order=order)
    return result


def sort(a: Any, axis: int | None = -1, kind: str = "quicksort", order: Any = None) -> ndarray:
    """Sorted copy of `a` (`cupynumeric/_module/ssc_sorting.py:77-121`); flat when `axis` is None."""
    a = convert_to_ndarray(a)
    if axis is None:
        result = ndarray((a.size,), a.dtype)
    else:
        result = ndarray(a.shape, a.dtype)
    result._thunk.sort(rhs=a._thunk, axis=axis, kind=kind, order=order)
    return result


def sort_complex(a: Any) -> ndarray:
    """Sorted copy along the last axis, always complex (`cupynumeric/_module/ssc_sorting.py:124-159`):
    complex input keeps its type, integers of at most 16 bits give complex64, everything else
    complex128."""
    result = sort(a)
    # force complex result upon return
    if np.issubdtype(result.dtype, np.complexfloating):
        return result
    elif np.issubdtype(result.dtype, np.integer) and result.dtype.itemsize <= 2:
        return result.astype_complex(np.complex64)
    else:
        return result.astype_complex(np.complex128)


def argpartition(a: Any, kth: Any, axis: int | None = -1, kind: str = "introselect", order: Any = None) -> ndarray:
    """Indirect partition (`cupynumeric/_module/ssc_sorting.py:165-218`); falls back to argsort."""
    a = convert_to_ndarray(a)
    result = ndarray(a.shape, np.int64)
    result._thunk.partition(rhs=a._thunk, argpartition=True, kth=kth, axis=axis, kind=kind, order=order)
    if axis is None and a.ndim > 1:
        result._thunk.shape = (a.size,)
    return result


def partition(a: Any, kth: Any, axis: int | None = -1, kind: str = "introselect", order: Any = None) -> ndarray:
    """Partitioned copy (`cupynumeric/_module/ssc_sorting.py:221-268`); falls back to sort."""
    a = convert_to_ndarray(a)
    result = ndarray(a.shape, a.dtype)
    result._thunk.partition(rhs=a._thunk, kth=kth, axis=axis, kind=kind, order=order)
    if axis is None and a.ndim > 1:
        result._thunk.shape = (a.size,)
    return result


def lexsort(keys: Any, axis: int | None = -1) -> ndarray:
    """Indirect stable sort on several keys, the last key being the primary one
    (`cupynumeric/_module/ssc_sorting.py:271-444`).  `keys` is a sequence of arrays of one
    shape, or one array whose first dimension runs over the keys.  Returns int64 indices of
    the shape of one key.  `axis=None` is rejected as NumPy does."""
    from numpy.exceptions import AxisError

    from ._sort import lexsort_deferred

    if keys is None:
        raise TypeError("'NoneType' object is not iterable")
    if axis is None:
        raise TypeError("'NoneType' object cannot be interpreted as an integer")

    if isinstance(keys, ndarray):
        if keys.ndim == 0:
            raise TypeError("need sequence of keys with len > 0 in lexsort")
        key_list = _split_first_axis(keys)
    else:
        try:
            key_list = [convert_to_ndarray(k) for k in keys]
        except TypeError as exc:
            if "does not support dtype" in str(exc):
                raise
            raise TypeError(str(exc))
    if len(key_list) == 0:
        raise TypeError("Need at least one key to sort")

    # all keys must have one shape
    first_shape = key_list[0].shape
    for i, key in enumerate(key_list[1:], 1):
        if key.shape != first_shape:
            raise ValueError(
                f"All keys must have the same shape. Key {i} has shape {key.shape}, expected {first_shape}"
            )

    # scalar keys: there is only one element
    if len(first_shape) == 0:
        return array(np.zeros((), dtype=np.int64))

    ndim = len(first_shape)
    if axis >= ndim or axis < -ndim:
        raise AxisError(f"axis {axis} is out of bounds for array of dimension {ndim}")

    # valid keys without data
    if key_list[0].size == 0:
        return ndarray(first_shape, np.int64)

    thunk = lexsort_deferred([k._thunk for k in key_list], axis)
    return ndarray(thunk.shape, np.int64, thunk=thunk)


def searchsorted(a: Any, v: Any, side: str = "left", sorter: Any = None) -> ndarray:
    """Indices at which `v` would be inserted into the sorted 1-D array `a` keeping it sorted
    (`cupynumeric/_module/ssc_searching.py:31-68`).  `a` must be an array object
    (the reference calls `a.searchsorted`, so `None` fails with AttributeError there too)."""
    if not isinstance(a, ndarray):
        if a is None:
            raise AttributeError("'NoneType' object has no attribute 'searchsorted'")
        a = convert_to_ndarray(a)
    return a.searchsorted(v, side, sorter)


def unique(
    ar: Any,
    return_index: bool = False,
    return_inverse: bool = False,
    return_counts: bool = False,
    axis: int | None = None,
) -> ndarray:
    """Sorted distinct elements of `ar`, flattened (`cupynumeric/_module/sets_making.py:25-122`).
    The optional outputs and `axis` are not supported, as in the reference."""
    ar = convert_to_ndarray(ar)
    if any((return_index, return_inverse, return_counts)) or axis is not None:
        raise NotImplementedError("Keyword arguments for `unique` are not yet supported")
    return ar.unique()


def take_along_axis(a: Any, indices: Any, axis: int | None) -> ndarray:
    """Values of `a` at `indices` along `axis` (`cupynumeric/_module/indexing.py:657-770`): every
    dimension other than `axis` agrees between `a` and `indices` or is 1 on one side (NumPy's
    broadcasting; shapes that do not broadcast raise IndexError, as in NumPy).  `axis=None` flattens
    `a` and wants 1-D indices.  Indices out of range raise IndexError from this call."""
    from numpy.lib.array_utils import normalize_axis_index

    a = convert_to_ndarray(a)
    indices = convert_to_ndarray(indices)
    if not np.issubdtype(indices.dtype, np.integer):
        raise TypeError("`indices` must be an integer array")

    computed_axis = 0
    if axis is None:
        if indices.ndim != 1:
            raise ValueError("indices must be 1D if axis=None")
        if a.ndim > 1:
            a = ndarray((a.size,), a.dtype, thunk=a._thunk.reshape((a.size,)))
    else:
        computed_axis = normalize_axis_index(axis, a.ndim)

    if a.ndim != indices.ndim:
        raise ValueError("`indices` and `a` must have the same number of dimensions")
    if indices.dtype != np.dtype(np.int64):
        indices = indices.astype(np.int64)

    last = a.ndim - 1
    src, idx = a._thunk, indices._thunk
    if computed_axis != last:
        src = src.swapaxes_copy(computed_axis, last)
        idx = idx.swapaxes_copy(computed_axis, last)
    out = src.take_along_last_axis(idx)
    if computed_axis != last:
        out = out.swapaxes_copy(last, computed_axis)
    return ndarray(out.shape, out.dtype, thunk=out)


def _split_first_axis(a: ndarray) -> list[ndarray]:
    """The keys of a single stacked array: `a[0], a[1], ...` as dense arrays sharing nothing."""
    if a.shape[0] == 0:
        return []
    host_or_dev = a._thunk
    inner = a.shape[1:]
    n_inner = int(np.prod(inner, dtype=np.int64))
    out = []
    for i in range(a.shape[0]):
        out.append(ndarray(inner, a.dtype, thunk=host_or_dev.slice_first_axis(i, n_inner, inner)))
    return out


from ._stats import median, nanmedian, nanpercentile, nanquantile, percentile, quantile  # noqa: E402  (they call `sort` of this module)
