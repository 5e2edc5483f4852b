"""`ndarray`: the part of `cupynumeric/_array/array.py` that the sort path and its tests use
(`sort` :3773-3796, `argsort` :3798-3824, `__array__` :820-832, shape/dtype accessors).
"""
from __future__ import annotations

from typing import Any

import numpy as np

from ._thunk import DeviceArray, check_dtype


def convert_to_ndarray(obj: Any) -> "ndarray":
    """What `@add_boilerplate` does to array-like arguments (`cupynumeric/_array/util.py:115-182`)."""
    if isinstance(obj, ndarray):
        return obj
    host = np.asarray(obj)
    check_dtype(host.dtype)
    return ndarray(host.shape, host.dtype, thunk=DeviceArray.from_numpy(host))


class ndarray:
    def __init__(self, shape: Any, dtype: Any = np.float64, thunk: DeviceArray | None = None) -> None:
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        dtype = check_dtype(dtype)
        self._thunk = thunk if thunk is not None else DeviceArray(tuple(shape), dtype)
        self._writeable = True

    # -- metadata -----------------------------------------------------------------------------
    @property
    def shape(self) -> tuple[int, ...]:
        return self._thunk.shape

    @property
    def ndim(self) -> int:
        return self._thunk.ndim

    @property
    def dtype(self) -> np.dtype:
        return self._thunk.dtype

    @property
    def size(self) -> int:
        return self._thunk.size

    @property
    def itemsize(self) -> int:
        return self._thunk.dtype.itemsize

    @property
    def nbytes(self) -> int:
        return self.size * self.itemsize

    def __len__(self) -> int:
        if self.ndim == 0:
            raise TypeError("len() of unsized object")
        return self.shape[0]

    def __repr__(self) -> str:
        return f"cupynumeric_amd.ndarray(shape={self.shape}, dtype={self.dtype})"

    # -- host interop -------------------------------------------------------------------------
    def __array__(self, dtype: Any = None, copy: bool | None = None) -> np.ndarray:
        out = self._thunk.__numpy_array__()
        if dtype is not None and np.dtype(dtype) != out.dtype:
            out = out.astype(dtype)
        return out

    def __getitem__(self, key: Any) -> "ndarray":
        """`a[indices]` for a 1-D array and a 1-D integer array of positions (a cuPyNumeric or NumPy
        array, or a list), negative positions counting from the end: the indexing that the reference's
        sort tests apply to `argsort` results (`tests/integration/test_argsort.py:243-245`; advanced
        indexing in the reference, `cupynumeric/_array/array.py:1236-1263`).  A position out of range
        raises IndexError when data next reaches the host, not from this call, so that the stream
        keeps running.  Other kinds of index are not provided."""
        if isinstance(key, list):
            key = np.asarray(key, dtype=np.int64) if len(key) == 0 else np.asarray(key)
        if isinstance(key, np.ndarray):
            key = convert_to_ndarray(key)
        if not isinstance(key, ndarray) or key.ndim != 1 or self.ndim != 1 or not np.issubdtype(key.dtype, np.integer):
            raise NotImplementedError(
                "only a[indices] with a 1-D integer index array on a 1-D array is provided by this package"
            )
        return self.take_1d(key)

    def flatten(self, order: str = "C") -> "ndarray":
        """Dense 1-D copy (C order)."""
        if order not in ("C", "K", "A"):
            raise NotImplementedError("only C-order flatten is supported")
        thunk = self._thunk.copy().reshape((self.size,))
        return ndarray(thunk.shape, thunk.dtype, thunk=thunk)

    def reshape(self, *shape: Any, order: str = "C") -> "ndarray":
        """View of the same dense storage under another shape (`cupynumeric/_array/array.py:3222-3283`;
        C order only, one dimension may be -1)."""
        if order not in ("C", "A"):
            raise NotImplementedError("only C-order reshape is supported")
        if len(shape) == 1 and not isinstance(shape[0], (int, np.integer)):
            shape = tuple(shape[0])
        dims = [int(d) for d in shape]
        if dims.count(-1) > 1:
            raise ValueError("can only specify one unknown dimension")
        if -1 in dims:
            known = int(np.prod([d for d in dims if d != -1], dtype=np.int64))
            if known == 0 or self.size % known != 0:
                raise ValueError(f"cannot reshape array of size {self.size} into shape {tuple(dims)}")
            dims[dims.index(-1)] = self.size // known
        if int(np.prod(dims, dtype=np.int64)) != self.size or any(d < 0 for d in dims):
            raise ValueError(f"cannot reshape array of size {self.size} into shape {tuple(dims)}")
        thunk = self._thunk.reshape(tuple(dims))
        return ndarray(thunk.shape, thunk.dtype, thunk=thunk)

    def setflags(self, write: bool | None = None) -> None:
        if write is not None:
            self._writeable = bool(write)

    # -- sorting ------------------------------------------------------------------------------
    def sort(self, axis: Any = -1, kind: str = "quicksort", order: Any = None) -> None:
        """a.sort(axis=-1, kind=None, order=None): sort in place
        (`cupynumeric/_array/array.py:3773-3796`)."""
        if not self._writeable:
            raise ValueError("array is not writeable")
        self._thunk.sort(rhs=self._thunk, axis=axis, kind=kind, order=order)
        _adopt_shape(self, self, axis)

    def argsort(self, axis: Any = -1, kind: str = "quicksort", order: Any = None) -> "ndarray":
        """a.argsort(axis=-1, kind=None, order=None) (`cupynumeric/_array/array.py:3798-3824`)."""
        result = ndarray(self.shape, np.int64)
        result._thunk.sort(rhs=self._thunk, argsort=True, axis=axis, kind=kind, order=order)
        _adopt_shape(result, self, axis)
        return result


    def partition(self, kth: Any, axis: Any = -1, kind: str = "introselect", order: Any = None) -> None:
        """a.partition(kth, axis=-1, kind='introselect', order=None): in place
        (`cupynumeric/_array/array.py:3441-3467`)."""
        if not self._writeable:
            raise ValueError("array is not writeable")
        self._thunk.partition(rhs=self._thunk, kth=kth, axis=axis, kind=kind, order=order)
        _adopt_shape(self, self, axis)

    def argpartition(self, kth: Any, axis: Any = -1, kind: str = "introselect", order: Any = None) -> "ndarray":
        """a.argpartition(kth, axis=-1, kind='introselect', order=None)
        (`cupynumeric/_array/array.py:3469-3501`)."""
        result = ndarray(self.shape, np.int64)
        result._thunk.partition(rhs=self._thunk, argpartition=True, kth=kth, axis=axis, kind=kind, order=order)
        _adopt_shape(result, self, axis)
        return result

    def astype(self, dtype: Any) -> "ndarray":
        """Copy of the array cast to `dtype` (`cupynumeric/_array/array.py:2277-2343`, default casting)."""
        dtype = check_dtype(dtype)
        if dtype == self.dtype:
            return self
        thunk = self._thunk.astype(dtype)
        return ndarray(thunk.shape, thunk.dtype, thunk=thunk)

    def take_1d(self, indices: "ndarray") -> "ndarray":
        """`a.take(indices)` for 1-D `a` and 1-D integer `indices`: what `searchsorted` does with
        its `sorter` (`cupynumeric/_array/array.py:3766`)."""
        idx = indices if indices.dtype == np.dtype(np.int64) else indices.astype(np.int64)
        thunk = self._thunk.take_along_last_axis(idx._thunk, check="deferred")
        return ndarray(thunk.shape, thunk.dtype, thunk=thunk)

    def searchsorted(self, v: Any, side: str = "left", sorter: Any = None) -> "ndarray":
        """a.searchsorted(v, side='left', sorter=None) (`cupynumeric/_array/array.py:3700-3771`):
        insertion points of `v` into the sorted 1-D array; int64, shape of `v`."""
        if self.ndim != 1:
            raise ValueError("Dimension mismatch: self must be a 1D array")

        # this is needed in case v is a scalar
        v_ndarray = convert_to_ndarray(v)

        a = self
        # in case we have different dtypes we need to find a common type
        if a.dtype != v_ndarray.dtype:
            ch_dtype = np.result_type(a.dtype, v_ndarray.dtype)

            if v_ndarray.dtype != ch_dtype:
                v_ndarray = v_ndarray.astype(ch_dtype)
            if a.dtype != ch_dtype:
                a = a.astype(ch_dtype)

        if sorter is not None and a.shape[0] > 1:
            sorter = convert_to_ndarray(sorter)
            if sorter.ndim != 1:
                raise ValueError("Dimension mismatch: sorter must be a 1D array")
            if sorter.shape != a.shape:
                raise ValueError("Shape mismatch: sorter must have the same shape as self")
            if not np.issubdtype(sorter.dtype, np.integer):
                raise ValueError("Dtype mismatch: sorter must be of integer type")
            a = a.take_1d(sorter)

        result = ndarray(v_ndarray.shape, np.int64)
        result._thunk.searchsorted(a._thunk, v_ndarray._thunk, side)
        return result

    def unique(self) -> "ndarray":
        """a.unique(): sorted distinct values of the flattened array (`cupynumeric/_array/array.py:4208-4227`)."""
        thunk = self._thunk.unique()
        return ndarray(thunk.shape, thunk.dtype, thunk=thunk)

    def astype_complex(self, dtype: Any) -> "ndarray":
        """Real -> complex64/complex128 copy (the cast `sort_complex` needs)."""
        thunk = self._thunk.to_complex(dtype)
        return ndarray(thunk.shape, thunk.dtype, thunk=thunk)


def _adopt_shape(result: ndarray, source: ndarray, axis: Any) -> None:
    """Results of `axis=None` sorts are flat; nothing else changes shape."""
    if axis is None and source.ndim > 1:
        result._thunk.shape = (source.size,)
