"""Device-array thunk: the slice of the reference's `DeferredArray` that the sort path uses
(`cupynumeric/_thunk/deferred.py`: `sort` :5453-5474, `copy` :394-398, `swapaxes` :2341-2351,
`reshape` :2136-2316), over a dense row-major device buffer instead of a Legate store.
"""
from __future__ import annotations

import ctypes
from typing import TYPE_CHECKING, Any

import numpy as np

from . import _lib
from .runtime import runtime

if TYPE_CHECKING:
    import torch

# dtypes the reference supports (`cupynumeric/_utils/array.py:28-43`)
SUPPORTED_DTYPES = tuple(_lib.DTYPE_CODES.keys())


def check_dtype(dtype: Any) -> np.dtype:
    """Same error text as `to_core_type` (`cupynumeric/_utils/array.py:64-68`)."""
    try:
        dt = np.dtype(dtype)
    except TypeError:
        raise TypeError(f"cuPyNumeric does not support dtype={dtype}")
    if dt not in _lib.DTYPE_CODES:
        raise TypeError(f"cuPyNumeric does not support dtype={dt}")
    return dt


class Storage:
    """A dense device buffer.  Host data handed in at creation is uploaded on first device use,
    so that building an array does not need a GPU (Legate attaches host data lazily as well)."""

    def __init__(self, nbytes: int, host: np.ndarray | None = None) -> None:
        self.nbytes = int(nbytes)
        self._host = host
        self._dev: "torch.Tensor | None" = None

    def device(self) -> "torch.Tensor":
        if self._dev is None:
            if self._host is not None:
                self._dev = runtime.upload(self._host)
                self._host = None
            else:
                self._dev = runtime.empty_bytes(self.nbytes)
        return self._dev

    def ptr(self) -> int:
        return int(self.device().data_ptr())

    def to_numpy(self, shape: tuple[int, ...], dtype: np.dtype) -> np.ndarray:
        if 0 in shape:
            return np.empty(shape, dtype=dtype)  # nothing to fetch; works without a device
        if self._dev is None and self._host is not None:
            return np.array(self._host, dtype=dtype).reshape(shape)
        return runtime.download(self.device(), shape, dtype)


class DeviceArray:
    """Shape + dtype + `base` storage.  `base` can be re-bound, as the reference's sort helpers
    do with `output.base = result.base` (`cupynumeric/_thunk/_sort.py:47,73,76`)."""

    def __init__(self, shape: tuple[int, ...], dtype: Any, base: Storage | None = None) -> None:
        self.shape = tuple(int(s) for s in shape)
        self.dtype = check_dtype(dtype)
        self.base = base if base is not None else Storage(self.size * self.dtype.itemsize)

    @classmethod
    def from_numpy(cls, arr: np.ndarray) -> "DeviceArray":
        dt = check_dtype(arr.dtype)
        host = np.array(arr, dtype=dt, order="C", copy=True)
        return cls(host.shape, dt, Storage(host.nbytes, host=host))

    @classmethod
    def from_device(cls, buf: "torch.Tensor", shape: tuple[int, ...], dtype: Any) -> "DeviceArray":
        """An array over device memory that already holds its dense row-major data: `buf` is a
        contiguous torch tensor on the GPU (any element type) of exactly the array's bytes.  The
        memory is shared, not copied."""
        dt = check_dtype(dtype)
        raw = buf.reshape(-1).view(runtime.torch.uint8)
        out = cls(shape, dt, Storage(raw.numel()))
        if raw.numel() != out.size * dt.itemsize or not raw.is_cuda:
            raise ValueError("from_device: the buffer must be device memory of exactly shape x dtype bytes")
        out.base._dev = raw
        return out

    @property
    def ndim(self) -> int:
        return len(self.shape)

    @property
    def size(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    def __numpy_array__(self) -> np.ndarray:
        return self.base.to_numpy(self.shape, self.dtype)

    # -- data movement the sort path needs ------------------------------------------------
    def reshape(self, newshape: tuple[int, ...], order: str = "C") -> "DeviceArray":
        """C-order reshape.  Buffers are always dense row-major, so the storage is shared."""
        if order != "C":
            raise NotImplementedError("only C-order reshape is used by the sort path")
        out = DeviceArray(newshape, self.dtype, self.base)
        if out.size != self.size:
            raise ValueError("cannot reshape array: sizes differ")
        return out

    def copy(self) -> "DeviceArray":
        """Dense copy with storage of its own (`DeferredArray.copy(deep=True)`, `cupynumeric/_thunk/deferred.py:394-398`);
        host data that has not been uploaded yet is copied on the host."""
        if self.base._dev is None and self.base._host is not None:
            return DeviceArray.from_numpy(np.asarray(self.base._host).reshape(self.shape))
        sub = Storage(self.size * self.dtype.itemsize)
        if self.size:
            sub._dev = self.base.device()[: sub.nbytes].clone()
        return DeviceArray(self.shape, self.dtype, sub)

    def slice_first_axis(self, i: int, count: int, shape: tuple[int, ...]) -> "DeviceArray":
        """`self[i]` as an array of `shape` (`count` elements) over the same memory: rows of a
        dense row-major buffer are themselves dense."""
        nbytes = count * self.dtype.itemsize
        sub = Storage(nbytes)
        if self.base._dev is None and self.base._host is not None:
            host = np.asarray(self.base._host).reshape(self.shape)
            sub._host = np.ascontiguousarray(host[i])
        else:
            sub._dev = self.base.device()[i * nbytes : (i + 1) * nbytes] if nbytes else runtime.empty_bytes(0)
        return DeviceArray(shape, self.dtype, sub)

    def swapaxes_copy(self, axis1: int, axis2: int) -> "DeviceArray":
        """Dense copy with two axes exchanged: the reference's `swapaxes` view followed by
        `copy(deep=True)` (`cupynumeric/_thunk/_sort.py:59-65`) in one kernel."""
        shape = list(self.shape)
        shape[axis1], shape[axis2] = shape[axis2], shape[axis1]
        out = DeviceArray(tuple(shape), self.dtype)
        if self.size == 0:
            return out
        lib = _lib.load()
        c_shape = (ctypes.c_int64 * max(self.ndim, 1))(*self.shape)
        status = lib.cpn_swapaxes_copy(
            self.dtype.itemsize,
            self.base.ptr(),
            out.base.ptr(),
            c_shape,
            self.ndim,
            axis1,
            axis2,
            runtime.stream_handle(),
        )
        _lib.check(status, "cpn_swapaxes_copy")
        return out

    def take_along_last_axis(self, indices: "DeviceArray", check: str = "now") -> "DeviceArray":
        """`take_along_axis(self, indices, axis=-1)` for arrays whose leading dimensions agree
        (`cupynumeric/_module/indexing.py:648-760`; the TAKE task's no-broadcast case).

        `check`: what happens to the kernel's out-of-bounds flag.  "now": read back before returning
        (one stream synchronisation; the public `take_along_axis` raises IndexError from the call, as
        the reference does); "deferred": reported with the next host read (`runtime.flush_status`), so
        that the stream keeps running; "trusted": no flag at all, for indices that this package
        produced itself (the argsorts inside `lexsort`)."""
        if indices.dtype != np.dtype(np.int64):
            raise TypeError("`indices` must be an int64 array")
        if self.ndim != indices.ndim or self.ndim == 0:
            raise ValueError("`indices` and `a` must have the same number of dimensions")
        lead_a, lead_i = self.shape[:-1], indices.shape[:-1]
        if any(m != n and m != 1 and n != 1 for m, n in zip(lead_a, lead_i)):
            raise IndexError(
                "shape mismatch: indexing arrays could not be broadcast together with shapes "
                f"{self.shape} {indices.shape} (every dimension but the axis must agree or be 1)"
            )
        lead_out = tuple(max(m, n) if min(m, n) != 0 else 0 for m, n in zip(lead_a, lead_i))
        out = DeviceArray(lead_out + indices.shape[-1:], self.dtype)
        if out.size == 0:
            return out
        if self.shape[-1] == 0:
            raise IndexError("index out of bounds: cannot take from an empty axis")
        lib = _lib.load()
        if runtime.check_mode == "off":
            check = "trusted"
        elif runtime.check_mode == "eager" and check == "deferred":
            check = "now"
        flag = runtime.zero_flag() if check != "trusted" else None
        flag_ptr = flag.data_ptr() if flag is not None else None
        stream = ctypes.c_void_p(runtime.stream_handle())
        if lead_a == lead_i:
            status = lib.cpn_take_along_last_axis(
                self.dtype.itemsize, self.base.ptr(), indices.base.ptr(), out.base.ptr(), out.size // indices.shape[-1],
                self.shape[-1], indices.shape[-1], flag_ptr, stream,
            )
        else:
            # rows per step of each leading dimension on either side: the dense stride, 0 where broadcast
            def row_strides(lead: tuple[int, ...]) -> list[int]:
                strides, run = [0] * len(lead), 1
                for d in range(len(lead) - 1, -1, -1):
                    strides[d] = run if lead[d] != 1 else 0
                    run *= lead[d]
                return strides

            n = len(lead_out)
            u64 = ctypes.c_uint64 * max(n, 1)
            status = lib.cpn_take_along_last_axis_broadcast(
                self.dtype.itemsize, self.base.ptr(), indices.base.ptr(), out.base.ptr(), n, u64(*lead_out),
                u64(*row_strides(lead_a)), u64(*row_strides(lead_i)), self.shape[-1], indices.shape[-1], flag_ptr, stream,
            )
        _lib.check(status, "cpn_take_along_last_axis")
        if check == "deferred":
            runtime.defer_flag(flag, "index")
        elif check == "now":
            runtime.flush_status()  # (errors of earlier work first: the read below synchronises anyway)
            if int(flag.item()) != 0:
                raise IndexError("index out of bounds in take_along_axis")
        return out

    # -- the sort entry point ---------------------------------------------------------------
    def sort(
        self,
        rhs: "DeviceArray",
        argsort: bool = False,
        axis: int | None = -1,
        kind: str = "quicksort",
        order: str | list[str] | None = None,
    ) -> None:
        """`DeferredArray.sort` (`cupynumeric/_thunk/deferred.py:5453-5474`): `self` receives the
        result of sorting `rhs`."""
        from ._sort import sort_deferred

        # (messages and exception types are the reference's: callers and its tests match on them)
        if order is not None:
            raise NotImplementedError(
                "cuPyNumeric does not support sorting with 'order' as "
                "ndarray only supports numeric values"
            )
        if axis is not None and not -rhs.ndim <= axis < rhs.ndim:
            raise ValueError("invalid axis")
        # only "stable" sets the flag (any other kind, "mergesort" included, does not); every kernel
        # here is stable whatever the flag says
        sort_deferred(self, rhs, argsort, axis, stable=(kind == "stable"))

    def partition(
        self,
        rhs: "DeviceArray",
        kth: Any,
        argpartition: bool = False,
        axis: int | None = -1,
        kind: str = "introselect",
        order: str | list[str] | None = None,
    ) -> None:
        """`DeferredArray.partition` (`cupynumeric/_thunk/deferred.py:5476-5494`): falls back to an
        (unstable-flagged) sort, which satisfies the partition property for every `kth`."""
        from ._sort import sort_deferred

        if order is not None:
            raise NotImplementedError(
                "cuPyNumeric does not support partitioning with 'order' as "
                "ndarray only supports numeric values"
            )
        if axis is not None and not -rhs.ndim <= axis < rhs.ndim:
            raise ValueError("invalid axis")
        sort_deferred(self, rhs, argpartition, axis, False)  # a sorted row is partitioned at every kth

    def astype(self, dtype: Any) -> "DeviceArray":
        """Dense copy converted to `dtype` (`DeferredArray.convert`, `cupynumeric/_thunk/deferred.py:1899-1937`,
        a UNARY_OP convert task in the reference)."""
        dt = check_dtype(dtype)
        out = DeviceArray(self.shape, dt)
        if self.size == 0:
            return out
        lib = _lib.load()
        status = lib.cpn_astype(
            _lib.DTYPE_CODES[self.dtype],
            self.base.ptr(),
            _lib.DTYPE_CODES[dt],
            out.base.ptr(),
            self.size,
            ctypes.c_void_p(runtime.stream_handle()),
        )
        _lib.check(status, "cpn_astype")
        return out

    def searchsorted(self, rhs: "DeviceArray", v: "DeviceArray", side: str = "left") -> None:
        """`DeferredArray.searchsorted` (`cupynumeric/_thunk/deferred.py:5425-5451`): `self` (int64,
        shape of `v`) receives the insertion points of `v` into the sorted 1-D `rhs`.  Any
        `side` other than "left" means "right", as in the reference (`is_left = side == "left"`)."""
        is_left = side == "left"
        if v.size == 0:
            return
        if rhs.dtype != v.dtype or self.dtype != np.dtype(np.int64):
            raise TypeError("searchsorted: arrays must share one dtype and the result must be int64")
        lib = _lib.load()
        code = _lib.DTYPE_CODES[rhs.dtype]
        temp_bytes = lib.cpn_searchsorted_temp_bytes(code, rhs.size, v.size)
        temp = runtime.empty_bytes(temp_bytes) if temp_bytes else None
        stream = ctypes.c_void_p(runtime.stream_handle())
        status = lib.cpn_searchsorted(
            code,
            rhs.base.ptr() if rhs.size else None,
            rhs.size,
            v.base.ptr(),
            v.size,
            int(is_left),
            self.base.ptr(),
            temp.data_ptr() if temp is not None else None,
            temp_bytes,
            stream,
        )
        _lib.check(status, "cpn_searchsorted")
        if temp is not None and runtime.check_mode == "lazy":
            runtime.defer_status(temp)  # (the values were sorted first: that sort's status word)
        elif temp is not None and runtime.check_mode == "eager":
            _lib.check(lib.cpn_local_sort_check(temp.data_ptr(), stream), "cpn_searchsorted")

    def unique(self) -> "DeviceArray":
        """`DeferredArray.unique` (`cupynumeric/_thunk/deferred.py:5375-5395`): sorted distinct
        values of the flattened array.  The result size is only known on the device (an unbound
        store in the reference); reading it back is the one synchronisation of this call."""
        if self.size == 0:
            return DeviceArray((0,), self.dtype)
        lib = _lib.load()
        code = _lib.DTYPE_CODES[self.dtype]
        temp_bytes = lib.cpn_unique_temp_bytes(code, self.size)
        if temp_bytes == 0:
            raise NotImplementedError(f"cpn_unique: no workspace layout for dtype={self.dtype}, size={self.size}")
        temp = runtime.empty_bytes(temp_bytes)
        out = DeviceArray((self.size,), self.dtype)
        count = runtime.torch.zeros(1, dtype=runtime.torch.int64, device=runtime.require_device())
        stream = ctypes.c_void_p(runtime.stream_handle())
        status = lib.cpn_unique(
            code, self.base.ptr(), out.base.ptr(), self.size, count.data_ptr(), temp.data_ptr(), temp_bytes, stream
        )
        _lib.check(status, "cpn_unique")
        if runtime.check_mode != "off":  # (reading the count below synchronises anyway)
            runtime.flush_status()  # errors of earlier work first
            _lib.check(lib.cpn_local_sort_check(temp.data_ptr(), stream), "cpn_unique")
        n_unique = int(count.item())
        return DeviceArray((n_unique,), self.dtype, out.base)

    def to_complex(self, dtype: Any) -> "DeviceArray":
        """Real -> complex cast (`astype` in `sort_complex`, `cupynumeric/_module/ssc_sorting.py:150-159`)."""
        dt = check_dtype(dtype)
        out = DeviceArray(self.shape, dt)
        if self.size == 0:
            return out
        lib = _lib.load()
        status = lib.cpn_real_to_complex(
            _lib.DTYPE_CODES[self.dtype],
            self.base.ptr(),
            _lib.DTYPE_CODES[dt],
            out.base.ptr(),
            self.size,
            runtime.stream_handle(),
        )
        _lib.check(status, "cpn_real_to_complex")
        return out
