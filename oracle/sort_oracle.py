"""TEST INFRASTRUCTURE -- CPU oracle for the sort path.  Not part of the product: only tests/,
`__graft_entry__.smoke()` and `bench.py`'s `cpu_baseline` leg may import this module.

Two layers, mirroring the reference:

* `local_sort` calls the C restatement (`sort_oracle.c`) of `SortImplBodyCpu` /
  `thrust_local_sort_inplace` (`src/cupynumeric/sort/sort_cpu.inl:52-85,937-1074`): rows of the
  last axis, stable, NumPy ordering, indices `i % seg + offset`.
* `sort` / `argsort` restate the Python side: `cupynumeric/_module/ssc_sorting.py:29-121` (result
  shape and dtype), `DeferredArray.sort` (`cupynumeric/_thunk/deferred.py:5453-5474`: kind -> stable
  flag, `order` -> NotImplementedError, axis range -> ValueError) and the axis dispatch of
  `cupynumeric/_thunk/_sort.py:37-136` (flatten / last axis / swap-sort-swap), with NumPy doing the
  `swapaxes` copies.

* `lexsort` restates the loop of `cupynumeric/_module/ssc_sorting.py:271-444` over `argsort`
  above, with NumPy's `take_along_axis` between the steps.

* `searchsorted` restates `cupynumeric/_array/array.py:3700-3771` (common type, `sorter`) over the
  binary searches of `src/cupynumeric/sort/searchsorted.cc` (lower / upper bound per value);
  `unique` restates `src/cupynumeric/set/unique.cc:31-55` (copy, sort, drop repeated neighbours).
  Both use NumPy's order and equality (NaN last and equal to itself) where the reference's
  backends compare with `<` / `==`.

Deviation kept on purpose (same as the product): results are always stable.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np
from numpy.exceptions import AxisError
from numpy.lib.array_utils import normalize_axis_index

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "_build" / "libcpnoracle.so"

# same codes as enum cpn_dtype (include/cpn_sort.h)
DTYPE_CODES = {
    np.dtype(np.bool_): 0,
    np.dtype(np.int8): 1,
    np.dtype(np.int16): 2,
    np.dtype(np.int32): 3,
    np.dtype(np.int64): 4,
    np.dtype(np.uint8): 5,
    np.dtype(np.uint16): 6,
    np.dtype(np.uint32): 7,
    np.dtype(np.uint64): 8,
    np.dtype(np.float16): 9,
    np.dtype(np.float32): 10,
    np.dtype(np.float64): 11,
    np.dtype(np.complex64): 12,
    np.dtype(np.complex128): 13,
}

_lib = None


THRUST_LIB_PATH = HERE / "_build" / "libcpnthrust.so"
_thrust = None


def thrust_local_sort(x: np.ndarray, argsort: bool, stable: bool = True, use_omp: bool = False,
                      transparent: bool = False):
    """Baseline only (bench.py): the reference's CPU / OpenMP variant over rocThrust's host backends
    (thrust_baseline.cpp).  Copy + index initialisation as in `SortImplBodyCpu`
    (`src/cupynumeric/sort/sort_cpu.inl:974-1025`), then the per-row thrust calls, with the typed
    comparator `thrust::less<VAL>` (rocThrust's host radix sort) or, `transparent`, with
    `thrust::less<>` as the reference passes it (`sort_cpu.inl:62-83`; rocThrust's merge sort).
    Floats with NaN or -0.0 do not come out in NumPy's order either way."""
    global _thrust
    if _thrust is None:
        if not THRUST_LIB_PATH.exists():
            build()
        import torch  # noqa: F401  (its bundled HIP runtime must be the one the process binds, see Makefile)

        _thrust = ctypes.CDLL(str(THRUST_LIB_PATH))
        _thrust.cpn_thrust_local_sort.restype = ctypes.c_int
        _thrust.cpn_thrust_local_sort.argtypes = [
            ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int, ctypes.c_int,
            ctypes.c_int,
        ]
    x = np.ascontiguousarray(x)
    seg = x.shape[-1]
    values = x.copy()
    indices = None
    if argsort:
        indices = np.ascontiguousarray(np.broadcast_to(np.arange(seg, dtype=np.int64), x.shape))
    rc = _thrust.cpn_thrust_local_sort(
        DTYPE_CODES[x.dtype], values.ctypes.data, indices.ctypes.data if argsort else None, x.size, seg,
        int(stable), int(use_omp), int(transparent),
    )
    if rc != 0:
        raise RuntimeError(f"cpn_thrust_local_sort failed: {rc}")
    return indices if argsort else values


def build(force: bool = False) -> Path:
    """Compile sort_oracle.c with gcc and thrust_baseline.cpp with hipcc (see Makefile)."""
    sources = [HERE / "sort_oracle.c", HERE / "thrust_baseline.cpp"]
    stale = any(not lib.exists() or lib.stat().st_mtime < src.stat().st_mtime
                for lib, src in zip([LIB_PATH, THRUST_LIB_PATH], sources))
    if force or stale:
        subprocess.run(["make", "-C", str(HERE), "-B" if force else "-s"], check=True, capture_output=True)
    return LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        lib = ctypes.CDLL(str(LIB_PATH))
        lib.cpn_oracle_local_sort.restype = ctypes.c_int
        lib.cpn_oracle_local_sort.argtypes = [
            ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
            ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
        ]
        lib.cpn_oracle_max_threads.restype = ctypes.c_int
        _lib = lib
    return _lib


def max_threads() -> int:
    return int(load().cpn_oracle_max_threads())


def local_sort(x: np.ndarray, argsort: bool, stable: bool = True, offset: int = 0, threads: int = 1):
    """Sort the rows (last axis) of a C-contiguous array.  Returns sorted values, or int64 row
    positions when `argsort`."""
    x = np.ascontiguousarray(x)
    if x.dtype not in DTYPE_CODES:
        raise TypeError(f"cuPyNumeric does not support dtype={x.dtype}")
    values = np.empty_like(x)
    indices = np.empty(x.shape, dtype=np.int64) if argsort else None
    seg = x.shape[-1] if x.ndim > 0 else 1
    if x.size:
        rc = load().cpn_oracle_local_sort(
            DTYPE_CODES[x.dtype],
            x.ctypes.data,
            values.ctypes.data,
            indices.ctypes.data if argsort else None,
            x.size,
            seg,
            offset,
            int(stable),
            threads,
        )
        if rc != 0:
            raise RuntimeError(f"cpn_oracle_local_sort failed: {rc}")
    return indices if argsort else values


def _sort_deferred(x: np.ndarray, argsort: bool, axis, stable: bool, threads: int) -> np.ndarray:
    # cupynumeric/_thunk/_sort.py:110-136
    if x.ndim == 0:
        if axis is not None:
            raise AxisError(axis, x.ndim)
        return np.zeros(1, dtype=np.int64) if argsort else x.copy()
    if axis is None and x.ndim > 1:
        return _sort_deferred(x.reshape(-1), argsort, -1, stable, threads)  # sort_flattened :37-47
    computed_axis = 0 if axis is None else normalize_axis_index(axis, x.ndim)
    if computed_axis == x.ndim - 1:
        return local_sort(x, argsort, stable, 0, threads)  # sort_task :79-107
    # sort_swapped :50-76
    swapped_copy = np.ascontiguousarray(np.swapaxes(x, computed_axis, x.ndim - 1))
    res = local_sort(swapped_copy, argsort, stable, 0, threads)
    return np.ascontiguousarray(np.swapaxes(res, x.ndim - 1, computed_axis))


def _thunk_sort(x: np.ndarray, argsort: bool, axis, kind: str, order, threads: int) -> np.ndarray:
    # cupynumeric/_thunk/deferred.py:5453-5474
    stable = kind == "stable"
    if order is not None:
        raise NotImplementedError(
            "cuPyNumeric does not support sorting with 'order' as ndarray only supports numeric values"
        )
    if axis is not None and (axis >= x.ndim or axis < -x.ndim):
        raise ValueError("invalid axis")
    return _sort_deferred(x, argsort, axis, stable, threads)


def sort(a, axis=-1, kind="quicksort", order=None, threads: int = 1) -> np.ndarray:
    x = np.asarray(a)
    if x.dtype not in DTYPE_CODES:
        raise TypeError(f"cuPyNumeric does not support dtype={x.dtype}")
    return _thunk_sort(x, False, axis, kind, order, threads)


def argsort(a, axis=-1, kind="quicksort", order=None, threads: int = 1) -> np.ndarray:
    x = np.asarray(a)
    if x.dtype not in DTYPE_CODES:
        raise TypeError(f"cuPyNumeric does not support dtype={x.dtype}")
    return _thunk_sort(x, True, axis, kind, order, threads)


def sort_complex(a, threads: int = 1) -> np.ndarray:
    """`cupynumeric/_module/ssc_sorting.py:124-159`: sort along the last axis, then force a complex
    result: complex input keeps its type, integers of at most 16 bits become complex64, everything
    else complex128."""
    result = sort(a, threads=threads)
    if np.issubdtype(result.dtype, np.complexfloating):
        return result
    if np.issubdtype(result.dtype, np.integer) and result.dtype.itemsize <= 2:
        return result.astype(np.complex64)
    return result.astype(np.complex128)


def lexsort(keys, axis=-1, threads: int = 1) -> np.ndarray:
    """`cupynumeric/_module/ssc_sorting.py:271-444`: validation, then a stable argsort of the first
    key and, for every further key, reorder / argsort / reorder.  Keys keep their own element
    type; the oracle's ordering already is -inf < finite < +inf < NaN, which is what the
    reference's remapping of special values (:352-420) establishes before it sorts."""
    if keys is None:
        raise TypeError("'NoneType' object is not iterable")
    if axis is None:
        raise TypeError("'NoneType' object cannot be interpreted as an integer")
    if isinstance(keys, np.ndarray):
        if keys.ndim == 0:
            raise TypeError("need sequence of keys with len > 0 in lexsort")
        key_list = [keys[i] for i in range(keys.shape[0])]
    else:
        key_list = [np.asarray(k) for k in keys]
    if len(key_list) == 0:
        raise TypeError("Need at least one key to sort")
    for k in key_list:
        if k.dtype not in DTYPE_CODES:
            raise TypeError(f"cuPyNumeric does not support dtype={k.dtype}")
    first_shape = key_list[0].shape
    for i, key in enumerate(key_list[1:], 1):
        if key.shape != first_shape:
            raise ValueError(
                f"All keys must have the same shape. Key {i} has shape {key.shape}, expected {first_shape}"
            )
    if key_list[0].ndim == 0:
        return np.zeros((), dtype=np.int64)
    ndim = key_list[0].ndim
    if axis >= ndim or axis < -ndim:
        raise AxisError(f"axis {axis} is out of bounds for array of dimension {ndim}")
    if key_list[0].size == 0:
        return np.empty(first_shape, dtype=np.int64)
    indices = argsort(key_list[0], axis=axis, kind="stable", threads=threads)
    for key in key_list[1:]:
        key_reordered = np.take_along_axis(key, indices, axis=axis)
        order = argsort(key_reordered, axis=axis, kind="stable", threads=threads)
        indices = np.take_along_axis(indices, order, axis=axis)
    return indices


def _less(a, b) -> bool:
    """NumPy's sort order for one pair of scalars (npysort_common.h: FLOAT_LT, CFLOAT_LT)."""
    if isinstance(a, (complex, np.complexfloating)):
        ar, ai, br, bi = a.real, a.imag, b.real, b.imag
        if ar < br:
            return ai == ai or bi != bi
        if ar > br:
            return bi != bi and ai == ai
        if ar == br or (ar != ar and br != br):
            return ai < bi or (bi != bi and ai == ai)
        return br != br
    if isinstance(a, (float, np.floating)):
        return bool(a < b or (b != b and a == a))
    return bool(a < b)


def searchsorted(a, v, side="left", sorter=None) -> np.ndarray:
    """`ndarray.searchsorted` (`cupynumeric/_array/array.py:3737-3771`) with one binary search per
    value (`src/cupynumeric/sort/searchsorted.cc:45-70`: std::lower_bound / std::upper_bound).
    Pure-Python loops: for small inputs."""
    a = np.asarray(a)
    if a.ndim != 1:
        raise ValueError("Dimension mismatch: self must be a 1D array")
    v = np.asarray(v)
    for x in (a, v):
        if x.dtype not in DTYPE_CODES:
            raise TypeError(f"cuPyNumeric does not support dtype={x.dtype}")
    if a.dtype != v.dtype:
        ch_dtype = np.result_type(a.dtype, v.dtype)
        v = v.astype(ch_dtype)
        a = a.astype(ch_dtype)
    if sorter is not None and a.shape[0] > 1:
        sorter = np.asarray(sorter)
        if sorter.ndim != 1:
            raise ValueError("Dimension mismatch: sorter must be a 1D array")
        if sorter.shape != a.shape:
            raise ValueError("Shape mismatch: sorter must have the same shape as self")
        if not np.issubdtype(sorter.dtype, np.integer):
            raise ValueError("Dtype mismatch: sorter must be of integer type")
        a = a.take(sorter).copy()
    is_left = side == "left"
    out = np.empty(v.shape, dtype=np.int64)
    flat_v = v.reshape(-1)
    flat_o = out.reshape(-1)
    for i in range(flat_v.size):
        x = flat_v[i]
        lo, hi = 0, a.shape[0]
        while lo < hi:
            mid = (lo + hi) // 2
            right = _less(a[mid], x) if is_left else not _less(x, a[mid])
            if right:
                lo = mid + 1
            else:
                hi = mid
        flat_o[i] = lo
    return out


def unique(ar, threads: int = 1) -> np.ndarray:
    """`UniqueImplBody<CPU>` (`src/cupynumeric/set/unique.cc:31-55`): flatten, sort, keep the first
    of every run of equal neighbours.  Equality is NumPy's for `unique`: NaNs are equal, complex
    numbers with a NaN part are all equal."""
    x = np.asarray(ar)
    if x.dtype not in DTYPE_CODES:
        raise TypeError(f"cuPyNumeric does not support dtype={x.dtype}")
    flat = np.ascontiguousarray(x.reshape(-1))
    if flat.size == 0:
        return flat.copy()
    s = local_sort(flat, argsort=False, stable=True, threads=threads)
    with np.errstate(invalid="ignore"):
        differ = s[1:] != s[:-1]
    if s.dtype.kind in "fc":
        nan = np.isnan(s)
        differ &= ~(nan[1:] & nan[:-1])
    keep = np.concatenate(([True], differ))
    return s[keep]


# ---- order statistics on top of the sort (`cupynumeric/_module/stats_order.py`) -------------------------
_DESIRED_MOD_2 = int(np.lib.NumpyVersion(np.__version__) < "2.0.1")  # `stats_order.py:126`


def _quantile_position(method: str, q: float, n: int):
    """`stats_order.py:106-232`: (gamma, 0-based left position) of the thirteen estimators; gamma None
    means the method picks a sample."""
    import math

    if method == "inverted_cdf":
        pos = q * n
        left = int(pos)
        return (1.0 if pos - left > 0 else 0.0, left - 1)
    if method == "averaged_inverted_cdf":
        pos = q * n
        left = int(pos)
        return (1.0 if pos - left > 0 else 0.5, left - 1)
    if method == "closest_observation":
        pos = q * n - 0.5
        left = int(pos)
        gamma = 1 if (left != pos or left % 2 != _DESIRED_MOD_2) else 0
        return (None, left - 1 + gamma)
    one_based = {
        "interpolated_inverted_cdf": lambda: q * n,
        "hazen": lambda: q * n + 0.5,
        "weibull": lambda: q * (n + 1),
        "linear": lambda: q * (n - 1) + 1,
        "median_unbiased": lambda: q * (n + 1.0 / 3.0) + 1.0 / 3.0,
        "normal_unbiased": lambda: q * (n + 0.25) + 3.0 / 8.0,
    }
    if method in one_based:
        pos = one_based[method]()
        left = int(pos)
        return (pos - left, left - 1)
    pos = q * (n - 1)
    if method == "lower":
        return (None, int(pos))
    if method == "higher":
        return (None, int(math.ceil(pos)))
    if method == "midpoint":
        left = int(pos)
        return (0.5 if pos != left else 0.0, left)
    if method == "nearest":
        return (None, int(np.round(pos)))
    raise KeyError(method)


def quantile(a, q, axis=None, method: str = "linear", keepdims: bool = False, threads: int = 1) -> np.ndarray:
    """`stats_order.py:358-536` with `_quantile_impl` (`:249-337`) and `_reshuffle_reshape` (`:51-85`):
    sort along the (merged) axis with the oracle's sort, then per quantile the sample at `left`, or
    `(1.0 - gamma) * left_samples + gamma * right_samples` in NumPy's own arithmetic (a Python float
    times an array keeps a float array's type and makes integers float64), assigned into an array of the
    result type.  `out` and `overwrite_input` change no value and are left out."""
    x = np.asarray(a)
    original_shape = x.shape
    axes_set = ()
    if axis is not None and not np.isscalar(axis):
        axes_set = tuple(int(ax) % x.ndim for ax in axis)
        if len(axes_set) == 1:
            real_axis, x_rr = axes_set[0], x
        else:
            wanted = sorted(axes_set)
            first = wanted[0]
            moved = np.moveaxis(x, wanted, range(first, first + len(wanted)))
            merged = int(np.prod(moved.shape[first : first + len(wanted)], dtype=np.int64))
            x_rr = np.ascontiguousarray(moved).reshape(moved.shape[:first] + (merged,) + moved.shape[first + len(wanted) :])
            real_axis = first
    else:
        real_axis, x_rr = axis, x
        if real_axis is not None:
            axes_set = (int(real_axis) % x.ndim,)
            real_axis = axes_set[0]
    q_arr = np.asarray(q)
    arr = sort(x_rr, axis=real_axis, threads=threads)
    if arr.dtype.kind == "c":
        raise TypeError("input array cannot be of complex type")
    to_dtype = arr.dtype if method in ("inverted_cdf", "closest_observation", "lower", "higher", "nearest") else np.dtype(np.float64)
    if real_axis is None:
        n = arr.size
        remaining = (1,) * len(original_shape) if keepdims else ()
    else:
        n = arr.shape[real_axis]
        if keepdims:
            remaining = tuple(1 if k in axes_set else original_shape[k] for k in range(len(original_shape)))
        else:
            remaining = tuple(arr.shape[k] for k in range(arr.ndim) if k != real_axis)
    res = np.zeros((*q_arr.shape, *remaining), dtype=to_dtype)
    for index, qv in np.ndenumerate(q_arr):
        gamma, left = _quantile_position(method, float(qv), n)
        right = left + 1
        if left >= n - 1:
            left = right = n - 1
        elif left < 0:
            left = right = 0
        if gamma is None:
            res[index] = arr.take(left, real_axis).reshape(remaining)
        else:
            lvals = arr.take(left, real_axis).reshape(remaining)
            rvals = arr.take(right, real_axis).reshape(remaining)
            with np.errstate(invalid="ignore", over="ignore"):
                res[index] = ((1.0 - gamma) * lvals + gamma * rvals).astype(to_dtype)
    return res


def percentile(a, q, axis=None, method: str = "linear", keepdims: bool = False, threads: int = 1) -> np.ndarray:
    """`stats_order.py:540-650`."""
    return quantile(a, np.asarray(q) / 100.0, axis, method=method, keepdims=keepdims, threads=threads)


def median(a, axis=None, keepdims: bool = False, threads: int = 1) -> np.ndarray:
    """`cupynumeric/_module/stats_avgs_vars.py:373-443`."""
    return quantile(a, 0.5, axis=axis, method="midpoint", keepdims=keepdims, threads=threads)


def nanquantile(a, q, axis=None, method: str = "linear", keepdims: bool = False, threads: int = 1) -> np.ndarray:
    """`stats_order.py:763-951` with `nanquantile_impl` (`:653-760`): count the elements of every slice
    that are not NaN, replace the NaNs by the largest finite value of the type, sort, and per quantile
    and slice take the position that the estimator gives for that count; weights, `1 - weights`, the
    two products and the sum are arrays of the input's type (`:708-710,748-757`).  A slice with no
    element left gives NaN.  With `axis=None` the input is flattened first (NumPy's meaning of it)."""
    x = np.asarray(a)
    original_shape = x.shape
    axes_set = ()
    if axis is not None and not np.isscalar(axis):
        axes_set = tuple(int(ax) % x.ndim for ax in axis)
        if len(axes_set) == 1:
            real_axis, x_rr = axes_set[0], x
        else:
            wanted = sorted(axes_set)
            first = wanted[0]
            moved = np.moveaxis(x, wanted, range(first, first + len(wanted)))
            merged = int(np.prod(moved.shape[first : first + len(wanted)], dtype=np.int64))
            x_rr = np.ascontiguousarray(moved).reshape(moved.shape[:first] + (merged,) + moved.shape[first + len(wanted) :])
            real_axis = first
    else:
        real_axis, x_rr = axis, x
        if real_axis is not None:
            axes_set = (int(real_axis) % x.ndim,)
            real_axis = axes_set[0]
    if x_rr.dtype.kind == "c":
        raise TypeError("input array cannot be of complex type")
    if real_axis is None:
        x_rr, real_axis, flat = x_rr.reshape(-1), 0, True
    else:
        flat = False
    counts = np.count_nonzero(~np.isnan(x_rr), axis=real_axis)
    q_arr = np.asarray(q)
    arr = sort(np.where(np.isnan(x_rr), np.finfo(x_rr.dtype).max, x_rr), axis=real_axis, threads=threads)
    to_dtype = arr.dtype if method in ("inverted_cdf", "closest_observation", "lower", "higher", "nearest") else np.dtype(np.float64)
    plain = tuple(arr.shape[k] for k in range(arr.ndim) if k != real_axis)
    if keepdims:
        remaining = (1,) * len(original_shape) if flat else tuple(
            1 if k in axes_set else original_shape[k] for k in range(len(original_shape)))
    else:
        remaining = plain
    res = np.zeros((*q_arr.shape, *remaining), dtype=to_dtype)
    gammas = np.zeros(plain, dtype=arr.dtype)
    lvals = np.zeros(plain, dtype=arr.dtype)
    rvals = np.zeros(plain, dtype=arr.dtype)
    for qindex, qv in np.ndenumerate(q_arr):
        gamma = None
        for aindex, n in np.ndenumerate(counts):
            n = int(n)
            if n == 0:
                lvals[aindex] = np.nan
                rvals[aindex] = np.nan
                continue
            gamma, left = _quantile_position(method, float(qv), n)
            right = left + 1
            if left >= n - 1:
                left = right = n - 1
            elif left < 0:
                left = right = 0
            lvals[aindex] = arr[(*aindex[:real_axis], left, *aindex[real_axis:])]
            if gamma is not None:
                gammas[aindex] = gamma
                rvals[aindex] = arr[(*aindex[:real_axis], right, *aindex[real_axis:])]
        with np.errstate(invalid="ignore", over="ignore"):
            if gamma is None:
                res[qindex] = lvals.reshape(remaining)
            else:
                res[qindex] = ((1 - gammas) * lvals + gammas * rvals).reshape(remaining)
    return res


def nanpercentile(a, q, axis=None, method: str = "linear", keepdims: bool = False, threads: int = 1) -> np.ndarray:
    """`stats_order.py:954-1080`."""
    return nanquantile(a, np.asarray(q) / 100.0, axis, method=method, keepdims=keepdims, threads=threads)


def nanmedian(a, axis=None, keepdims: bool = False, threads: int = 1) -> np.ndarray:
    """`cupynumeric/_module/stats_avgs_vars.py:445-512`."""
    return nanquantile(a, 0.5, axis=axis, method="midpoint", keepdims=keepdims, threads=threads)
