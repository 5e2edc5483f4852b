"""Order statistics that sit on top of the sort: `quantile`, `percentile`, `median` and the
variants that ignore NaNs, `nanquantile`, `nanpercentile`, `nanmedian`.

The reference sorts along the requested axis and then, for every quantile, takes the elements
at one or two positions of that axis and combines them (`cupynumeric/_module/stats_order.py:358-650`,
`cupynumeric/_module/stats_avgs_vars.py:373-443`).  Here the sort is the HIP sort of this
package and everything after it is one `cpn_quantile_sorted` launch for all quantiles.
"""
from __future__ import annotations

import ctypes
import math
from collections.abc import Iterable
from typing import Any

import numpy as np

from . import _lib
from ._array import convert_to_ndarray, ndarray
from ._thunk import DeviceArray
from .runtime import runtime

# `numpy.quantile`'s rule for exact ties of 'closest_observation' changed in NumPy 2.0.1; the
# reference follows the NumPy it runs with (`stats_order.py:126`)
_DESIRED_MOD_2 = int(np.lib.NumpyVersion(np.__version__) < "2.0.1")


def _position(method: str, q: float, n: int) -> tuple[float | None, int]:
    """(gamma, left): weight of the right neighbour (None: no interpolation) and 0-based position of the
    left one, for quantile `q` of `n` sorted samples.  The thirteen estimators of
    `stats_order.py:106-232`, with the virtual position `pos` evaluated exactly as there (the
    floating-point value of gamma depends on the order of the operations)."""
    if method in ("inverted_cdf", "averaged_inverted_cdf", "interpolated_inverted_cdf"):
        pos = q * n
        left = int(pos)
        g = pos - left
        if method == "inverted_cdf":
            return (1.0 if g > 0 else 0.0, left - 1)
        if method == "averaged_inverted_cdf":
            return (1.0 if g > 0 else 0.5, left - 1)
        return (g, left - 1)
    if method == "closest_observation":
        pos = q * n - 0.5
        left = int(pos)
        # the next sample unless the position is hit exactly; then round half to even
        step = 1 if (left != pos or left % 2 != _DESIRED_MOD_2) else 0
        return (None, left - 1 + step)
    if method in ("hazen", "weibull", "linear", "median_unbiased", "normal_unbiased"):
        if method == "hazen":
            pos = q * n + 0.5
        elif method == "weibull":
            pos = q * (n + 1)
        elif method == "linear":
            pos = q * (n - 1) + 1
        elif method == "median_unbiased":
            fract = 1.0 / 3.0
            pos = q * (n + fract) + fract
        else:
            pos = q * (n + 0.25) + 3.0 / 8.0
        left = int(pos)
        return (pos - left, left - 1)
    pos = q * (n - 1)  # the four variants of 'linear' count positions from 0
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


METHODS = (
    "inverted_cdf", "averaged_inverted_cdf", "closest_observation", "interpolated_inverted_cdf", "hazen", "weibull",
    "linear", "median_unbiased", "normal_unbiased", "lower", "higher", "midpoint", "nearest",
)
# the result keeps the input's type (`stats_order.py:501-510`); every other method gives float64
_KEEP_DTYPE = ("inverted_cdf", "closest_observation", "lower", "higher", "nearest")


def _normalize_axes(axis: Any, ndim: int) -> tuple[int, ...]:
    axes = tuple(axis) if isinstance(axis, Iterable) else (axis,)
    out = []
    for ax in axes:
        ax = int(ax)
        if not -ndim <= ax < ndim:
            raise np.exceptions.AxisError(ax, ndim)
        out.append(ax % ndim)
    if len(set(out)) != len(out):
        raise ValueError("repeated axis")
    return tuple(out)


def _collapse_axes(a: ndarray, axes: tuple[int, ...]) -> tuple[int, ndarray]:
    """Brings the axes of `axes` together at the position of the smallest one and merges them into one
    (`_reshuffle_reshape`, `stats_order.py:51-85`): returns (that position, the reshaped array)."""
    wanted = sorted(axes)
    first, count = wanted[0], len(wanted)
    thunk = a._thunk
    # moveaxis(arr, wanted, range(first, first + count)) as successive exchanges of two axes
    order = list(range(a.ndim))
    target = [ax for ax in order if ax not in wanted]
    target[first:first] = wanted
    for dst in range(a.ndim):
        src = order.index(target[dst])
        if src != dst:
            thunk = thunk.swapaxes_copy(dst, src)
            order[dst], order[src] = order[src], order[dst]
    shape = thunk.shape
    merged = int(np.prod(shape[first : first + count], dtype=np.int64))
    thunk = thunk.reshape(shape[:first] + (merged,) + shape[first + count :])
    return first, ndarray(thunk.shape, thunk.dtype, thunk=thunk)


def quantile(
    a: Any,
    q: Any,
    axis: Any = None,
    out: ndarray | None = None,
    overwrite_input: bool = False,
    method: str = "linear",
    keepdims: bool = False,
) -> ndarray:
    """q-th quantile(s) of the data along the given axis or axes (`stats_order.py:358-536`).

    The result has shape `q.shape + (shape of a without the reduced axes)`; its type is float64
    unless the method only picks samples ('inverted_cdf', 'closest_observation', 'lower', 'higher',
    'nearest'), which keep the input's type.  Complex input raises TypeError.
    """
    a = convert_to_ndarray(a)
    original_shape = a.shape
    axes_set: tuple[int, ...] = ()
    if axis is not None and isinstance(axis, Iterable):
        axes_set = _normalize_axes(axis, a.ndim)
        if len(axes_set) == 1:
            real_axis, a_rr = axes_set[0], a
        else:
            real_axis, a_rr = _collapse_axes(a, axes_set)
            overwrite_input = False  # (the merged copy is sorted, not the caller's array)
    else:
        real_axis, a_rr = axis, a
        if real_axis is not None:
            axes_set = _normalize_axes(real_axis, a.ndim)
            real_axis = axes_set[0]
    if method not in METHODS:
        raise KeyError(method)
    q_arr = np.asarray(q)

    from . import sort  # (the module-level function; imported here to keep the import order free)

    if overwrite_input:
        a_rr.sort(axis=real_axis)
        arr = a_rr
    else:
        arr = sort(a_rr, axis=real_axis)
    if arr.dtype.kind == "c":
        raise TypeError("input array cannot be of complex type")
    to_dtype = arr.dtype if method in _KEEP_DTYPE else np.dtype(np.float64)

    # sort() with axis=None flattens: the quantile then runs over the one axis of the flat array
    if real_axis is None:
        n, outer, inner = arr.size, 1, 1
        remaining = (1,) * len(original_shape) if keepdims else ()
    else:
        n = arr.shape[real_axis]
        outer = int(np.prod(arr.shape[:real_axis], dtype=np.int64))
        inner = int(np.prod(arr.shape[real_axis + 1 :], dtype=np.int64))
        if keepdims:
            remaining = tuple(1 if k in axes_set else original_shape[k] for k in range(len(original_shape)))
        else:
            remaining = tuple(arr.shape[k] for k in range(arr.ndim) if k != real_axis)
    result_shape = (*q_arr.shape, *remaining)
    if out is not None and out.shape != result_shape:
        raise ValueError("wrong shape on output array")
    if n == 0:
        raise IndexError("index out of bounds: quantile of an empty axis")

    # positions and weights of every quantile, clipped into the axis (`stats_order.py:310-321`)
    left = np.empty(q_arr.size, dtype=np.int64)
    right = np.empty(q_arr.size, dtype=np.int64)
    gamma = np.zeros(q_arr.size, dtype=np.float64)
    interpolate = True
    for k, qv in enumerate(q_arr.reshape(-1)):
        g, lpos = _position(method, float(qv), n)
        rpos = lpos + 1
        if lpos >= n - 1:
            lpos = rpos = n - 1
        elif lpos < 0:
            lpos = rpos = 0
        left[k], right[k] = lpos, rpos
        if g is None:
            interpolate = False
        else:
            gamma[k] = g

    # the weighted sum is float64 whatever the method ('inverted_cdf' has weights 0 and 1 and assigns
    # the sum to an array of the input's type: the conversion below)
    computed = np.dtype(np.float64) if interpolate else arr.dtype
    result = DeviceArray(result_shape, computed)
    if result.size:
        lib = _lib.load()
        torch = runtime.torch
        dev = runtime.require_device()
        d_left = torch.from_numpy(left).to(dev)
        d_right = torch.from_numpy(right).to(dev)
        d_gamma = torch.from_numpy(gamma).to(dev)
        status = lib.cpn_quantile_sorted(
            _lib.DTYPE_CODES[arr.dtype],
            arr._thunk.base.ptr(),
            outer,
            n,
            inner,
            q_arr.size,
            d_left.data_ptr(),
            d_right.data_ptr(),
            d_gamma.data_ptr(),
            int(interpolate),
            result.base.ptr(),
            ctypes.c_void_p(runtime.stream_handle()),
        )
        _lib.check(status, "cpn_quantile_sorted")
    res = ndarray(result_shape, computed, thunk=result)
    if computed != to_dtype:
        res = res.astype(to_dtype)
    if out is None:
        return res
    converted = res if out.dtype == res.dtype else res.astype(out.dtype)
    out._thunk.base = converted._thunk.base  # (assignment into `out`: it now holds the values, in its own type)
    return out


def percentile(
    a: Any,
    q: Any,
    axis: Any = None,
    out: ndarray | None = None,
    overwrite_input: bool = False,
    method: str = "linear",
    keepdims: bool = False,
) -> ndarray:
    """q-th percentile(s): `quantile` of q / 100 (`stats_order.py:540-650`)."""
    q01 = np.asarray(q) / 100.0
    return quantile(a, q01, axis, out=out, overwrite_input=overwrite_input, method=method, keepdims=keepdims)


def median(a: Any, axis: Any = None, out: ndarray | None = None, overwrite_input: bool = False, keepdims: bool = False) -> ndarray:
    """Median along the given axis or axes: the 0.5 quantile with method 'midpoint'
    (`cupynumeric/_module/stats_avgs_vars.py:373-443`)."""
    if a is None:
        raise TypeError("'None' is not suported input to 'median'")
    return quantile(a, 0.5, axis=axis, out=out, overwrite_input=overwrite_input, keepdims=keepdims, method="midpoint")


def nanquantile(
    a: Any,
    q: Any,
    axis: Any = None,
    out: ndarray | None = None,
    overwrite_input: bool = False,
    method: str = "linear",
    keepdims: bool = False,
) -> ndarray:
    """q-th quantile(s) along the given axis or axes, ignoring NaNs (`stats_order.py:653-951`).

    A slice without any element that is not NaN gives NaN.  As in the reference, the position of a
    quantile follows from the number of elements of its slice that are not NaN, the weights are
    rounded to the array's type and so is every step of the weighted sum; the input has to be of a
    floating-point type (`numpy.finfo` of the input's type is taken); complex input raises
    TypeError.  The reference replaces NaNs by the largest finite value before it sorts, so a slice
    that holds NaNs and +inf reads that value where `numpy.nanquantile` reads +inf: kept.
    With `axis=None` the array is flattened first, as NumPy does.
    """
    a = convert_to_ndarray(a)
    original_shape = a.shape
    axes_set: tuple[int, ...] = ()
    if axis is not None and isinstance(axis, Iterable):
        axes_set = _normalize_axes(axis, a.ndim)
        if len(axes_set) == 1:
            real_axis, a_rr = axes_set[0], a
        else:
            real_axis, a_rr = _collapse_axes(a, axes_set)
            overwrite_input = False
    else:
        real_axis, a_rr = axis, a
        if real_axis is not None:
            axes_set = _normalize_axes(real_axis, a.ndim)
            real_axis = axes_set[0]
    if method not in METHODS:
        raise KeyError(method)
    q_arr = np.asarray(q)
    if a_rr.dtype.kind == "c":
        raise TypeError("input array cannot be of complex type")
    np.finfo(a_rr.dtype)  # (integer and bool input: the reference fails here, with this error)

    from . import sort

    if overwrite_input:
        a_rr.sort(axis=real_axis)
        arr = a_rr
    else:
        arr = sort(a_rr, axis=real_axis)  # NaNs last in every slice
    to_dtype = arr.dtype if method in _KEEP_DTYPE else np.dtype(np.float64)

    if real_axis is None:
        n, outer, inner = arr.size, 1, 1
        remaining = (1,) * len(original_shape) if keepdims else ()
    else:
        n = arr.shape[real_axis]
        outer = int(np.prod(arr.shape[:real_axis], dtype=np.int64))
        inner = int(np.prod(arr.shape[real_axis + 1 :], dtype=np.int64))
        if keepdims:
            remaining = tuple(1 if k in axes_set else original_shape[k] for k in range(len(original_shape)))
        else:
            remaining = tuple(arr.shape[k] for k in range(arr.ndim) if k != real_axis)
    result_shape = (*q_arr.shape, *remaining)
    if out is not None and out.shape != result_shape:
        raise ValueError("wrong shape on output array")

    slices = outer * inner
    result = DeviceArray(result_shape, to_dtype)
    if result.size:
        lib = _lib.load()
        torch = runtime.torch
        dev = runtime.require_device()
        stream = ctypes.c_void_p(runtime.stream_handle())
        code = _lib.DTYPE_CODES[arr.dtype]
        src = arr._thunk.base.ptr() if arr.size else None
        d_counts = torch.empty(slices, dtype=torch.int64, device=dev)
        _lib.check(lib.cpn_count_not_nan_sorted(code, src, outer, n, inner, d_counts.data_ptr(), stream),
                   "cpn_count_not_nan_sorted")
        runtime.flush_status()  # a failed sort must not reach the host through the counts
        counts = d_counts.cpu().numpy()  # (synchronises: the positions below depend on the counts)
        # positions and weights per quantile and slice, worked out once per different count
        # (`stats_order.py:713-746`)
        distinct, which = np.unique(counts, return_inverse=True)
        left = np.zeros((q_arr.size, slices), dtype=np.int64)
        right = np.zeros((q_arr.size, slices), dtype=np.int64)
        gamma = np.zeros((q_arr.size, slices), dtype=np.float64)
        interpolate = True
        for k, qv in enumerate(q_arr.reshape(-1)):
            l_of = np.zeros(distinct.size, dtype=np.int64)
            r_of = np.zeros(distinct.size, dtype=np.int64)
            g_of = np.zeros(distinct.size, dtype=np.float64)
            for j, cnt in enumerate(distinct):
                cnt = int(cnt)
                if cnt == 0:
                    continue
                g, lpos = _position(method, float(qv), cnt)
                rpos = lpos + 1
                if lpos >= cnt - 1:
                    lpos = rpos = cnt - 1
                elif lpos < 0:
                    lpos = rpos = 0
                l_of[j], r_of[j] = lpos, rpos
                if g is None:
                    interpolate = False
                else:
                    g_of[j] = g
            left[k], right[k], gamma[k] = l_of[which], r_of[which], g_of[which]
        if method in ("closest_observation", "lower", "higher", "nearest"):
            interpolate = False  # (also when every slice is empty and no position was worked out)
        d_left = torch.from_numpy(left).to(dev)
        d_right = torch.from_numpy(right).to(dev)
        d_gamma = torch.from_numpy(gamma).to(dev)
        status = lib.cpn_nanquantile_sorted(
            code, src, outer, n, inner, q_arr.size, d_counts.data_ptr(), d_left.data_ptr(), d_right.data_ptr(),
            d_gamma.data_ptr(), int(interpolate), int(to_dtype == arr.dtype), result.base.ptr(), stream,
        )
        _lib.check(status, "cpn_nanquantile_sorted")
    res = ndarray(result_shape, to_dtype, thunk=result)
    if out is None:
        return res
    converted = res if out.dtype == res.dtype else res.astype(out.dtype)
    out._thunk.base = converted._thunk.base
    return out


def nanpercentile(
    a: Any,
    q: Any,
    axis: Any = None,
    out: ndarray | None = None,
    overwrite_input: bool = False,
    method: str = "linear",
    keepdims: bool = False,
) -> ndarray:
    """q-th percentile(s) ignoring NaNs: `nanquantile` of q / 100 (`stats_order.py:954-1080`)."""
    q01 = np.asarray(q) / 100.0
    return nanquantile(a, q01, axis, out=out, overwrite_input=overwrite_input, method=method, keepdims=keepdims)


def nanmedian(a: Any, axis: Any = None, out: ndarray | None = None, overwrite_input: bool = False, keepdims: bool = False) -> ndarray:
    """Median ignoring NaNs: the 0.5 `nanquantile` with method 'midpoint'
    (`cupynumeric/_module/stats_avgs_vars.py:445-512`)."""
    if a is None:
        raise TypeError("'None' is not suported input to 'nanmedian'")
    return nanquantile(a, 0.5, axis=axis, out=out, overwrite_input=overwrite_input, keepdims=keepdims, method="midpoint")
