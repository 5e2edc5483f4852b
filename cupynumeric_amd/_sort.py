"""Axis dispatch of sort/argsort, following `cupynumeric/_thunk/_sort.py` function by
function; `sort_task` calls the C ABI (`cpn_local_sort`) where the reference launches the
Legate SORT task.
"""
from __future__ import annotations

import ctypes
from typing import TYPE_CHECKING

from numpy.exceptions import AxisError
from numpy.lib.array_utils import normalize_axis_index

from . import _lib
from .runtime import runtime

if TYPE_CHECKING:
    from ._thunk import DeviceArray


def sort_flattened(output: "DeviceArray", input: "DeviceArray", argsort: bool, stable: bool) -> None:
    """`axis=None` on an array of several dimensions (`cupynumeric/_thunk/_sort.py:37-47`): the
    C-order flattening is a view of the same dense storage, its 1-D sort is the result."""
    from ._thunk import DeviceArray

    flat = input.reshape((input.size,), order="C")
    result = DeviceArray(flat.shape, dtype=output.dtype)
    sort_deferred(result, flat, argsort, stable=stable)
    output.base = result.base


def sort_swapped(output: "DeviceArray", input: "DeviceArray", argsort: bool, sort_axis: int, stable: bool) -> None:
    """A sort along an axis that is not the last (`cupynumeric/_thunk/_sort.py:50-76`): transposed
    dense copy, last-axis sort of the copy, transposed back.  The reference hands back a transposed
    view of the sorted copy; here the result is copied back so that every array stays dense row-major."""
    from ._thunk import DeviceArray

    sort_axis = normalize_axis_index(sort_axis, input.ndim)
    last = input.ndim - 1
    moved = input.swapaxes_copy(sort_axis, last)
    if argsort:
        positions = DeviceArray(moved.shape, dtype=output.dtype)
        sort_deferred(positions, moved, argsort, stable=stable)
        output.base = positions.swapaxes_copy(last, sort_axis).base
    else:
        sort_deferred(moved, moved, argsort, stable=stable)  # the copy is ours: sorted in place
        output.base = moved.swapaxes_copy(last, sort_axis).base


def sort_task(output: "DeviceArray", input: "DeviceArray", argsort: bool, stable: bool) -> None:
    """`cupynumeric/_thunk/_sort.py:79-107`: sort the rows (last axis) of a dense array.

    The task's scalars (argsort flag, shape, stable flag) become arguments of `cpn_local_sort`;
    the output is aligned with the input (same shape), values for `sort`, int64 row positions
    for `argsort`.
    """
    lib = _lib.load()
    volume = input.size
    if volume == 0:
        return  # empty rectangle: nothing to do (`src/cupynumeric/sort/sort_template.inl:67-72`)
    seg = input.shape[-1]
    code = _lib.DTYPE_CODES[input.dtype]
    in_place = (not argsort) and (output.base is input.base)

    values_in = input.base.ptr()
    if argsort:
        values_out = None
        indices_out = output.base.ptr()
    else:
        values_out = output.base.ptr()
        indices_out = None

    temp_bytes = lib.cpn_local_sort_temp_bytes(code, volume, seg, int(not argsort), int(argsort), int(in_place))
    if temp_bytes == 0:
        _lib.check(
            lib.cpn_local_sort(code, values_in, values_out, indices_out, volume, seg, 0, int(stable), None, 0, None),
            "cpn_local_sort",
        )
        raise NotImplementedError(f"cpn_local_sort: no workspace layout for dtype={input.dtype}, shape={input.shape}")
    stream = ctypes.c_void_p(runtime.stream_handle())

    def issue(options: int = 0):
        temp = runtime.empty_bytes(temp_bytes)
        status = lib.cpn_local_sort_ex(
            code,
            values_in,
            values_out,
            indices_out,
            volume,
            seg,
            0,  # rect.lo[last] of a single-GPU launch (`src/cupynumeric/sort/sort.cu:1851`)
            int(stable),
            options,
            temp.data_ptr(),
            temp_bytes,
            stream,
        )
        _lib.check(status, "cpn_local_sort")
        return temp

    temp = issue()
    # Rows sorted by the per-row kernels cannot fail on the device (the request then needs nothing but
    # the workspace header).  The global sort can: a bounded wait between its tiles may run out.
    if runtime.check_mode == "off" or temp_bytes == lib.cpn_local_sort_temp_bytes(code, 0, 0, 1, 0, 0):
        return
    if runtime.check_mode == "lazy":
        runtime.defer_status(temp)
        return
    status = lib.cpn_local_sort_check(temp.data_ptr(), stream)
    if status == _lib.CPN_ERR_DEVICE and not in_place:
        # once more, from a fresh workspace, with the tiles of this one call handed out through one
        # counter: that order does not depend on every XCD taking part (the input was not touched: it
        # is not the output).  Nothing process-wide changes, so other threads sort on undisturbed.
        temp = issue(_lib.CPN_SORT_SINGLE_TICKET)
        status = lib.cpn_local_sort_check(temp.data_ptr(), stream)
    _lib.check(status, "cpn_local_sort")


def sort_deferred(
    output: "DeviceArray",
    input: "DeviceArray",
    argsort: bool,
    axis: int | None = -1,
    stable: bool = False,
) -> None:
    """Axis dispatch of sort and argsort (`cupynumeric/_thunk/_sort.py:110-136`): 0-D input, `axis=None`
    (flatten, or axis 0 of a 1-D array), the last axis (the kernel call), any other axis (transposes)."""
    if input.ndim == 0:
        if axis is not None:
            raise AxisError(axis, input.ndim)  # NumPy's answer to any axis of a scalar
        if argsort:
            # (the reference aliases the input store here even for argsort; a value buffer is not an
            # index buffer, so the only possible index is handed back instead)
            import numpy as np

            from ._thunk import Storage

            output.base = Storage(8, host=np.zeros(1, dtype=np.int64))
        else:
            output.base = input.base  # a scalar is sorted
        return
    if axis is None and input.ndim > 1:
        sort_flattened(output, input, argsort, stable)
        return
    sort_axis = 0 if axis is None else normalize_axis_index(axis, input.ndim)
    if sort_axis == input.ndim - 1:
        sort_task(output, input, argsort, stable)
    else:
        sort_swapped(output, input, argsort, sort_axis, stable)


def _pack_keys(group: "list[DeviceArray]", indices: "DeviceArray | None") -> "DeviceArray":
    """One unsigned word per element holding the keys of `group` (least significant first) as
    order-preserving images, read through `indices` when given (`cpn_lexsort_pack`)."""
    import numpy as np

    from ._thunk import DeviceArray

    lib = _lib.load()
    width = sum(k.dtype.itemsize for k in group)
    packed_dtype = np.dtype(np.uint32) if width <= 4 else np.dtype(np.uint64)
    shape = group[0].shape
    out = DeviceArray(shape, packed_dtype)
    n = len(group)
    dtypes = (ctypes.c_int * n)(*[_lib.DTYPE_CODES[k.dtype] for k in group])
    ptrs = (ctypes.c_void_p * n)(*[k.base.ptr() for k in group])
    seg = shape[-1]
    status = lib.cpn_lexsort_pack(
        n,
        dtypes,
        ptrs,
        indices.base.ptr() if indices is not None else None,
        packed_dtype.itemsize,
        out.base.ptr(),
        out.size // seg,
        seg,
        ctypes.c_void_p(runtime.stream_handle()),
    )
    _lib.check(status, "cpn_lexsort_pack")
    return out


def _lexsort_groups(keys: "list[DeviceArray]") -> "list[list[DeviceArray]]":
    """Consecutive real keys whose widths add up to at most 8 bytes (and at most 8 keys) are
    sorted as one packed key; a complex key, or a real key that would not fit, starts a new
    group."""
    groups: list[list] = []
    width = 0
    for k in keys:
        kb = k.dtype.itemsize
        packable = k.dtype.kind != "c"
        if groups and packable and groups[-1][0].dtype.kind != "c" and width + kb <= 8 and len(groups[-1]) < 8:
            groups[-1].append(k)
            width += kb
        else:
            groups.append([k])
            width = kb if packable else 16
    return groups


def lexsort_deferred(keys: "list[DeviceArray]", axis: int) -> "DeviceArray":
    """The loop of `lexsort` (`cupynumeric/_module/ssc_sorting.py:423-444`): a stable argsort of
    the least significant key, then for every further key: reorder the key by the indices so
    far, argsort it (stable), reorder the indices by that order.  `keys[-1]` is the primary key.

    Two changes of schedule, none of result.  Neighbouring real keys of at most 8 bytes together
    are packed into one unsigned word and sorted in one argsort (a lexicographic order is the
    order of the concatenated order-preserving images), and the reordering of the keys of a
    later group is fused into its packing.  Axes other than the last are moved there once (one
    transpose per key, one for the result) instead of once per argsort.

    Every key is sorted in its own element type under the NumPy order, which already puts
    -inf < finite < +inf < NaN, so the reference's remapping of special float values
    (`ssc_sorting.py:352-420`) has nothing to do here.
    """
    from ._thunk import DeviceArray

    ndim = keys[0].ndim
    axis = normalize_axis_index(axis, ndim)
    last = ndim - 1
    if axis != last:
        keys = [k.swapaxes_copy(axis, last) for k in keys]

    indices = None
    for group in _lexsort_groups(keys):
        if len(group) == 1 and indices is None:
            key_reordered = group[0]  # first key: nothing to reorder, no need to pack
        elif group[0].dtype.kind == "c":
            key_reordered = group[0].take_along_last_axis(indices, check="trusted")
        else:
            key_reordered = _pack_keys(group, indices)
        order = DeviceArray(key_reordered.shape, dtype="int64")
        sort_task(order, key_reordered, True, True)
        indices = order if indices is None else indices.take_along_last_axis(order, check="trusted")

    if axis != last:
        indices = indices.swapaxes_copy(last, axis)
    return indices
