"""ctypes binding of `libcpnsort.so` (declared in `include/cpn_sort.h`).

The reference loads its native library with cffi and registers Legate tasks
(`cupynumeric/config.py:330-383`); here the library is a plain C ABI and is loaded with
ctypes.  There is no fallback: if the shared library is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int64, c_uint64, c_void_p
from pathlib import Path

import numpy as np

LIB_NAME = "libcpnsort.so"
# (CUPYNUMERIC_AMD_LIBRARY names another build of the same library, for A/B runs of kernel variants)
LIB_PATH = Path(os.environ.get("CUPYNUMERIC_AMD_LIBRARY") or (Path(__file__).resolve().parent / LIB_NAME))

# element type codes of include/cpn_sort.h (enum cpn_dtype)
DTYPE_CODES: dict[np.dtype, int] = {
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

# enum cpn_status
CPN_OK = 0
CPN_ERR_DTYPE = -1
CPN_ERR_NULL = -2
CPN_ERR_SHAPE = -3
CPN_ERR_TEMP = -4
CPN_ERR_ALIGN = -5
CPN_ERR_HIP = -6
CPN_ERR_DEVICE = -7
CPN_ERR_UNSUPPORTED = -8
CPN_ERR_SCRATCH = -9

# include/cpn_sort.h: options of cpn_local_sort_ex
CPN_SORT_SINGLE_TICKET = 1

# include/cpn_sort.h: workspace of cpn_local_sort_static
STATIC_SCRATCH_BYTES = 64 << 20

# name -> (restype, argtypes); every symbol include/cpn_sort.h declares
PROTOTYPES: dict[str, tuple] = {
    "cpn_sort_version": (c_int, []),
    "cpn_status_string": (c_char_p, [c_int]),
    "cpn_last_hip_error": (c_int, []),
    "cpn_set_lds_row_limit": (c_int64, [c_int64]),
    "cpn_set_wide_row_threshold": (c_int64, [c_int64]),
    "cpn_set_lookback_spin_limit": (c_int64, [c_int64]),
    "cpn_set_virtual_digit_threshold": (c_int64, [c_int64]),
    "cpn_set_wave_row_limit": (c_int64, [c_int64]),
    "cpn_set_merge_rows": (c_int, [c_int]),
    "cpn_set_bitonic_rows": (c_int, [c_int]),
    "cpn_set_tile_order": (c_int, [c_int]),
    "cpn_dtype_size": (c_uint64, [c_int]),
    "cpn_key_order_bits": (c_uint64, [c_int, c_uint64]),
    "cpn_local_sort_temp_bytes": (c_uint64, [c_int, c_uint64, c_uint64, c_int, c_int, c_int]),
    "cpn_local_sort": (
        c_int,
        [c_int, c_void_p, c_void_p, c_void_p, c_uint64, c_uint64, c_int64, c_int, c_void_p, c_uint64, c_void_p],
    ),
    "cpn_local_sort_ex": (
        c_int,
        [c_int, c_void_p, c_void_p, c_void_p, c_uint64, c_uint64, c_int64, c_int, ctypes.c_uint32, c_void_p, c_uint64,
         c_void_p],
    ),
    "cpn_local_sort_static": (
        c_int, [c_int, c_void_p, c_void_p, c_void_p, c_uint64, c_uint64, c_int64, c_int, c_void_p, c_void_p]
    ),
    "cpn_local_sort_check": (c_int, [c_void_p, c_void_p]),
    "cpn_real_to_complex": (c_int, [c_int, c_void_p, c_int, c_void_p, c_uint64, c_void_p]),
    "cpn_astype": (c_int, [c_int, c_void_p, c_int, c_void_p, c_uint64, c_void_p]),
    "cpn_searchsorted_temp_bytes": (c_uint64, [c_int, c_uint64, c_uint64]),
    "cpn_searchsorted": (
        c_int, [c_int, c_void_p, c_uint64, c_void_p, c_uint64, c_int, c_void_p, c_void_p, c_uint64, c_void_p]
    ),
    "cpn_unique_temp_bytes": (c_uint64, [c_int, c_uint64]),
    "cpn_unique": (c_int, [c_int, c_void_p, c_void_p, c_uint64, c_void_p, c_void_p, c_uint64, c_void_p]),
    "cpn_quantile_sorted": (
        c_int,
        [c_int, c_void_p, c_uint64, c_uint64, c_uint64, c_uint64, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p],
    ),
    "cpn_count_not_nan_sorted": (c_int, [c_int, c_void_p, c_uint64, c_uint64, c_uint64, c_void_p, c_void_p]),
    "cpn_nanquantile_sorted": (
        c_int,
        [c_int, c_void_p, c_uint64, c_uint64, c_uint64, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
         c_void_p, c_void_p],
    ),
    "cpn_take_along_last_axis": (
        c_int, [c_int, c_void_p, c_void_p, c_void_p, c_uint64, c_uint64, c_uint64, c_void_p, c_void_p]
    ),
    "cpn_take_along_last_axis_broadcast": (
        c_int,
        [c_int, c_void_p, c_void_p, c_void_p, c_int, ctypes.POINTER(c_uint64), ctypes.POINTER(c_uint64),
         ctypes.POINTER(c_uint64), c_uint64, c_uint64, c_void_p, c_void_p],
    ),
    "cpn_lexsort_pack": (
        c_int,
        [c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_void_p), c_void_p, c_int, c_void_p, c_uint64, c_uint64, c_void_p],
    ),
    "cpn_profile_enable": (c_int, [c_int]),
    "cpn_profile_collect": (c_int, [c_void_p, c_uint64, c_void_p, c_int]),
    "cpn_stream_probe": (c_int, [c_int, c_void_p, c_void_p, c_uint64, c_void_p]),
    "cpn_swapaxes_copy": (c_int, [c_int, c_void_p, c_void_p, ctypes.POINTER(c_int64), c_int, c_int, c_int, c_void_p]),
}

_lib: ctypes.CDLL | None = None


class NativeLibraryError(RuntimeError):
    """The HIP shared library is missing or incomplete."""


def load() -> ctypes.CDLL:
    """Load the shared library once and attach prototypes.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise NativeLibraryError(
            f"{LIB_PATH} not found: build it with `python -m cupynumeric_amd.build` "
            "(there is no CPU fallback for the sort path)"
        )
    # PyTorch ships its own copy of the HIP runtime (same soname).  Import it first so that the
    # dynamic loader binds this library to the runtime torch already initialised; two HIP
    # runtimes in one process do not share a device context.
    import torch  # noqa: F401

    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in PROTOTYPES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise NativeLibraryError(f"{LIB_PATH} does not export {name}") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def profile_collect(max_records: int = 65536) -> list[tuple[str, float]]:
    """(label, milliseconds) of every kernel launch recorded since the last collect."""
    lib = load()
    stride = 32
    labels = ctypes.create_string_buffer(stride * max_records)
    ms = (ctypes.c_float * max_records)()
    n = lib.cpn_profile_collect(labels, stride, ms, max_records)
    raw = labels.raw
    return [(raw[i * stride : (i + 1) * stride].split(b"\0", 1)[0].decode(), float(ms[i])) for i in range(n)]


def status_string(status: int) -> str:
    return load().cpn_status_string(status).decode()


def check(status: int, what: str) -> None:
    """Map a negative cpn_status to a Python exception."""
    if status == CPN_OK:
        return
    msg = f"{what}: {status_string(status)} (cpn_status {status})"
    if status == CPN_ERR_HIP:
        msg += f", hipError {load().cpn_last_hip_error()}"
    if status in (CPN_ERR_SHAPE, CPN_ERR_NULL, CPN_ERR_ALIGN, CPN_ERR_DTYPE):
        raise ValueError(msg)
    if status == CPN_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
