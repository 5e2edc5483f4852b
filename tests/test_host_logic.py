"""CPU-only checks of the host side: the C-ABI library loads and exports every symbol the header
declares, pure-host entry points behave, the Python layer validates arguments like the
reference, and the product has no CPU fallback."""
from __future__ import annotations

import re
from pathlib import Path

import numpy as np
import pytest
from conftest import ALL_REAL_DTYPES, ROOT, make_input

import cupynumeric_amd as num
from cupynumeric_amd import _lib


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def test_every_declared_symbol_is_exported(lib):
    header = (ROOT / "include" / "cpn_sort.h").read_text()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(cpn_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found in include/cpn_sort.h"
    assert declared == set(_lib.PROTOTYPES), "ctypes prototypes and header differ"
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared but not exported"


def test_dtype_codes_match_header():
    header = (ROOT / "include" / "cpn_sort.h").read_text()
    codes = dict(re.findall(r"CPN_([A-Z0-9]+)\s*=\s*(\d+)", header))
    names = {"BOOL": np.bool_, "INT8": np.int8, "INT16": np.int16, "INT32": np.int32, "INT64": np.int64,
             "UINT8": np.uint8, "UINT16": np.uint16, "UINT32": np.uint32, "UINT64": np.uint64,
             "FLOAT16": np.float16, "FLOAT32": np.float32, "FLOAT64": np.float64,
             "COMPLEX64": np.complex64, "COMPLEX128": np.complex128}
    for name, np_type in names.items():
        assert _lib.DTYPE_CODES[np.dtype(np_type)] == int(codes[name])


def test_version_status_strings_and_sizes(lib):
    assert lib.cpn_sort_version() >= 1
    assert lib.cpn_status_string(0) == b"ok"
    for status in range(-9, 0):
        assert lib.cpn_status_string(status) not in (b"ok", b"unknown status")
    assert lib.cpn_status_string(-99) == b"unknown status"
    for dt, code in _lib.DTYPE_CODES.items():
        assert lib.cpn_dtype_size(code) == dt.itemsize
    assert lib.cpn_dtype_size(99) == 0


def test_argument_validation_without_a_device(lib):
    # every check below fails before the first HIP call
    sort = lib.cpn_local_sort
    assert sort(99, 16, 16, None, 4, 4, 0, 1, 256, 1024, None) == _lib.CPN_ERR_DTYPE
    assert sort(3, None, None, None, 0, 0, 0, 1, None, 0, None) == _lib.CPN_OK  # volume 0: no-op
    assert sort(3, 16, 32, None, 10, 3, 0, 1, 256, 1024, None) == _lib.CPN_ERR_SHAPE  # 3 does not divide 10
    assert sort(3, 16, 32, None, 10, 0, 0, 1, 256, 1024, None) == _lib.CPN_ERR_SHAPE
    assert sort(3, None, 32, None, 4, 4, 0, 1, 256, 1024, None) == _lib.CPN_ERR_NULL
    assert sort(3, 16, None, None, 4, 4, 0, 1, 256, 1024, None) == _lib.CPN_ERR_NULL  # no output at all
    assert sort(3, 18, 32, None, 4, 4, 0, 1, 256, 1024, None) == _lib.CPN_ERR_ALIGN
    assert sort(3, 16, None, 36, 4, 4, 0, 1, 256, 1024, None) == _lib.CPN_ERR_ALIGN  # int64 out misaligned
    assert sort(3, 16, 32, None, 4, 4, 0, 1, None, 0, None) == _lib.CPN_ERR_TEMP
    assert sort(3, 16, 32, None, 4, 4, 0, 1, 256, 16, None) == _lib.CPN_ERR_TEMP  # too small
    assert sort(3, 16, 32, None, 4, 4, 0, 1, 264, 4096, None) == _lib.CPN_ERR_TEMP  # misaligned
    assert sort(13, 24, 32, None, 4, 4, 0, 1, 256, 1024, None) == _lib.CPN_ERR_ALIGN  # complex128 needs 16-byte alignment
    assert lib.cpn_local_sort_check(None, None) == _lib.CPN_ERR_NULL
    swap = lib.cpn_swapaxes_copy
    import ctypes

    shape = (ctypes.c_int64 * 2)(3, 4)
    assert swap(4, 16, 64, shape, 2, 0, 2, None) == _lib.CPN_ERR_SHAPE
    assert swap(3, 16, 64, shape, 2, 0, 1, None) == _lib.CPN_ERR_SHAPE
    assert swap(4, None, 64, shape, 2, 0, 1, None) == _lib.CPN_ERR_NULL
    assert swap(4, 18, 64, shape, 2, 0, 1, None) == _lib.CPN_ERR_ALIGN
    empty = (ctypes.c_int64 * 2)(0, 4)
    assert swap(4, None, None, empty, 2, 0, 1, None) == _lib.CPN_OK
    # an element size the gather does not know is refused before anything is computed from it
    take = lib.cpn_take_along_last_axis
    assert take(0, 16, 64, 128, 1, 4, 4, None, None) == _lib.CPN_ERR_DTYPE
    assert take(3, 16, 64, 128, 1, 4, 4, None, None) == _lib.CPN_ERR_DTYPE
    assert take(4, 18, 64, 128, 1, 4, 4, None, None) == _lib.CPN_ERR_ALIGN


def test_temp_bytes_layout(lib):
    def align256(v):
        return (v + 255) // 256 * 256

    tb = lib.cpn_local_sort_temp_bytes
    f32, i64, u8, f16 = 10, 4, 5, 9
    assert tb(99, 100, 100, 1, 0, 0) == 0
    assert tb(f32, 100, 7, 1, 0, 0) == 0  # 7 does not divide 100
    header = tb(f32, 0, 0, 1, 0, 0)
    assert header == 2048
    assert tb(f32, 1 << 20, 1024, 1, 1, 0) == header  # rows that fit LDS need only the header
    # longest rows of the per-row kernels: 16 384 keys of up to 4 bytes; 8-byte keys 16 384 for values
    # only, 14 336 when positions are staged beside them; 16-byte keys 4096
    f64, c128_ = 11, 13
    assert tb(f32, 4 * 16384, 16384, 1, 1, 0) == header and tb(f32, 4 * 16385, 16385, 1, 0, 0) > header
    # float16: values-only rows are counted up to 57 344 keys; with positions the radix rows end at 16 384
    assert tb(9, 4 * 57344, 57344, 1, 0, 0) == header and tb(9, 4 * 57345, 57345, 1, 0, 0) > header
    assert tb(9, 4 * 16384, 16384, 0, 1, 0) == header and tb(9, 4 * 16385, 16385, 0, 1, 0) > header
    assert tb(f64, 4 * 16384, 16384, 1, 0, 0) == header and tb(f64, 4 * 16385, 16385, 1, 0, 0) > header
    assert tb(f64, 4 * 14336, 14336, 0, 1, 0) == header and tb(f64, 4 * 14337, 14337, 0, 1, 0) > header
    assert tb(f64, 4 * 14337, 14337, 1, 0, 0) == header
    assert tb(c128_, 4 * 4096, 4096, 1, 1, 0) == header and tb(c128_, 4 * 4097, 4097, 1, 0, 0) > header
    # longer rows of real keys of 4 and 8 bytes, merged from sorted pieces: a table of chunk starts (one word
    # per 2048 outputs of a row and per piece), the rows once more and their positions; both twice from two
    # levels of merging on; up to 2 levels for 4-byte keys, 6 for 8-byte keys (5 with positions)
    def table(rows, seg, levels):
        return align256(rows * ((seg + 2047) // 2048 + (1 << levels)) * 4)

    assert tb(f32, 4 * 20000, 20000, 1, 0, 0) == header + table(4, 20000, 1) + align256(4 * 20000 * 4)
    assert tb(f64, 4 * 20000, 20000, 0, 1, 0) == header + table(4, 20000, 1) + align256(4 * 20000 * 8) + align256(4 * 20000 * 8)
    assert tb(f32, 4 * 32769, 32769, 1, 0, 0) == header + table(4, 32769, 2) + 2 * align256(4 * 32769 * 4)
    assert tb(f32, 4 * 65536, 65536, 1, 1, 0) == header + table(4, 65536, 2) + 2 * (align256(4 * 65536 * 4) + align256(4 * 65536 * 8))
    assert tb(f32, 4 * 65537, 65537, 1, 0, 0) == header + 4 * 4 * 256 * 4 + 4 * 20 * 256 * 4 + align256(4 * 65537 * 4)  # global layout: histograms, tile descriptors, one key buffer
    assert tb(f64, 2 * (1 << 20), 1 << 20, 1, 0, 0) == header + table(2, 1 << 20, 6) + 2 * align256(2 * (1 << 20) * 8)
    assert tb(f64, 2 * 458752, 458752, 0, 1, 0) == header + table(2, 458752, 5) + 4 * align256(2 * 458752 * 8)
    prev = lib.cpn_set_merge_rows(0)
    try:
        assert lib.cpn_set_merge_rows(0) == 0
        assert tb(f32, 4 * 20000, 20000, 1, 0, 0) != header + table(4, 20000, 1) + align256(4 * 20000 * 4)
        lib.cpn_set_merge_rows(2)  # one level for every key
        assert tb(f32, 4 * 20000, 20000, 1, 0, 0) == header + table(4, 20000, 1) + align256(4 * 20000 * 4)
        assert tb(f32, 4 * 32769, 32769, 1, 0, 0) != header + table(4, 32769, 2) + 2 * align256(4 * 32769 * 4)
    finally:
        lib.cpn_set_merge_rows(prev)
    assert lib.cpn_set_merge_rows(-1) == 1 and lib.cpn_set_merge_rows(1) == 1
    n = 1 << 24
    tiles = n // 16384  # 512 threads x 32 keys per tile for keys of up to 4 bytes

    fixed = header + 4 * 256 * 4 + 4 * tiles * 256 * 4
    assert tb(f32, n, n, 1, 0, 0) == fixed + 4 * n  # one key buffer
    assert tb(f32, n, n, 1, 0, 1) == fixed + 2 * 4 * n  # in place: a second buffer, in case an odd number of passes runs
    assert tb(f32, n, n, 0, 1, 0) == fixed + 2 * 4 * n + 4 * n  # index-only: two key buffers + narrow indices
    assert tb(f32, n, n, 1, 1, 0) == fixed + 4 * n + 4 * n
    # 8-bit keys take one pass: no key buffer unless sorting in place
    t8 = header + 256 * 4 + tiles * 256 * 4
    assert tb(u8, n, n, 1, 0, 0) == t8
    assert tb(u8, n, n, 1, 0, 1) == t8 + n
    assert tb(u8, n, n, 0, 1, 0) == t8
    # monotone in the request
    assert tb(i64, n, n, 0, 1, 0) > tb(f32, n, n, 0, 1, 0) > tb(f16, n, n, 0, 1, 0)
    # complex keys take one more pass (the NaN class) than their bytes
    c64, c128 = 12, 13
    assert tb(c64, n, n, 1, 0, 0) == header + 9 * 256 * 4 + 9 * (n // 16384) * 256 * 4 + 8 * n  # 8-byte keys: 1024 x 16
    assert tb(c128, n, n, 1, 0, 0) == header + align256(17 * 256 * 4) + 17 * (n // 8192) * 256 * 4 + 16 * n
    # the row-length switch moves work to the global path
    prev = lib.cpn_set_lds_row_limit(0)
    try:
        assert tb(f32, 1 << 20, 1024, 1, 1, 0) > header
    finally:
        lib.cpn_set_lds_row_limit(prev)
    assert tb(f32, 1 << 20, 1024, 1, 1, 0) == header


@pytest.mark.parametrize("dtype", ALL_REAL_DTYPES)
def test_key_transform_orders_like_numpy(lib, dtype):
    """Sorting by the library's key transform (a stable integer sort) must reproduce NumPy's
    stable argsort: pins NaN-last, -0 == +0 and the signed/unsigned flips on the host."""
    dt = np.dtype(dtype)
    code = _lib.DTYPE_CODES[dt]
    ub = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[dt.itemsize]
    if dt.itemsize <= 2:
        raw = np.arange(1 << (8 * dt.itemsize), dtype=np.uint32).astype(ub)  # every bit pattern
        if dt.kind == "b":
            raw = np.array([0, 1], dtype=ub)
        raw = np.random.default_rng(0).permutation(raw)
    else:
        raw = make_input(dtype, (20000,), seed=3).view(ub)
    x = raw.view(dt)
    keys = np.array([lib.cpn_key_order_bits(code, int(b)) for b in raw], dtype=np.uint64)
    assert np.array_equal(np.argsort(keys, kind="stable"), np.argsort(x, kind="stable"))
    assert int(keys.max()) < (1 << (8 * dt.itemsize)) or dt.itemsize == 8


# ---- Python layer: the reference's observable behaviour, no GPU needed ----------------------------
def test_python_validation_before_any_device_work():
    a = num.array(np.arange(6, dtype=np.int32).reshape(2, 3))
    # cupynumeric/_thunk/deferred.py:5471-5472, tests/integration/test_sort.py:67-70
    for axis in (2, -3):
        with pytest.raises(ValueError, match="invalid axis"):
            num.sort(a, axis=axis)
        with pytest.raises(ValueError, match="invalid axis"):
            num.argsort(a, axis=axis)
        with pytest.raises(ValueError, match="invalid axis"):
            a.sort(axis=axis)
    with pytest.raises(ValueError):
        num.sort([-1, 0, 1, 2, 10], axis=2)
    # cupynumeric/_thunk/deferred.py:5466-5470
    with pytest.raises(NotImplementedError, match="does not support sorting with 'order'"):
        num.sort(a, order="x")
    # cupynumeric/_utils/array.py:64-68, tests/integration/test_sort.py:185-192
    with pytest.raises(TypeError, match="cuPyNumeric does not support dtype="):
        num.sort(np.array(["a", "b", "c"]))
    with pytest.raises(TypeError, match="cuPyNumeric does not support dtype="):
        num.array(np.array(["a"]))
    # 0-D with an axis: the ValueError of the thunk pre-empts AxisError
    # (tests/integration/test_sort.py:249-264)
    with pytest.raises(ValueError):
        num.sort(num.array(np.int32(3)), axis=0)


def test_result_metadata_of_empty_inputs():
    # tests/integration/test_sort.py:60-65: no device work is needed for empty arrays
    for arr in ([], [[]], [[], []]):
        res = num.sort(arr)
        assert np.array_equal(res, np.sort(arr))
        idx = num.argsort(arr)
        assert np.array_equal(idx, np.argsort(arr))
        assert idx.dtype == np.int64
    for shape in [(0,), (0, 1), (1, 0), (1, 0, 0), (1, 1, 0), (1, 0, 1)]:
        x = np.zeros(shape, dtype=np.int32)
        for axis in range(-len(shape) + 1, len(shape)):
            assert num.sort(x, axis=axis).shape == shape
            assert num.argsort(x, axis=axis).shape == shape
        assert num.sort(x, axis=None).shape == (0,)


def test_no_cpu_fallback():
    """Without a HIP device the sort must fail loudly instead of computing on the host."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        num.sort(np.array([3, 1, 2], dtype=np.int32))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        num.argsort(np.array([[3.0, 1.0], [2.0, 0.0]]), axis=0)


def test_product_does_not_reach_the_oracle():
    """Nothing under cupynumeric_amd/ may import or load the CPU oracle."""
    for path in (ROOT / "cupynumeric_amd").rglob("*"):
        if path.suffix in (".py", ".h", ".hip"):
            text = path.read_text()
            assert "oracle" not in text.lower(), f"{path} mentions the oracle"


def test_missing_library_is_an_error(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libcpnsort.so")
    with pytest.raises(_lib.NativeLibraryError, match="no CPU fallback"):
        _lib.load()


def test_resource_remarks_are_parsed():
    from cupynumeric_amd import build as B

    tag = "[-Rpass-analysis=kernel-resource-usage]"
    lines = [
        "In file included from a.hip:1:",
        f"./k.h:83:1: remark: Function Name: _Zkernel_a {tag}",
        "   83 | {",
        "      | ^",
        f"./k.h:83:1: remark:     VGPRs: 59 {tag}",
        "   83 | {",
        "      | ^",
        f"./k.h:83:1: remark:     ScratchSize [bytes/lane]: 516 {tag}",
        "   83 | {",
        "      | ^",
        f"./k.h:83:1: remark:     LDS Size [bytes/block]: 10536 {tag}",
        "   83 | {",
        "      | ^",
        "a.hip:7:3: warning: something else",
        "11 remarks generated when compiling for gfx950.",
    ]
    resources, rest = B._split_resource_remarks(lines)
    assert resources == {"_Zkernel_a": {"vgprs": 59, "scratch_bytes_per_lane": 516, "lds_bytes": 10536}}
    assert rest == ["a.hip:7:3: warning: something else"]


def test_built_row_kernels_do_not_spill():
    """A row kernel that spills still sorts correctly, several times slower: the build refuses
    it, and this test reads the reports of the build that produced the library under test."""
    import json

    from cupynumeric_amd import build as B

    reports = sorted(B.OBJ_DIR.glob("*.resources.json"))
    if not reports:
        pytest.skip("no resource reports beside the objects (library built elsewhere)")
    seen_row_kernels = 0
    for report in reports:
        for kernel, use in json.loads(report.read_text()).items():
            for pattern, limit in B.SCRATCH_LIMITS:
                if pattern in kernel:
                    seen_row_kernels += pattern != "onesweep_kernel"
                    assert use.get("scratch_bytes_per_lane", 0) <= limit, (report.name, kernel, use)
    assert seen_row_kernels > 100  # the row kernels of five key widths were all looked at


def test_setter_between_size_query_and_sort_is_refused(lib):
    """A test hook that enlarges the workspace a request needs, called between the size query and the
    sort: the sort works the size out again and returns CPN_ERR_TEMP before it launches anything (the
    pointers below are not device memory)."""
    code = _lib.DTYPE_CODES[np.dtype(np.float32)]
    volume, seg = 1 << 20, 1 << 10  # rows the per-row kernel takes: the header only
    small = lib.cpn_local_sort_temp_bytes(code, volume, seg, 1, 0, 0)
    prev = lib.cpn_set_lds_row_limit(0)  # every row down the global path: histograms, descriptors, key buffers
    try:
        assert lib.cpn_local_sort_temp_bytes(code, volume, seg, 1, 0, 0) > small
        assert lib.cpn_local_sort(code, 4096, 8192, None, volume, seg, 0, 1, 256, small, None) == _lib.CPN_ERR_TEMP
        assert lib.cpn_local_sort_ex(code, 4096, 8192, None, volume, seg, 0, 1, 0, 256, small, None) == _lib.CPN_ERR_TEMP
    finally:
        lib.cpn_set_lds_row_limit(prev)
    # the same for the switch of the merged rows: a row just past the per-row kernels
    seg = 20_000
    merged = lib.cpn_local_sort_temp_bytes(code, seg, seg, 1, 0, 0)
    prev = lib.cpn_set_merge_rows(0)
    try:
        need = lib.cpn_local_sort_temp_bytes(code, seg, seg, 1, 0, 0)
        if need > merged:
            assert lib.cpn_local_sort(code, 4096, 1 << 20, None, seg, seg, 0, 1, 256, merged, None) == _lib.CPN_ERR_TEMP
    finally:
        lib.cpn_set_merge_rows(prev)
    # unknown option bits of cpn_local_sort_ex are refused before anything else happens
    assert lib.cpn_local_sort_ex(code, 4096, 8192, None, 16, 16, 0, 1, 0x80, 256, 4096, None) == _lib.CPN_ERR_UNSUPPORTED


def test_merged_row_levels_and_workspace_over_the_limits(lib):
    """Rows longer than the per-row kernels take: the number of pieces doubles at every multiple of the
    per-row capacity up to the limit of levels, after which the global path takes over; the workspace
    follows (one copy of the rows for one level, two from two levels on, plus the table of chunk starts)."""
    f64, f32 = _lib.DTYPE_CODES[np.dtype(np.float64)], _lib.DTYPE_CODES[np.dtype(np.float32)]

    def temp(code, seg, idx):
        return lib.cpn_local_sort_temp_bytes(code, seg, seg, int(not idx), int(idx), 0)

    # float64, values only: capacity 16384 keys, up to 6 levels -> rows of up to 1 048 576 keys
    cap, prev_bytes = 16384, 0
    for level in range(1, 7):
        seg = cap << level
        b = temp(f64, seg, False)
        copies = 1 if level == 1 else 2
        assert copies * seg * 8 <= b < copies * seg * 8 + (1 << 20), (level, b)
        assert b > prev_bytes
        prev_bytes = b
    # one key past the limit: the global path (one key buffer beside the caller's output, histograms, descriptors)
    over = (cap << 6) + 1
    assert over * 8 < temp(f64, over, False) < over * 12
    # with positions: capacity 14336, 5 levels -> 458 752 keys in two copies of (key, int64 position);
    # one key more: the global path with the keys twice and 4-byte positions
    seg = 14336 << 5
    assert 2 * seg * 16 <= temp(f64, seg, True) < 2 * seg * 16 + (1 << 20)
    assert (seg + 1) * 20 < temp(f64, seg + 1, True) < (seg + 1) * 24
    # 4-byte keys: 2 levels -> 65 536 keys in two copies; one key more: the global path
    assert 2 * 65536 * 4 <= temp(f32, 65536, False) < 2 * 65536 * 4 + (1 << 16)
    assert 65537 * 4 < temp(f32, 65537, False) < 2 * 65536 * 4


def test_no_allocation_calls_in_the_native_sources():
    """cpn_local_sort_static promises that nothing on its path allocates: no translation unit of the
    library calls hipMalloc, hipFree or creates events outside the profiling helper, which is off
    unless a benchmark switches it on."""
    csrc = ROOT / "cupynumeric_amd" / "csrc"
    pattern = re.compile(r"\bhip(Malloc\w*|Free\w*|HostMalloc|EventCreate\w*|StreamCreate\w*|MemPool\w*)\s*\(")
    for path in sorted(csrc.glob("*.h")) + sorted(csrc.glob("*.hip")):
        text = re.sub(r"//[^\n]*", "", path.read_text())
        hits = sorted({m.group(0) for m in pattern.finditer(text)})
        if path.name == "profile.hip":
            assert all(h.startswith("hipEventCreate") for h in hits), hits  # events, only while profiling is on
        else:
            assert hits == [], f"{path.name} calls {hits}"
