"""GPU parity tests: the HIP sort path (through the C ABI and through the Python API on top of
it) against the CPU oracle, the reference's golden vectors and NumPy.  Integer, byte and index
results must be bit-exact; float values are compared by bit pattern as well."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
from conftest import ALL_REAL_DTYPES, COMPLEX_DTYPES, assert_same_bits, case_array, make_input

ALL_DTYPES = ALL_REAL_DTYPES + COMPLEX_DTYPES

import cupynumeric_amd as num
from cupynumeric_amd import _lib
from oracle import sort_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "these tests need a HIP device"
    return torch


@pytest.fixture()
def global_path(lib):
    """Send every row, however short, down the global onesweep path."""
    prev = lib.cpn_set_lds_row_limit(0)
    yield
    lib.cpn_set_lds_row_limit(prev)


def abi_sort(lib, torch, x: np.ndarray, want_values=True, want_indices=False, in_place=False, offset=0):
    """Call cpn_local_sort directly on torch-owned device buffers; returns (values, indices)."""
    x = np.ascontiguousarray(x)
    dev = torch.device("cuda")
    seg = x.shape[-1]
    volume = x.size
    code = _lib.DTYPE_CODES[x.dtype]
    d_in = torch.from_numpy(x.reshape(-1).view(np.uint8).copy()).to(dev)
    d_val = d_in if in_place else (torch.zeros_like(d_in) if want_values else None)
    d_idx = torch.full((volume,), -7, dtype=torch.int64, device=dev) if want_indices else None
    tb = lib.cpn_local_sort_temp_bytes(code, volume, seg, int(want_values), int(want_indices), int(in_place))
    assert tb >= 1024
    temp = torch.full((tb,), 0xFF, dtype=torch.uint8, device=dev)  # a dirty workspace: the call clears what it needs
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.cpn_local_sort(
        code, d_in.data_ptr(), d_val.data_ptr() if want_values else None,
        d_idx.data_ptr() if want_indices else None, volume, seg, offset, 1, temp.data_ptr(), tb, stream,
    )
    assert rc == 0, _lib.status_string(rc)
    assert lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
    vals = d_val.cpu().numpy().view(x.dtype).reshape(x.shape) if want_values else None
    idx = d_idx.cpu().numpy().reshape(x.shape) if want_indices else None
    if not in_place:  # the input must not be touched
        assert np.array_equal(d_in.cpu().numpy(), x.reshape(-1).view(np.uint8))
    return vals, idx


def check_rows(lib, torch, x, what):
    want_v = oracle.local_sort(x, argsort=False)
    want_i = oracle.local_sort(x, argsort=True)
    v, _ = abi_sort(lib, torch, x, want_values=True, want_indices=False)
    assert_same_bits(v, want_v, f"{what} sort")
    _, i = abi_sort(lib, torch, x, want_values=False, want_indices=True)
    assert_same_bits(i, want_i, f"{what} argsort")
    return want_v, want_i


# ---- golden vectors of the reference, through the public API ------------------------------------
def test_reference_golden_vectors(reference_vectors):
    for case in reference_vectors:
        x = case_array(case["input"], case["dtype"], case["shape"])
        a = num.array(x)
        kinds = ["mergesort", "stable"] if case["stable_only"] else ["quicksort", "mergesort", "heapsort", "stable"]
        for kind in kinds:
            where = f"{case['where']} shape={case['shape']} axis={case['axis']} kind={kind}"
            if case["op"] == "sort":
                want = case_array(case["expect"], case["dtype"], case["shape"])
                assert_same_bits(np.asarray(num.sort(a, axis=case["axis"], kind=kind)), want, where)
            else:
                want = np.array(case["expect"], dtype=np.int64).reshape(case["shape"])
                assert_same_bits(np.asarray(num.argsort(a, axis=case["axis"], kind=kind)), want, where)
                assert_same_bits(np.asarray(a.argsort(axis=case["axis"], kind=kind)), want, where)


def test_reference_large_reversed():
    # tests/cpp/integration/test_argsort.cc:379-410
    count = 10000
    want = count - 1 - np.arange(count, dtype=np.int64)
    for x in (np.array([count - i for i in range(count)], dtype=np.int32),
              np.array([count * 1.1 - i for i in range(count)], dtype=np.float64)):
        for kind in ("quicksort", "mergesort", "heapsort", "stable"):
            assert np.array_equal(np.asarray(num.argsort(x, axis=0, kind=kind)), want)


# ---- the reference's integration tests, case for case --------------------------------------------
DIM = 5
SIZES = [(0,), (1), (DIM), (0, 1), (1, 0), (1, 1), (1, DIM), (DIM, 1), (DIM, DIM), (1, 0, 0), (1, 1, 0),
         (1, 0, 1), (1, 1, 1), (DIM, 1, 1), (1, DIM, 1), (1, 1, DIM), (DIM, DIM, DIM)]
SORT_TYPES = ["quicksort", "mergesort", "heapsort", "stable"]


@pytest.mark.parametrize("size", SIZES)
def test_integration_sort_and_argsort(size):
    # tests/integration/test_sort.py:84-125, test_argsort.py (same structure); duplicates are
    # present, so every kind is held to the stable result
    rng = np.random.default_rng(1000 + SIZES.index(size))
    arr_np = rng.integers(-100, 100, size)
    arr_num = num.array(arr_np)
    for kind in SORT_TYPES:
        for axis in range(-arr_np.ndim + 1, arr_np.ndim):
            assert np.array_equal(num.sort(arr_num, axis=axis, kind=kind), np.sort(arr_np, axis=axis, kind="stable"))
            assert np.array_equal(num.sort(arr_num, axis=axis, kind=kind), oracle.sort(arr_np, axis=axis, kind=kind))
            assert np.array_equal(
                num.argsort(arr_num, axis=axis, kind=kind), np.argsort(arr_np, axis=axis, kind="stable")
            )
            assert np.array_equal(
                arr_num.argsort(axis=axis, kind=kind), oracle.argsort(arr_np, axis=axis, kind=kind)
            )
            in_place = num.array(arr_np)
            in_place.sort(axis=axis, kind=kind)
            assert np.array_equal(in_place, np.sort(arr_np, axis=axis, kind="stable"))


@pytest.mark.parametrize("size", [s for s in SIZES if not isinstance(s, int)] + [(DIM,)])
def test_integration_axis_none(size):
    # tests/integration/test_sort.py:194-225
    arr_np = np.random.default_rng(3).integers(-100, 100, size)
    arr_num = num.array(arr_np)
    res = num.sort(arr_num, axis=None)
    assert res.shape == (arr_np.size,)
    assert np.array_equal(res, np.sort(arr_np, axis=None, kind="stable"))
    idx = num.argsort(arr_num, axis=None, kind="stable")
    assert idx.shape == (arr_np.size,)
    assert np.array_equal(idx, np.argsort(arr_np, axis=None, kind="stable"))


def test_random_module_and_flatten():
    a = num.random.randint(-100, 100, (4, 6))
    flat = a.flatten()
    assert flat.shape == (24,)
    assert np.array_equal(num.sort(flat), np.sort(np.asarray(a).reshape(-1), kind="stable"))


# ---- per-row LDS path: every dtype, lengths around every workgroup-shape boundary -------------------
LDS_LENGTHS = [1, 2, 3, 63, 64, 65, 129, 130, 200, 255, 256, 257, 300, 511, 512, 513, 600, 767, 768, 769, 1000, 1023, 1024, 1025, 1535, 1536, 1537, 3071, 3072, 3073, 4095, 4096, 4097, 6143, 6144, 6145, 8191,
               8192, 8193, 12000, 12287, 12288, 12289, 14335, 14336, 14337, 16383, 16384, 16385]


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_lds_rows_all_dtypes(lib, torch_cuda, dtype):
    for seg in LDS_LENGTHS + [2047, 2048, 2049]:
        for rows in (1, 3):
            x = make_input(dtype, (rows, seg), seed=seg * 7 + rows)
            check_rows(lib, torch_cuda, x, f"{np.dtype(dtype)} rows={rows} seg={seg}")


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.float32, np.int64, np.uint64, np.float64])
def test_lds_rows_split_on_leading_bits(lib, torch_cuda, dtype):
    """Values-only sorts of rows whose ties are the same bits take the split on the leading bits and
    the counting inside each bin: rows of distinct keys, rows with pairs and small groups of equal
    keys, keys that differ in few bits or only in low bits, clusters that fill a bin up to and past
    the limit (the radix passes take over), all lengths of the row kernels that have the path."""
    rng = np.random.default_rng(np.dtype(dtype).itemsize * 31 + np.dtype(dtype).num)
    dt = np.dtype(dtype)
    for seg in (129, 200, 256, 257, 300, 512, 513, 700, 768, 769, 1024, 1025, 1500, 1536, 1537, 2048, 2049, 3000, 3072, 3073, 4095, 4096, 4097, 6000, 6144, 6145, 8192, 8193, 12000, 12288,
                12289, 16384):
        rows = 7
        if dt.kind == "f":
            x = rng.standard_normal((rows, seg)).astype(dtype)
            x[1] = rng.random(seg).astype(dtype)                    # [0, 1): most exponent bits idle
            x[2] = (1.0 + rng.random(seg) * 1e-3).astype(dtype)      # keys differ in low bits only
            x[3, : seg // 2] = x[3, seg // 2 : 2 * (seg // 2)]      # every key twice
            x[4] = np.round(x[4] * 64) / 64                          # a few hundred different keys: crowded bins
            x[5, ::3] = dtype(0.5)                                   # one third of the row in one bin
            x[x == 0] = dtype(1.0)                                   # (no zeros: -0.0 would leave the path)
        else:
            info = np.iinfo(dtype)
            x = rng.integers(info.min, info.max, (rows, seg), dtype=dtype, endpoint=True)
            x[1] = rng.integers(0, 1 << 20, seg).astype(dtype)       # 20 varying bits
            x[2] = (rng.integers(0, 200, seg) + 1000).astype(dtype)  # 8 varying bits: bins of equal keys
            x[3, : seg // 2] = x[3, seg // 2 : 2 * (seg // 2)]
            x[4] = (x[4] >> dtype(dt.itemsize * 8 - 9))              # 512 different keys
            x[5, ::3] = x[5, 0]
        x[6] = np.sort(x[6])[::-1]
        want = np.sort(x, axis=-1, kind="stable")
        got, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False)
        assert_same_bits(got, want, f"{dt} seg={seg}")
        got, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False, in_place=True)
        assert_same_bits(got, want, f"{dt} seg={seg} in place")
        # sorts that carry positions take the split as well: ties go by position, which is the stable order
        want_i = np.argsort(x, axis=-1, kind="stable")
        _, got_i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
        assert_same_bits(got_i, want_i, f"{dt} seg={seg} argsort")
        got, got_i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, offset=7)
        assert_same_bits(got, want, f"{dt} seg={seg} values with positions")
        assert_same_bits(got_i, want_i + 7, f"{dt} seg={seg} positions with values")
    # groups of equal keys of every size around the limit of a bin (24; 48 where a bin holds four keys on average)
    for seg, groups in ((256, (23, 24, 25)), (512, (23, 24, 25)), (768, (23, 24, 25)), (1536, (23, 24, 25)), (3072, (23, 24, 25)), (6144, (23, 24, 25)), (8192, (2, 23, 24, 25, 40, 47, 48, 49)), (12288, (24, 25, 48, 49)),
                        (16384, (24, 47, 48, 49, 100))):
        for group in groups:
            base = rng.permutation(seg // group + 1).astype(dtype)
            x = np.repeat(base, group)[:seg].reshape(1, seg).copy()
            rng.shuffle(x[0])
            got, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False)
            assert_same_bits(got, np.sort(x, axis=-1, kind="stable"), f"{dt} seg={seg} groups of {group}")
            _, got_i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
            assert_same_bits(got_i, np.argsort(x, axis=-1, kind="stable"), f"{dt} seg={seg} groups of {group}, argsort")


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.float32])
def test_wave_rows_split_into_ranges(lib, torch_cuda, dtype):
    """One-wave-per-row sorts of 4-byte keys, values only, on rows whose ties are the same bits: the
    split into value ranges with counting inside each range, rows that crowd a range (the radix passes
    take over), keys in a narrow range, pairs of equal keys, every length class of the kernel."""
    rng = np.random.default_rng(np.dtype(dtype).num + 7)
    dt = np.dtype(dtype)
    for seg in (33, 64, 65, 100, 128, 129, 200, 256, 300, 512, 777, 1024):
        rows = 9
        if dt.kind == "f":
            x = rng.standard_normal((rows, seg)).astype(dtype)
            x[1] = rng.random(seg).astype(dtype)
            x[2] = (1.0 + rng.random(seg) * 1e-3).astype(dtype)
            x[3, : seg // 2] = x[3, seg // 2 : 2 * (seg // 2)]
            x[4] = np.round(x[4] * 4) / 4                      # few different keys: crowded ranges
            x[5, ::3] = dtype(0.5)
            x[7, 0] = np.inf                                   # an infinite span: one crowded range
            x[8] = x[8] * dtype(1e30)
            x[x == 0] = dtype(1.0)                             # (no zeros: -0.0 would leave the path)
        else:
            info = np.iinfo(dtype)
            x = rng.integers(info.min, info.max, (rows, seg), dtype=dtype, endpoint=True)
            x[1] = rng.integers(0, 1 << 20, seg).astype(dtype)
            x[2] = (rng.integers(0, 100000, seg) + 5000).astype(dtype)
            x[3, : seg // 2] = x[3, seg // 2 : 2 * (seg // 2)]
            x[4] = (x[4] >> dtype(28)) if dt.kind == "u" else (x[4] // dtype(1 << 28))   # 16 different keys
            x[5, ::3] = x[5, 0]
            x[7, 0], x[7, 1] = info.min, info.max
            x[8] = rng.integers(0, 3, seg).astype(dtype) * dtype(1 << 24) + rng.integers(0, 7, seg).astype(dtype)
        x[6] = np.sort(x[6])[::-1]
        want = np.sort(x, axis=-1, kind="stable")
        got, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False)
        assert_same_bits(got, want, f"{dt} seg={seg}")
        got, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False, in_place=True)
        assert_same_bits(got, want, f"{dt} seg={seg} in place")
        # with positions the split runs as well and ties go by position; rows with zeros and NaNs keep the passes
        want_i = np.argsort(x, axis=-1, kind="stable")
        _, got_i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
        assert_same_bits(got_i, want_i, f"{dt} seg={seg} argsort")
        got, got_i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, offset=3)
        assert_same_bits(got, want, f"{dt} seg={seg} values with positions")
        assert_same_bits(got_i, want_i + 3, f"{dt} seg={seg} positions with values")
        if dt.kind == "f":
            y = x.copy()
            y[0, ::5] = np.nan
            y[1, ::4] = -0.0
            y[1, 1::4] = 0.0
            check_rows(lib, torch_cuda, y, f"{dt} seg={seg} rows with NaN and zeros")
    big = rng.standard_normal((20000, 128)).astype(np.float32).view(np.uint32).view(dtype) if dt.kind != "f" else \
        rng.standard_normal((20000, 128)).astype(dtype)
    got, _ = abi_sort(lib, torch_cuda, big, want_values=True, want_indices=False)
    assert_same_bits(got, np.sort(big, axis=-1, kind="stable"), f"{dt} many rows of 128")
    _, got_i = abi_sort(lib, torch_cuda, big, want_values=False, want_indices=True)
    assert_same_bits(got_i, np.argsort(big, axis=-1, kind="stable"), f"{dt} many rows of 128, argsort")


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
def test_short_float_rows_without_nans_or_negative_zeros(lib, torch_cuda, dtype):
    """Values-only sorts of short rows sort bare images of the keys when no row of a wavefront holds a NaN
    or a -0.0: inputs with none of them at every row length, with infinities, the largest finite values
    and +0.0 (the images next to the one that padding slots hold), in place and out of place; then many rows
    of which a few hold a NaN or a -0.0, so that wavefronts of both kinds run in one launch."""
    dt = np.dtype(dtype)
    rng = np.random.default_rng(dt.num * 17 + 3)
    for seg in list(range(2, 70)) + [80, 81, 95, 96, 100, 113, 127, 128, 129, 161, 200, 255, 256, 257, 321, 385, 449, 512, 600, 768, 900, 1024]:
        rows = 1 + (seg * 5) % 19 if seg % 3 else 150 + seg
        x = rng.standard_normal((rows, seg)).astype(dtype)
        x[0] = x[0, 0]
        if rows > 3:
            x[1, ::2] = np.inf
            x[1, 1::4] = -np.inf
            x[2, ::3] = np.finfo(dtype).max
            x[2, 1::3] = 0.0
            x[3] = np.sort(x[3])[::-1]
        want = np.sort(x, axis=-1, kind="stable")
        got, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False)
        assert_same_bits(got, want, f"{dt} seg={seg} clean rows")
        if seg in (2, 7, 8, 33, 64, 100, 128, 256):
            got, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False, in_place=True)
            assert_same_bits(got, want, f"{dt} seg={seg} clean rows, in place")
    for seg in (8, 24, 64, 128):
        x = rng.standard_normal((30000, seg)).astype(dtype)
        x[::97, 1] = np.nan
        x[5::211, 0] = -0.0
        x[7::211, seg - 1] = 0.0
        got, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False)
        assert_same_bits(got, np.sort(x, axis=-1, kind="stable"), f"{dt} seg={seg} rows with and without special values")


@pytest.mark.parametrize("dtype", [np.uint8, np.float16, np.int32, np.float32, np.int64, np.float64])
def test_short_rows_at_pointers_that_are_not_16_byte_aligned(lib, torch_cuda, dtype):
    """Full rows are moved as 16-byte vectors only when the buffers allow it: the same sorts with input,
    output and index buffers that start 1 ... 3 elements into an allocation, with a guard word on either
    side of the index buffer."""
    torch = torch_cuda
    dt = np.dtype(dtype)
    rng = np.random.default_rng(dt.num + 77)
    word = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[dt.itemsize]
    np_word = {1: np.uint8, 2: np.int16, 4: np.int32, 8: np.int64}[dt.itemsize]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for seg, rows, offs in ((8, 1000, (1, 2, 3)), (32, 777, (3, 0, 1)), (64, 300, (0, 1, 0)), (128, 513, (2, 2, 1)),
                            (256, 100, (1, 3, 3)), (512, 65, (3, 1, 2)), (100, 400, (1, 1, 1))):
        if dt.kind == "f":
            x = rng.standard_normal((rows, seg)).astype(dtype)
            x[::7, 0] = np.nan
            x[3::11, seg - 1] = -0.0
        else:
            x = rng.integers(np.iinfo(dtype).min, np.iinfo(dtype).max, (rows, seg), endpoint=True, dtype=dtype)
        n = x.size
        order = np.argsort(x.astype(np.float32) if dt == np.float16 else x, axis=-1, kind="stable")
        for want_values, want_indices in ((True, False), (False, True), (True, True)):
            d_in = torch.zeros(n + 8, dtype=word, device="cuda")
            d_in[offs[0]:offs[0] + n] = torch.from_numpy(x.reshape(-1).view(np_word).copy()).cuda()
            d_out = torch.zeros(n + 8, dtype=word, device="cuda")
            d_idx = torch.full((n + 8,), -7, dtype=torch.int64, device="cuda")
            tb = lib.cpn_local_sort_temp_bytes(_lib.DTYPE_CODES[dt], n, seg, int(want_values), int(want_indices), 0)
            temp = torch.full((tb,), 0xFF, dtype=torch.uint8, device="cuda")
            rc = lib.cpn_local_sort(_lib.DTYPE_CODES[dt], d_in.data_ptr() + offs[0] * dt.itemsize,
                                    d_out.data_ptr() + offs[1] * dt.itemsize if want_values else None,
                                    d_idx.data_ptr() + offs[2] * 8 if want_indices else None, n, seg, 0, 1,
                                    temp.data_ptr(), tb, stream)
            assert rc == 0, _lib.status_string(rc)
            where = f"{dt} rows of {seg}, offsets {offs}, values={want_values}, indices={want_indices}"
            if want_values:
                got = d_out[offs[1]:offs[1] + n].cpu().numpy().view(dtype).reshape(rows, seg)
                assert_same_bits(got, np.take_along_axis(x, order, axis=-1), where)
            if want_indices:
                got = d_idx.cpu().numpy()
                assert np.array_equal(got[offs[2]:offs[2] + n].reshape(rows, seg), order), where
                assert (got[:offs[2]] == -7).all() and (got[offs[2] + n:] == -7).all(), where + ": wrote outside the index buffer"


REAL_DTYPES = [np.bool_, np.int8, np.uint8, np.int16, np.uint16, np.float16, np.int32, np.uint32, np.float32,
               np.int64, np.uint64, np.float64]


@pytest.mark.parametrize("dtype", REAL_DTYPES)
def test_rows_of_up_to_128_keys_through_the_bitonic_network(lib, torch_cuda, dtype):
    """Rows of 2 ... 512 real keys (how far the network goes depends on the key width): every length up to 69
    and both sides of every change of lanes per row and of elements per lane above (full and partly filled rows),
    row counts that leave the last wavefront partly empty, rows of equal keys, of two keys, sorted and
    reversed rows, NaNs of several payloads and zeros of both signs (ties go by position: the stable
    order), the extreme values of the type (the image that padding slots hold), values and positions
    together, in place, an index offset; and the ranking kernels give the same bits with the network
    switched off."""
    dt = np.dtype(dtype)
    rng = np.random.default_rng(dt.num * 13 + 5)
    for seg in list(range(2, 70)) + [80, 81, 95, 96, 97, 100, 112, 113, 126, 127, 128, 129, 160, 161, 192, 193, 224, 225, 255, 256,
                                     257, 320, 321, 384, 385, 448, 449, 511, 512, 513, 640, 641, 768, 769, 896, 897, 1000, 1023, 1024, 1025]:
        rows = 1 + (seg * 7) % 23 if seg % 3 else 200 + seg
        x = make_input(dtype, (rows, seg), seed=seg)
        x[0] = x[0, 0]
        if rows > 4:
            x[1] = np.sort(x[1])
            x[2] = np.sort(x[2])[::-1]
            x[3] = np.where(rng.random(seg) < 0.5, x[3, 0], x[3, -1])
        if rows > 6:
            if dt.kind == "f":
                x[4, ::3] = np.nan
                x[4, 1::3] = -0.0
                x[4, 2::3] = 0.0
                x[5] = np.where(rng.random(seg) < 0.3, np.inf, x[5])
                x[5, ::4] = -np.inf
                x[6, ::2] = np.finfo(dtype).max
                nan_bits = x[4].view(f"u{dt.itemsize}")
                nan_bits[::6] |= 1  # another NaN payload
            elif dt.kind in "iu":
                x[4, ::2] = np.iinfo(dtype).max
                x[5, ::2] = np.iinfo(dtype).min
                x[6] = rng.integers(0, 3, seg).astype(dtype)
        want_v, want_i = check_rows(lib, torch_cuda, x, f"{dt} seg={seg}")
        if seg in (2, 3, 17, 32, 33, 64, 65, 100, 128, 161, 256, 321, 512, 641, 1024):
            v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, offset=-5)
            assert_same_bits(v, want_v, f"{dt} seg={seg} values+positions")
            assert_same_bits(i, want_i - 5, f"{dt} seg={seg} values+positions, offset")
            v, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False, in_place=True)
            assert_same_bits(v, want_v, f"{dt} seg={seg} in place")
    prev = lib.cpn_set_bitonic_rows(0)
    try:
        for seg in (2, 20, 32, 33, 64, 65, 128):
            check_rows(lib, torch_cuda, make_input(dtype, (77, seg), seed=seg), f"{dt} seg={seg}, ranking kernels")
    finally:
        assert lib.cpn_set_bitonic_rows(prev) == 0
    assert lib.cpn_set_bitonic_rows(1) == 1


COUNT16_CHILD = r"""
import numpy as np
import cupynumeric_amd as num
from cupynumeric_amd import _lib
lib = _lib.load()
rng = np.random.default_rng(5)
for dtype in (np.float16, np.int16, np.uint16):
    for seg in (4097, 6000, 8191, 8192, 9001, 16384):
        if dtype == np.float16:
            x = rng.standard_normal((5, seg)).astype(dtype)
            x[1, ::5] = np.nan
            x[1, 1::5] = -0.0
            x[1, 2::5] = 0.0
            x[2] = x[2, 0]
            b = x[3].view(np.uint16)
            b[::7] = 0xFE01  # negative NaN with a payload
        else:
            info = np.iinfo(dtype)
            x = rng.integers(info.min, info.max, (5, seg), dtype=dtype, endpoint=True)
            x[2] = x[2, 0]
        lib.cpn_profile_enable(1)
        _lib.profile_collect()
        got = np.asarray(num.sort(num.array(x)))
        labels = {k for k, _ in _lib.profile_collect()}
        lib.cpn_profile_enable(0)
        assert "count16_row_sort" in labels, (dtype, seg, labels)
        want = np.sort(x, axis=-1, kind="stable")
        u = np.uint16
        assert np.array_equal(got.view(u), want.view(u)), (dtype, seg)
print("ok")
"""


def test_counting_kernel_for_rows_of_up_to_8192_keys_behind_its_switch(torch_cuda):
    """Plain sorts of 4097 ... 8192 two-byte keys take the radix shapes by default; the counting kernel
    for such rows runs when CPN_SORT_COUNT16_MIN_ROW, read when the library is loaded, lowers its
    threshold: a child process with that setting sorts rows with NaNs of both signs, payloads, zeros
    of both signs and constant rows, checks the bits against NumPy's stable sort and that the counting
    kernel is the one that ran."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, CPN_SORT_COUNT16_MIN_ROW="4097", PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    out = subprocess.run([sys.executable, "-c", COUNT16_CHILD], env=env, cwd=root, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout[-1000:] + out.stderr[-3000:]


TWO_BYTE_LONG_ROWS_CHILD = r"""
import numpy as np
import cupynumeric_amd as num
from cupynumeric_amd import _lib
lib = _lib.load()
rng = np.random.default_rng(6)
u = np.uint16
for dtype in (np.float16, np.int16, np.uint16):
    for seg in (8193, 9001, 12000, 16383, 16384, 16385, 20001, 32768):
        if dtype == np.float16:
            x = rng.standard_normal((4, seg)).astype(dtype)
            x[1, ::5] = np.nan
            x[1, 1::5] = -0.0
            x[1, 2::5] = 0.0
            x[2] = x[2, 0]
            b = x[3].view(u)
            b[::7] = 0xFE01  # negative NaN with a payload
        else:
            info = np.iinfo(dtype)
            x = rng.integers(info.min, info.max, (4, seg), dtype=dtype, endpoint=True)
            x[2] = x[2, 0]
        lib.cpn_profile_enable(1)
        _lib.profile_collect()
        got = np.asarray(num.sort(num.array(x)))
        labels = {k for k, _ in _lib.profile_collect()}
        lib.cpn_profile_enable(0)
        assert labels == ({"lds_row_sort"} if seg <= 16384 else {"count16_row_sort"}), (dtype, seg, labels)
        order = np.argsort(x.astype(np.float32), axis=-1, kind="stable") if dtype == np.float16 else np.argsort(x, axis=-1, kind="stable")
        want = np.take_along_axis(x, order, axis=-1)
        assert np.array_equal(got.view(u), want.view(u)), (dtype, seg)
print("ok")
"""


def test_two_byte_rows_of_8193_to_16384_keys_through_the_radix_shape(torch_cuda):
    """With the counting kernel starting at 16 385 keys (CPN_SORT_COUNT16_MIN_ROW, read when the library is
    loaded), plain sorts of 8193 ... 16 384 two-byte keys take the radix kernel in its 1024 x 16 shape, rows
    shorter than the tile dealt in equal shares, and longer rows still the counting kernel: a child process
    checks bits and which kernel ran, with NaNs of both signs, payloads, zeros of both signs and constant rows."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, CPN_SORT_COUNT16_MIN_ROW="16385", PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    out = subprocess.run([sys.executable, "-c", TWO_BYTE_LONG_ROWS_CHILD], env=env, cwd=root, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout[-1000:] + out.stderr[-3000:]


@pytest.mark.parametrize("dtype", [np.float16, np.int16, np.uint16])
def test_two_byte_rows_of_up_to_57344_keys_are_counted(lib, torch_cuda, dtype):
    """Plain sorts of rows of 16 385 ... 57 344 two-byte keys: the counting kernel with 32 and 56 keys per thread
    (zeros and NaNs in input order); one key more, and the same rows with positions, take the global path."""
    u = np.uint16
    for seg in (16385, 16392, 20001, 32767, 32768, 32769, 40003, 49152, 57343, 57344, 57345):
        x = make_input(dtype, (5, seg), seed=seg)
        x[2] = x[2, 0]
        x[3] = np.sort(x[3])[::-1]
        lib.cpn_profile_enable(1)
        _lib.profile_collect()
        v, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False)
        labels = {k for k, _ in _lib.profile_collect()}
        lib.cpn_profile_enable(0)
        assert ("count16_row_sort" in labels) == (seg <= 57344), (seg, labels)
        assert_same_bits(v, oracle.local_sort(x, argsort=False), f"{np.dtype(dtype)} seg={seg}")
        v, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False, in_place=True)
        assert_same_bits(v, oracle.local_sort(x, argsort=False), f"{np.dtype(dtype)} seg={seg} in place")
        check_rows(lib, torch_cuda, x, f"{np.dtype(dtype)} seg={seg}")  # (also the argsort of the same rows)


def test_lds_many_short_rows(lib, torch_cuda):
    for dtype, shape in [(np.float64, (3000, 37)), (np.int8, (5000, 5)), (np.float16, (700, 401)), (np.uint32, (129, 1024))]:
        check_rows(lib, torch_cuda, make_input(dtype, shape, seed=11), f"{np.dtype(dtype)} {shape}")


@pytest.mark.parametrize("dtype", [np.int64, np.uint64, np.float64, np.complex64, np.complex128])
@pytest.mark.parametrize("seg", [600, 1024, 1500, 4096, 6000, 8192])
def test_lds_rows_leading_digit_shortcut(lib, torch_cuda, dtype, seg):
    """Wide keys in the row kernels: rows that the leading digits order completely, rows with ties on
    the leading digits whose low digits are out of order (the check must fail and every pass run),
    and rows with ties that happen to be in order; mixed in one launch."""
    rng = np.random.default_rng(seg + np.dtype(dtype).itemsize)
    rows = 12
    if np.dtype(dtype).kind == "c":
        comp = np.float32 if dtype == np.complex64 else np.float64
        re = rng.standard_normal((rows, seg)).astype(comp)
        im = rng.standard_normal((rows, seg)).astype(comp)
        re[3:6] = rng.integers(0, 3, (3, seg)).astype(comp)           # ties on the real part: imag decides
        im[6:8] = np.sort(im[6:8], axis=-1)
        re[6:8] = np.repeat(np.sort(rng.integers(0, 4, (2, seg // 4 + 1)), axis=-1), 4, axis=-1)[:, :seg]
        re[8, ::7] = np.nan
        im[9, ::5] = np.nan
        x = (re + 1j * im).astype(dtype)
        x.real[8, ::7] = np.nan
    else:
        info_bits = 8 * np.dtype(dtype).itemsize
        lo = rng.integers(0, 1 << 40, (rows, seg), dtype=np.uint64)
        hi = rng.integers(0, 1 << 23, (rows, seg), dtype=np.uint64) << np.uint64(40)
        hi[3:6] = rng.integers(0, 5, (3, seg), dtype=np.uint64) << np.uint64(40)     # heavy ties, low bits random
        hi[6:8] = np.sort(rng.integers(0, 9, (2, seg), dtype=np.uint64), axis=-1) << np.uint64(40)
        lo[6:8] = np.sort(lo[6:8], axis=-1)                                            # ties, already in order
        lo[8] &= np.uint64(0xFF)                                                       # few low digits vary
        bits = hi | lo
        if np.dtype(dtype).kind == "f":
            bits = (bits & np.uint64((1 << 62) - 1)) | (np.uint64(0x3F) << np.uint64(56)) & np.uint64((1 << 64) - 1)
            x = bits.view(np.float64).copy()
            x[9, ::3] *= -1.0
            x[10, ::11] = np.nan
            x[10, 1::11] = -0.0
            x[10, 2::11] = 0.0
        else:
            x = bits.view(dtype).copy()
            assert info_bits == 64
    check_rows(lib, torch_cuda, x, f"{np.dtype(dtype)} seg={seg} shortcut")
    v, i = abi_sort(lib, torch_cuda, x.copy(), want_values=True, want_indices=True, in_place=True)
    assert_same_bits(v, oracle.local_sort(x, argsort=False), "in place values")
    assert_same_bits(i, oracle.local_sort(x, argsort=True), "in place indices")


@pytest.mark.parametrize("dtype", [np.int64, np.float64, np.complex128])
@pytest.mark.parametrize("seg", [200, 512, 1024, 3000])
def test_row_shortcut_repairs_short_tie_runs(lib, torch_cuda, dtype, seg):
    """After the leading-digit passes the row kernels repair short runs of ties with odd-even
    transposition and fall back to every pass for long ones.  Each row holds runs of one length
    whose low digits descend (a run of L needs L exchange phases), with repeated keys inside the
    runs so that stability shows; runs of 2..8 are repaired, 9 and more take the fallback."""
    lengths = [2, 3, 5, 8, 9, 12, 40]
    pos = np.arange(seg, dtype=np.uint64)
    rows = []
    for L in lengths:
        run, k = pos // np.uint64(L), pos % np.uint64(L)
        lead = (run * np.uint64(0x010101)) << np.uint64(24) | (run & np.uint64(0xFF)) << np.uint64(16)
        for low in ((np.uint64(L) - k), (np.uint64(L) - k) // np.uint64(2)):
            rows.append(lead | low * np.uint64(0x0101))
    bits = np.stack(rows)
    if np.dtype(dtype).kind == "i":
        x = bits.view(np.int64)
    else:
        x = (bits | np.uint64(0x3FF0) << np.uint64(48)).view(np.float64)  # positive normal numbers, same order
        if np.dtype(dtype).kind == "c":
            x = x + 0j
    check_rows(lib, torch_cuda, np.ascontiguousarray(x), f"{np.dtype(dtype)} seg={seg} tie runs")


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.float32])
@pytest.mark.parametrize("seg", [40, 64, 130, 256])
def test_short_rows_of_4_byte_keys_take_the_shortcut(lib, torch_cuda, dtype, seg):
    """Rows of up to 256 four-byte keys sort by their 2 or 3 leading digits first; ties there
    (runs of 2..40 keys whose last byte descends, with repeats) are repaired or take every pass."""
    pos = np.arange(seg, dtype=np.uint32)
    rows = []
    for L in [2, 3, 5, 8, 9, 12, 40]:
        run, k = pos // np.uint32(L), pos % np.uint32(L)
        lead = (run * np.uint32(0x0101)) << np.uint32(16) | (run & np.uint32(0xFF)) << np.uint32(8)
        rows.append(lead | (np.uint32(L) - k))
        rows.append(lead | (np.uint32(L) - k) // np.uint32(2))
    rng = np.random.default_rng(seg)
    rows.append(rng.integers(0, 1 << 32, seg, dtype=np.uint64).astype(np.uint32))  # no ties to speak of
    x = np.ascontiguousarray(np.stack(rows).view(dtype))
    check_rows(lib, torch_cuda, x, f"{np.dtype(dtype)} seg={seg} tie runs")
    many = make_input(dtype, (500, seg), seed=seg)
    check_rows(lib, torch_cuda, many, f"{np.dtype(dtype)} seg={seg} random rows")


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
@pytest.mark.parametrize("seg", [33, 64, 100, 257, 512, 1000, 1024])
def test_short_float_rows_keys_only_with_zeros_and_nans(lib, torch_cuda, dtype, seg):
    """Keys-only sorts of short float rows rebuild every key from its sorted image except zeros and NaNs,
    whose bits (signs, payloads) are put back in input order from a second look at the input: rows of
    only zeros of both signs, only NaNs of several payloads, mixtures, rows without either, sorted out
    of place and in place."""
    if np.dtype(dtype).itemsize == 8 and seg > 512:
        pytest.skip("8-byte rows of this length take the workgroup kernel")
    dt = np.dtype(dtype)
    ub = {2: np.uint16, 4: np.uint32, 8: np.uint64}[dt.itemsize]
    rng = np.random.default_rng(seg * dt.itemsize)
    rows = 24
    x = (rng.standard_normal((rows, seg)) * 4).astype(dtype)
    bits = x.view(ub)
    sign = ub(1) << ub(8 * dt.itemsize - 1)
    nan_patterns = np.array([np.array(np.nan, dtype=dtype).view(ub), np.array(np.nan, dtype=dtype).view(ub) | sign,
                             np.array(np.nan, dtype=dtype).view(ub) | ub(1), np.array(np.nan, dtype=dtype).view(ub) | ub(5) | sign], dtype=ub)
    bits[0] = np.where(rng.random(seg) < 0.5, sign, ub(0))                         # zeros only
    bits[1] = nan_patterns[rng.integers(0, 4, seg)]                                # NaNs only
    for r in range(2, 12):                                                         # mixtures of growing density
        m = rng.random(seg)
        p = (r - 1) / 20
        bits[r] = np.where(m < p, np.where(rng.random(seg) < 0.5, sign, ub(0)), bits[r])
        bits[r] = np.where(m > 1 - p, nan_patterns[rng.integers(0, 4, seg)], bits[r])
    bits[12, ::3] = sign                                                           # -0.0 only among ordinary keys
    bits[13, 5] = nan_patterns[3]                                                  # a single NaN
    x = bits.view(dtype)
    want = oracle.local_sort(x, argsort=False)
    v, _ = abi_sort(lib, torch_cuda, x, want_values=True)
    assert_same_bits(v, want, f"{dt} seg={seg} keys only")
    v, _ = abi_sort(lib, torch_cuda, x.copy(), want_values=True, in_place=True)
    assert_same_bits(v, want, f"{dt} seg={seg} keys only, in place")


# ---- global onesweep path ---------------------------------------------------------------------------
GLOBAL_LENGTHS = [1, 2, 100, 4097, 8191, 8192, 8193, 16383, 16384, 16385, 3 * 16384 + 5, 100003]


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_global_path_all_dtypes(lib, torch_cuda, global_path, dtype):
    for seg in GLOBAL_LENGTHS:
        x = make_input(dtype, (seg,), seed=seg)
        check_rows(lib, torch_cuda, x, f"{np.dtype(dtype)} seg={seg} (global)")


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.float64, np.uint8, np.float16, np.complex64, np.complex128])
def test_global_path_batched_rows(lib, torch_cuda, global_path, dtype):
    # rows shorter than, equal to and longer than a tile; the look-back must stop at row starts
    for shape in [(50, 129), (7, 4096), (5, 8192), (3, 8193), (5, 16384), (3, 16385), (4, 40011), (300, 1)]:
        check_rows(lib, torch_cuda, make_input(dtype, shape, seed=shape[0]), f"{np.dtype(dtype)} {shape} (global)")


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.int64, np.float64, np.float16, np.uint8, np.complex64, np.complex128])
def test_global_path_default_dispatch(lib, torch_cuda, dtype):
    # long rows take the global path without any override
    for shape in [(1 << 20,), (3, 70001), (2, 8193), (2, 16385)]:
        check_rows(lib, torch_cuda, make_input(dtype, shape, seed=5), f"{np.dtype(dtype)} {shape}")


@pytest.mark.parametrize("path", ["lds", "global"])
@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.float32, np.int64, np.complex64, np.complex128])
def test_outputs_in_place_and_offset(lib, torch_cuda, path, dtype):
    prev = lib.cpn_set_lds_row_limit(0 if path == "global" else -1)
    try:
        for shape in [(4, 3000), (2, 9001)]:
            x = make_input(dtype, shape, seed=9)
            want_v = oracle.local_sort(x, argsort=False)
            want_i = oracle.local_sort(x, argsort=True, offset=1000)
            v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, offset=1000)
            assert_same_bits(v, want_v, f"values+indices {shape}")
            assert_same_bits(i, want_i, f"values+indices {shape}")
            v, _ = abi_sort(lib, torch_cuda, x, want_values=True, in_place=True)
            assert_same_bits(v, want_v, f"in place {shape}")
            v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, in_place=True, offset=-5)
            assert_same_bits(v, want_v, f"in place + indices {shape}")
            assert_same_bits(i, want_i - 1005, f"in place + indices {shape}")
    finally:
        lib.cpn_set_lds_row_limit(prev)


@pytest.fixture()
def wide_rows(lib):
    """Rows from 5000 elements on take the kernels with 64-bit counts, descriptors and row positions
    (by default only rows of 2^30 elements and more do)."""
    prev = lib.cpn_set_wide_row_threshold(5000)
    yield
    lib.cpn_set_wide_row_threshold(prev)


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_global_path_wide_rows(lib, torch_cuda, wide_rows, dtype):
    """The 64-bit variant of the global path: tiles are 8192 keys of 4 bytes or less, 16 384 keys of 8 bytes and 8192 of 16 bytes there."""
    for shape in [(5000,), (8192,), (8193,), (3, 20011), (100003,), (2, 4 * 8192)]:
        x = make_input(dtype, shape, seed=shape[-1])
        check_rows(lib, torch_cuda, x, f"{np.dtype(dtype)} {shape} (wide rows)")
    x = make_input(dtype, (2, 30001), seed=3)
    want_v = oracle.local_sort(x, argsort=False)
    want_i = oracle.local_sort(x, argsort=True, offset=-7)
    v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, in_place=True, offset=-7)
    assert_same_bits(v, want_v, "wide rows, in place + indices")
    assert_same_bits(i, want_i, "wide rows, in place + indices")
    # rows below the threshold in the same process keep the 32-bit kernels
    check_rows(lib, torch_cuda, make_input(dtype, (4999,), seed=1), f"{np.dtype(dtype)} below the threshold")


def test_wide_row_threshold_setter(lib):
    prev = lib.cpn_set_wide_row_threshold(12345)
    assert lib.cpn_set_wide_row_threshold(-1) == 12345
    assert lib.cpn_set_wide_row_threshold(prev) == -1
    code = _lib.DTYPE_CODES[np.dtype(np.float32)]
    narrow = lib.cpn_local_sort_temp_bytes(code, 1 << 20, 1 << 20, 0, 1, 0)
    lib.cpn_set_wide_row_threshold(1000)
    wide = lib.cpn_local_sort_temp_bytes(code, 1 << 20, 1 << 20, 0, 1, 0)
    lib.cpn_set_wide_row_threshold(prev)
    assert wide > narrow  # 64-bit row positions and descriptors


# ---- adversarial key distributions ------------------------------------------------------------------
@pytest.mark.parametrize("path", ["lds", "global"])
def test_skewed_and_degenerate_keys(lib, torch_cuda, path):
    prev = lib.cpn_set_lds_row_limit(0 if path == "global" else -1)
    try:
        n = 8192 if path == "lds" else 200001
        rng = np.random.default_rng(4)
        iota = np.arange(n, dtype=np.int64)
        cases = {
            "all equal": np.full(n, -3, dtype=np.int32),
            "sorted": iota.astype(np.int64),
            "reversed": (-iota).astype(np.int64),
            "16 distinct int64": rng.integers(-(2**63), 2**63 - 1, 16, dtype=np.int64)[rng.integers(0, 16, n)],
            "two values": rng.integers(0, 2, n).astype(np.uint16) * np.uint16(40000),
            "all NaN": np.full(n, np.nan, dtype=np.float32),
            "NaN and zeros": rng.choice(np.array([np.nan, 0.0, -0.0], dtype=np.float64), n),
            "bool": rng.integers(0, 2, n).astype(np.bool_),
            "complex real-only": rng.standard_normal(n).astype(np.complex64),
            "complex NaN classes": rng.choice(
                np.array([complex(np.nan, 1), complex(1, np.nan), complex(np.nan, np.nan), 1 + 1j, complex(1, -0.0)],
                         dtype=np.complex128), n),
        }
        for name, x in cases.items():
            _, want_i = check_rows(lib, torch_cuda, x, f"{name} ({path})")
            if name in ("all equal", "sorted", "all NaN"):
                assert np.array_equal(want_i, iota)
            if name == "reversed":
                assert np.array_equal(want_i, iota[::-1])
        perm = rng.permutation(n)
        inv = np.empty(n, dtype=np.int64)
        inv[perm] = iota
        _, i = abi_sort(lib, torch_cuda, perm.astype(np.uint32), want_values=False, want_indices=True)
        assert np.array_equal(i, inv)  # argsort of a permutation is its inverse
    finally:
        lib.cpn_set_lds_row_limit(prev)


# ---- passes on which all keys agree are skipped; the buffers used then depend on how many remain ----
@pytest.mark.parametrize("dtype,nbytes", [(np.uint32, 4), (np.int64, 8), (np.float32, 4), (np.uint16, 2)])
def test_global_path_skipped_passes(lib, torch_cuda, global_path, dtype, nbytes):
    rng = np.random.default_rng(21)
    n = 40000
    ub = {2: np.uint16, 4: np.uint32, 8: np.uint64}[nbytes]
    subsets = range(1 << nbytes) if nbytes <= 4 else [0, 1, 0x80, 0x11, 0x07, 0x70, 0xFE, 0x55, 0xFF]
    for mask in subsets:
        bits_ = np.zeros(n, dtype=ub)
        const = ub(int(rng.integers(0, 1 << 62)) & ((1 << (8 * nbytes)) - 1))
        for b in range(nbytes):
            byte = rng.integers(0, 256, n).astype(ub) if (mask >> b) & 1 else np.full(n, (const >> ub(8 * b)) & ub(0xFF), dtype=ub)
            bits_ |= byte << ub(8 * b)
        x = bits_.view(dtype)
        if np.dtype(dtype).kind == "f":
            x = np.where(np.isnan(x), np.float32(1.5), x).astype(dtype)
        want_v = oracle.local_sort(x, argsort=False)
        want_i = oracle.local_sort(x, argsort=True)
        what = f"{np.dtype(dtype)} varying-bytes mask {mask:#x}"
        v, _ = abi_sort(lib, torch_cuda, x, want_values=True)
        assert_same_bits(v, want_v, what + " sort")
        _, i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True, offset=3)
        assert_same_bits(i, want_i + 3, what + " argsort")
        v, _ = abi_sort(lib, torch_cuda, x, want_values=True, in_place=True)
        assert_same_bits(v, want_v, what + " in place")
        v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, in_place=True)
        assert_same_bits(v, want_v, what + " in place + indices")
        assert_same_bits(i, want_i, what + " in place + indices")


def test_global_path_skipping_needs_every_row(lib, torch_cuda, global_path):
    # a byte that is constant inside each row but differs between rows may be skipped; a byte
    # that varies in one row only may not
    rng = np.random.default_rng(22)
    rows, seg = 6, 20000
    x = rng.integers(0, 256, (rows, seg)).astype(np.uint32)  # byte 0 varies everywhere
    x |= (np.arange(rows, dtype=np.uint32)[:, None] + 1) << 8  # byte 1: constant per row
    x[3] |= rng.integers(0, 256, seg).astype(np.uint32) << 16  # byte 2 varies in row 3 only
    check_rows(lib, torch_cuda, x, "per-row constant bytes")
    check_rows(lib, torch_cuda, x.astype(np.int64), "per-row constant bytes, int64")


# ---- rows of up to twice the LDS capacity: two sorted halves, merged -----------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.uint32, np.float64, np.int64, np.uint64])
def test_rows_sorted_as_merged_halves(lib, torch_cuda, dtype):
    """Row lengths on both sides of the ranges that are sorted in 2, 4 and 8 pieces and merged (up to
    16 384 keys a piece; 14 336 for 8-byte keys with positions), odd and even lengths, rows with many ties
    across the pieces (stability of the merge), sorted, reversed and constant rows, special float values,
    values and positions together, in place, an index offset; and the same requests with the path
    switched off give the same bits through the global path."""
    dt = np.dtype(dtype)
    rng = np.random.default_rng(dt.num * 7 + 1)
    lengths = [16385, 16386, 20001, 28672, 28673, 32767, 32768, 32769, 40003, 57344, 57345, 65535, 65536, 65537]
    if dt.itemsize == 8:
        lengths += [14337, 14338, 114688, 114689, 131072, 131073]
    header = lib.cpn_local_sort_temp_bytes(_lib.DTYPE_CODES[dt], 0, 0, 1, 0, 0)
    for seg in lengths:
        rows = 5
        x = make_input(dtype, (rows, seg), seed=seg)
        x[1] = np.sort(x[1])
        x[2] = np.sort(x[2])[::-1]
        if dt.kind == "f":
            x[3] = rng.integers(0, 6, seg).astype(dtype)                 # six different keys: ties everywhere
            x[4, ::7] = np.nan
            x[4, 1::7] = -0.0
            x[4, 2::7] = 0.0
        else:
            x[3] = rng.integers(0, 6, seg).astype(dtype)
            x[4] = x[4, 0]
        check_rows(lib, torch_cuda, x, f"{dt} seg={seg}")
        want_v, want_i = oracle.local_sort(x, argsort=False), oracle.local_sort(x, argsort=True)
        v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, offset=1000)
        assert_same_bits(v, want_v, f"{dt} seg={seg} values+positions")
        assert_same_bits(i, want_i + 1000, f"{dt} seg={seg} values+positions, offset")
        v, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False, in_place=True)
        assert_same_bits(v, want_v, f"{dt} seg={seg} in place")
    # the path is the one that runs: its workspace is the table of chunk starts and the rows once (plus
    # positions; twice from two levels of merging on), not the global layout
    code, seg, rows = _lib.DTYPE_CODES[dt], 20000, 4
    merged_bytes = lib.cpn_local_sort_temp_bytes(code, rows * seg, seg, 1, 0, 0)
    table = (rows * ((seg + 2047) // 2048 + 2) * 4 + 255) // 256 * 256
    assert merged_bytes == header + table + (rows * seg * dt.itemsize + 255) // 256 * 256
    table = (rows * ((40000 + 2047) // 2048 + 4) * 4 + 255) // 256 * 256
    assert lib.cpn_local_sort_temp_bytes(code, rows * 40000, 40000, 1, 1, 0) == \
        header + table + 2 * ((rows * 40000 * dt.itemsize + 255) // 256 * 256 + (rows * 40000 * 8 + 255) // 256 * 256)
    prev = lib.cpn_set_merge_rows(0)
    try:
        assert lib.cpn_local_sort_temp_bytes(code, rows * seg, seg, 1, 0, 0) != merged_bytes
        x = make_input(dtype, (3, 20001), seed=5)
        check_rows(lib, torch_cuda, x, f"{dt} global path, merge switched off")
    finally:
        lib.cpn_set_merge_rows(prev)
    assert lib.cpn_local_sort_temp_bytes(code, rows * seg, seg, 1, 0, 0) == merged_bytes


@pytest.mark.parametrize("dtype", [np.float64, np.int64])
def test_rows_merged_over_five_and_six_levels(lib, torch_cuda, dtype):
    """8-byte keys: 32 pieces (five levels of merging; with positions the most there is) and 64 pieces (six
    levels, values only), and rows one key past each limit, which take the global path and must give the
    same bits."""
    dt = np.dtype(dtype)
    code = _lib.DTYPE_CODES[dt]
    x = make_input(dtype, (2, 300_001), seed=41)  # 32 pieces, values and positions
    x[1, ::3] = x[1, 0]                            # ties across every piece
    check_rows(lib, torch_cuda, x, f"{dt} 2 x 300001, five levels")
    v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, offset=3)
    assert_same_bits(v, oracle.local_sort(x, argsort=False), f"{dt} five levels, values+positions")
    assert_same_bits(i, oracle.local_sort(x, argsort=True) + 3, f"{dt} five levels, positions")
    y = make_input(dtype, (1, 600_001), seed=42)  # 64 pieces, values only
    v, _ = abi_sort(lib, torch_cuda, y, want_values=True, want_indices=False)
    assert_same_bits(v, oracle.local_sort(y, argsort=False), f"{dt} 1 x 600001, six levels")
    v, _ = abi_sort(lib, torch_cuda, y, want_values=True, want_indices=False, in_place=True)
    assert_same_bits(v, oracle.local_sort(y, argsort=False), f"{dt} six levels, in place")
    # the limits themselves and one key past them (the global path)
    for seg, idx in [(1_048_576, False), (1_048_577, False), (458_752, True), (458_753, True)]:
        z = make_input(dtype, (1, seg), seed=seg)
        per_key = lib.cpn_local_sort_temp_bytes(code, seg, seg, int(not idx), int(idx), 0) / seg
        # merged rows hold two copies of the keys (and of int64 positions); the global path one key buffer
        # beside the caller's output, or the keys twice and 4-byte positions
        assert per_key >= (32 if idx else 16) if seg in (1_048_576, 458_752) else per_key < (24 if idx else 12)
        v, i = abi_sort(lib, torch_cuda, z, want_values=not idx, want_indices=idx)
        if idx:
            assert_same_bits(i, oracle.local_sort(z, argsort=True), f"{dt} seg={seg} argsort")
        else:
            assert_same_bits(v, oracle.local_sort(z, argsort=False), f"{dt} seg={seg} sort")


def test_merged_rows_many_rows_and_narrow_keys_stay_out(lib, torch_cuda):
    # many rows: every workgroup of the merge finds its own part of its own row
    x = make_input(np.float32, (300, 17000), seed=3)
    check_rows(lib, torch_cuda, x, "300 rows of 17000")
    # 2-byte, 1-byte and complex keys of such lengths take the global path
    for dtype in (np.float16, np.uint8, np.complex64):
        x = make_input(dtype, (3, 17000), seed=4)
        check_rows(lib, torch_cuda, x, f"{np.dtype(dtype)} rows of 17000")


# ---- swapaxes copy ------------------------------------------------------------------------------------
@pytest.mark.parametrize("elem", [np.uint8, np.float16, np.int32, np.float64, np.complex128])
def test_swapaxes_copy(lib, torch_cuda, elem):
    torch = torch_cuda
    shapes = [((3, 4), 0, 1), ((65, 130), 0, 1), ((64, 64), 1, 0), ((5, 6, 7), 0, 2), ((5, 6, 7), 1, 2), ((5, 6, 7), 0, 1),
              ((2, 3, 4, 5), 1, 3), ((2, 3, 4, 5), 0, 2), ((1, 12, 1), 1, 2), ((7, 1), 0, 1), ((300, 3), 0, 1),
              ((4, 5), 1, 1), ((2, 2, 1, 1, 2, 1, 2), 0, 6),
              # even extents: 2-byte elements move as 32-bit words in 128 x 128 tiles
              ((128, 128), 0, 1), ((130, 258), 0, 1), ((2, 4), 0, 1), ((200, 2), 0, 1), ((6, 4, 10), 0, 2),
              ((3, 8, 6), 1, 2), ((2, 256, 3, 130), 1, 3), ((514, 126), 1, 0),
              # several tiles inside the array (the path without bounds checks) beside edge tiles, batched
              ((3, 300, 2, 260), 1, 3), ((384, 512), 0, 1), ((2, 129, 383), 1, 2)]
    rng = np.random.default_rng(0)
    for shape, a, b in shapes:
        x = rng.integers(0, 255, int(np.prod(shape)) * np.dtype(elem).itemsize, dtype=np.uint8).view(elem).reshape(shape)
        d_in = torch.from_numpy(x.reshape(-1).view(np.uint8).copy()).cuda()
        d_out = torch.zeros_like(d_in)
        c_shape = (ctypes.c_int64 * len(shape))(*shape)
        rc = lib.cpn_swapaxes_copy(np.dtype(elem).itemsize, d_in.data_ptr(), d_out.data_ptr(), c_shape, len(shape), a, b,
                                   ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0
        want = np.ascontiguousarray(np.swapaxes(x, a, b))
        got = d_out.cpu().numpy().view(elem).reshape(want.shape)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (shape, a, b)


@pytest.mark.parametrize("dtype", [np.int32, np.float16, np.float64, np.uint8, np.complex64, np.complex128])
def test_sort_along_other_axes(dtype):
    for shape in [(100, 70), (5, 6, 7), (65, 130), (2, 3, 4, 5), (1000, 3), (3, 9000)]:
        x = make_input(dtype, shape, seed=len(shape))
        a = num.array(x)
        for axis in range(len(shape)):
            assert_same_bits(np.asarray(num.sort(a, axis=axis)), oracle.sort(x, axis=axis), f"{shape} axis={axis}")
            assert_same_bits(np.asarray(num.argsort(a, axis=axis)), oracle.argsort(x, axis=axis), f"{shape} axis={axis}")


def test_complex_integration_cases():
    # tests/integration/test_sort.py:146-183: complex64 / complex128 inputs against NumPy
    rng = np.random.default_rng(8)
    for dtype in COMPLEX_DTYPES:
        for size in [(5,), (5, 5), (3, 4, 5), (1, 0, 1)]:
            arr_np = (rng.integers(-10, 10, size) + 1j * rng.integers(-10, 10, size)).astype(dtype)
            arr_num = num.array(arr_np)
            for axis in range(-arr_np.ndim + 1, arr_np.ndim):
                assert np.array_equal(num.sort(arr_num, axis=axis), np.sort(arr_np, axis=axis, kind="stable"))
                assert np.array_equal(
                    num.argsort(arr_num, axis=axis, kind="stable"), np.argsort(arr_np, axis=axis, kind="stable")
                )


# ---- seeded random sweep over shapes, axes, dtypes and entry points -----------------------------------
@pytest.mark.parametrize("seed", range(8))
def test_random_shapes_axes_dtypes(seed):
    """40 random cases per seed through the public API: 1-3 dimensions, any axis (or None), every dtype,
    sort / argsort / in-place sort, rows from empty to tens of thousands of elements, so that every row
    kernel and the global path meet odd lengths and odd batch counts."""
    rng = np.random.default_rng(1000 + seed)
    for case in range(40):
        dtype = ALL_DTYPES[int(rng.integers(len(ALL_DTYPES)))]
        ndim = int(rng.integers(1, 4))
        budget = int(rng.choice([64, 3000, 60_000, 200_000]))
        shape = []
        for d in range(ndim):
            hi = max(1, int(budget ** (1.0 / (ndim - d))))
            n = int(rng.integers(0 if rng.random() < 0.03 else 1, hi + 1))
            shape.append(n)
            budget = max(1, budget // max(n, 1))
        rng.shuffle(shape)
        shape = tuple(int(s) for s in shape)
        axis = None if rng.random() < 0.15 else int(rng.integers(-ndim, ndim))
        x = make_input(dtype, shape, seed=seed * 100 + case)
        a = num.array(x)
        what = f"seed={seed} case={case} {np.dtype(dtype)} {shape} axis={axis}"
        op = int(rng.integers(3))
        if op == 0:
            assert_same_bits(np.asarray(num.sort(a, axis=axis)), oracle.sort(x, axis=axis), what + " sort")
        elif op == 1:
            got = num.argsort(a, axis=axis, kind="stable")
            want = oracle.argsort(x, axis=axis, kind="stable")
            assert got.shape == want.shape and np.array_equal(np.asarray(got), want), what + " argsort"
        else:
            a.sort(axis=axis)
            assert_same_bits(np.asarray(a), oracle.sort(x, axis=axis), what + " in place")


# ---- stream capture --------------------------------------------------------------------------------------
def test_sort_call_is_capturable_into_a_graph(lib, torch_cuda):
    """cpn_local_sort enqueues only kernel launches (its workspace is cleared by a fill kernel, the pass
    plan is made on the device), so a call can be captured into a HIP graph.  The graph is replayed
    several times on changing input, with eager work and synchronisations in between, and every replay
    is compared with the eager result of the same input."""
    torch = torch_cuda
    dev = torch.device("cuda")
    n = 300_000
    code = _lib.DTYPE_CODES[np.dtype(np.float32)]
    rng = np.random.default_rng(3)
    d_in = torch.zeros(n, dtype=torch.float32, device=dev)
    d_idx = torch.zeros(n, dtype=torch.int64, device=dev)
    tb = lib.cpn_local_sort_temp_bytes(code, n, n, 0, 1, 0)
    temp = torch.zeros(tb, dtype=torch.uint8, device=dev)

    def enqueue():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.cpn_local_sort(code, d_in.data_ptr(), None, d_idx.data_ptr(), n, n, 0, 1, temp.data_ptr(), tb, stream)
        assert rc == 0, _lib.status_string(rc)

    d_in.copy_(torch.from_numpy(rng.standard_normal(n).astype(np.float32)))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue()  # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for rep in range(4):
        x = rng.standard_normal(n).astype(np.float32)
        if rep % 2:
            x = np.round(x * 3)  # many ties, some passes skipped: the device-side plan changes between replays
        x[::1000] = np.nan
        d_in.copy_(torch.from_numpy(x))
        d_idx.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        got = d_idx.cpu().numpy()
        assert np.array_equal(got, oracle.local_sort(x, argsort=True)), f"replay {rep}"
        # eager work between the replays
        v, i = abi_sort(lib, torch, x[:5000], want_values=True, want_indices=True)
        assert np.array_equal(i, oracle.local_sort(x[:5000], argsort=True))


def test_captured_sort_switches_plans_between_replays(lib, torch_cuda, virtual_digits_from_2_to_20):
    """A captured sort of 8-byte keys whose input changes between replays from few different keys (one pass
    on their ranks) to few values per byte (grouped digits) to random keys (byte passes) and back: every
    decision is taken on the device from the data of that replay, and the tables in the workspace are
    cleared by the call itself."""
    torch = torch_cuda
    dev = torch.device("cuda")
    rng = np.random.default_rng(21)
    n = (1 << 20) + 777
    code = _lib.DTYPE_CODES[np.dtype(np.int64)]
    d_in = torch.zeros(n, dtype=torch.int64, device=dev)
    d_val = torch.zeros(n, dtype=torch.int64, device=dev)
    d_idx = torch.zeros(n, dtype=torch.int64, device=dev)
    tb = lib.cpn_local_sort_temp_bytes(code, n, n, 1, 1, 0)
    temp = torch.full((tb,), 0xFF, dtype=torch.uint8, device=dev)

    def enqueue():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.cpn_local_sort(code, d_in.data_ptr(), d_val.data_ptr(), d_idx.data_ptr(), n, n, 0, 1,
                                temp.data_ptr(), tb, stream)
        assert rc == 0, _lib.status_string(rc)

    def few_keys():
        return _few_values(rng, np.int64, n, 16)

    def few_per_byte():
        x = np.zeros(n, dtype=np.uint64)
        for b in range(8):
            x |= rng.integers(0, 256, 4).astype(np.uint64)[rng.integers(0, 4, n)] << np.uint64(8 * b)
        return x.view(np.int64)

    def random_keys():
        return rng.integers(-(2**63), 2**63 - 1, n, dtype=np.int64)

    def all_equal():
        return np.full(n, 12345, dtype=np.int64)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue()  # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for rep, make in enumerate([few_keys, few_per_byte, random_keys, few_keys, all_equal, random_keys, few_per_byte]):
        x = make()
        d_in.copy_(torch.from_numpy(x))
        d_idx.fill_(-1)
        d_val.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
        assert np.array_equal(d_idx.cpu().numpy(), oracle.local_sort(x, argsort=True, threads=8)), f"replay {rep} {make.__name__}"
        assert np.array_equal(d_val.cpu().numpy(), oracle.local_sort(x, argsort=False, threads=8)), f"replay {rep} {make.__name__}"
        abi_sort(lib, torch, x[:3000], want_values=True, want_indices=True)  # eager work between the replays


# ---- concurrent callers ------------------------------------------------------------------------------------
def test_concurrent_streams_and_threads(lib, torch_cuda):
    """Two host threads, each with its own stream, buffers and workspace, sort at the same time: the
    library keeps no shared mutable state between calls (the tunables aside)."""
    import threading

    torch = torch_cuda
    dev = torch.device("cuda")
    errors: list[str] = []

    def worker(tid: int) -> None:
        try:
            rng = np.random.default_rng(50 + tid)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for it in range(6):
                    n = int(rng.integers(20_000, 400_000))
                    dtype = [np.float32, np.int64, np.uint16][(tid + it) % 3]
                    x = make_input(dtype, (n,), seed=tid * 100 + it)
                    code = _lib.DTYPE_CODES[np.dtype(dtype)]
                    d_in = torch.from_numpy(x.view(np.uint8).copy()).to(dev, non_blocking=False)
                    d_idx = torch.empty(n, dtype=torch.int64, device=dev)
                    tb = lib.cpn_local_sort_temp_bytes(code, n, n, 0, 1, 0)
                    temp = torch.empty(tb, dtype=torch.uint8, device=dev)
                    h = ctypes.c_void_p(stream.cuda_stream)
                    rc = lib.cpn_local_sort(code, d_in.data_ptr(), None, d_idx.data_ptr(), n, n, 0, 1, temp.data_ptr(), tb, h)
                    if rc != 0 or lib.cpn_local_sort_check(temp.data_ptr(), h) != 0:
                        errors.append(f"thread {tid} iteration {it}: status {rc}")
                        return
                    stream.synchronize()
                    if not np.array_equal(d_idx.cpu().numpy(), oracle.local_sort(x, argsort=True)):
                        errors.append(f"thread {tid} iteration {it}: wrong result ({np.dtype(dtype)}, n={n})")
                        return
        except Exception as exc:  # surfaced below; an exception in a thread would otherwise be lost
            errors.append(f"thread {tid}: {exc!r}")

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_global_sorts_overlapping_on_three_streams(lib, torch_cuda):
    """Global sorts of several hundred tiles each, enqueued on three streams without a host wait in
    between, so that their scatter passes compete for the workgroup slots of every XCD while each
    deals its tiles per XCD: every call must finish without the look-back giving up and match the
    oracle."""
    torch = torch_cuda
    dev = torch.device("cuda")
    jobs = []
    streams = [torch.cuda.Stream() for _ in range(3)]
    torch.cuda.synchronize()
    for rnd in range(3):
        for k, stream in enumerate(streams):
            dtype = [np.float32, np.int32, np.int64][(k + rnd) % 3]
            n = (1 << 22) + 12345 * (k + 1) + rnd
            x = make_input(dtype, (n,), seed=900 + 10 * rnd + k)
            code = _lib.DTYPE_CODES[np.dtype(dtype)]
            d_in = torch.from_numpy(x.view(np.uint8).copy()).to(dev)
            d_idx = torch.empty(n, dtype=torch.int64, device=dev)
            tb = lib.cpn_local_sort_temp_bytes(code, n, n, 0, 1, 0)
            temp = torch.full((tb,), 0xFF, dtype=torch.uint8, device=dev)
            jobs.append((x, d_in, d_idx, temp, tb, code, n, stream))
    torch.cuda.synchronize()
    for x, d_in, d_idx, temp, tb, code, n, stream in jobs:  # all enqueued before anything is waited for
        h = ctypes.c_void_p(stream.cuda_stream)
        assert lib.cpn_local_sort(code, d_in.data_ptr(), None, d_idx.data_ptr(), n, n, 0, 1, temp.data_ptr(), tb, h) == 0
    for x, d_in, d_idx, temp, tb, code, n, stream in jobs:
        h = ctypes.c_void_p(stream.cuda_stream)
        assert lib.cpn_local_sort_check(temp.data_ptr(), h) == 0, f"{x.dtype} n={n}: device status"
        assert np.array_equal(d_idx.cpu().numpy(), oracle.local_sort(x, argsort=True, threads=8)), f"{x.dtype} n={n}"


# ---- failure path of the bounded look-back wait -------------------------------------------------------
def test_lookback_gives_up_cleanly(lib, torch_cuda):
    """With the spin limit forced to one poll, a tile whose predecessor has not answered yet gives up:
    every kernel still runs to its end, nothing is written out of bounds, and the device status word
    reports the failure (CPN_ERR_DEVICE) instead of a hang or a silently wrong result.  Whether a given
    run hits an unanswered poll depends on timing, so a clean run must be fully correct and at least
    one of several runs over a thousand tiles is expected to report the failure (the test is reported as
    skipped if none does)."""
    torch = torch_cuda
    dev = torch.device("cuda")
    n = 1 << 24
    rng = np.random.default_rng(6)
    x = rng.integers(0, 1 << 31, n).astype(np.int32)
    code = _lib.DTYPE_CODES[np.dtype(np.int32)]
    d_in = torch.from_numpy(x).to(dev)
    guard = 4096
    d_out = torch.full((n + 2 * guard,), -1, dtype=torch.int32, device=dev)  # canaries on both sides
    out = d_out[guard : guard + n]
    tb = lib.cpn_local_sort_temp_bytes(code, n, n, 1, 0, 0)
    temp = torch.empty(tb, dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want = None
    seen_failure = False
    prev = lib.cpn_set_lookback_spin_limit(1)
    try:
        for _ in range(5):
            rc = lib.cpn_local_sort(code, d_in.data_ptr(), out.data_ptr(), None, n, n, 0, 1, temp.data_ptr(), tb, stream)
            assert rc == 0
            status = lib.cpn_local_sort_check(temp.data_ptr(), stream)
            assert status in (0, _lib.CPN_ERR_DEVICE)
            assert bool((d_out[:guard] == -1).all()) and bool((d_out[guard + n :] == -1).all()), "wrote outside the output"
            if status == 0:
                if want is None:
                    want = np.sort(x, kind="stable")
                assert np.array_equal(out.cpu().numpy(), want)
            else:
                seen_failure = True
    finally:
        assert lib.cpn_set_lookback_spin_limit(prev) == 1
    # back at the default limit the same call succeeds
    assert lib.cpn_local_sort(code, d_in.data_ptr(), out.data_ptr(), None, n, n, 0, 1, temp.data_ptr(), tb, stream) == 0
    assert lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
    assert np.array_equal(out.cpu().numpy(), np.sort(x, kind="stable") if want is None else want)
    if not seen_failure:  # timing: every poll of every tile happened to be answered at once
        pytest.skip("no look-back had to wait in five runs, the failure path was not reached")


def test_single_ticket_tile_order(lib, torch_cuda, global_path):
    """cpn_set_tile_order(1): tiles handed out through one counter instead of per XCD; same results."""
    prev = lib.cpn_set_tile_order(1)
    try:
        assert prev == 0
        for dtype, shape in [(np.float32, (300_001,)), (np.int64, (70_000,)), (np.uint16, (5, 40_000)), (np.int32, (3, 16385))]:
            check_rows(lib, torch_cuda, make_input(dtype, shape, seed=5), f"single ticket {np.dtype(dtype)} {shape}")
    finally:
        assert lib.cpn_set_tile_order(prev) == 1


def test_single_ticket_per_call(lib, torch_cuda, global_path):
    """cpn_local_sort_ex with CPN_SORT_SINGLE_TICKET: the same bits as the default order, the process-wide
    setting untouched; unknown option bits are refused."""
    for dtype, shape, argsort in [(np.float32, (300_001,), True), (np.int64, (70_000,), False), (np.uint16, (5, 40_000), True)]:
        x = make_input(dtype, shape, seed=6)
        code, seg = _lib.DTYPE_CODES[x.dtype], x.shape[-1]
        d_in = torch_cuda.from_numpy(x.reshape(-1).view(np.uint8).copy()).cuda()
        d_val = torch_cuda.zeros_like(d_in)
        d_idx = torch_cuda.zeros(x.size, dtype=torch_cuda.int64, device="cuda")
        tb = lib.cpn_local_sort_temp_bytes(code, x.size, seg, 1, int(argsort), 0)
        temp = torch_cuda.full((tb,), 0xFF, dtype=torch_cuda.uint8, device="cuda")
        stream = ctypes.c_void_p(torch_cuda.cuda.current_stream().cuda_stream)
        rc = lib.cpn_local_sort_ex(code, d_in.data_ptr(), d_val.data_ptr(), d_idx.data_ptr() if argsort else None, x.size, seg,
                                   0, 1, _lib.CPN_SORT_SINGLE_TICKET, temp.data_ptr(), tb, stream)
        assert rc == 0 and lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
        assert_same_bits(d_val.cpu().numpy().view(x.dtype).reshape(x.shape), oracle.local_sort(x, argsort=False), f"{shape}")
        if argsort:
            assert np.array_equal(d_idx.cpu().numpy().reshape(x.shape), oracle.local_sort(x, argsort=True))
        assert lib.cpn_local_sort_ex(code, d_in.data_ptr(), d_val.data_ptr(), None, x.size, seg, 0, 1, 2, temp.data_ptr(), tb,
                                     stream) == _lib.CPN_ERR_UNSUPPORTED
    assert lib.cpn_set_tile_order(0) == 0


def test_python_layer_status_modes(lib, torch_cuda, monkeypatch):
    """The Python layer's handling of the device status word: lazy (default: read when data next
    reaches the host), eager with one repeat in single-ticket order, off.  The failure is forced from
    the host: a spin limit of one poll (lazy), a status read that reports it (eager)."""
    from cupynumeric_amd import _sort
    from cupynumeric_amd.runtime import runtime

    rng = np.random.default_rng(8)
    x = rng.integers(0, 1 << 31, 1 << 22).astype(np.int32)
    want = np.argsort(x, kind="stable")
    a = num.array(x)
    # lazy: consecutive sorts, one read-back at the first host access
    monkeypatch.setattr(runtime, "check_mode", "lazy")
    first, second = num.argsort(a), num.sort(a)
    assert runtime._status_used == 2
    assert np.array_equal(np.asarray(first), want) and runtime._status_used == 0
    assert np.array_equal(np.asarray(second), x[want])
    # row sorts leave no status word behind
    rows = num.array(x.reshape(1 << 10, 1 << 12))
    num.sort(rows)
    assert runtime._status_used == 0
    # lazy, with every look-back forced to give up at its first unanswered poll: the error comes
    # with the host read, when a sort failed (timing decides whether one did), and the layer recovers
    prev = lib.cpn_set_lookback_spin_limit(1)
    try:
        results = [num.argsort(a) for _ in range(4)]
        torch_cuda.cuda.synchronize()
    finally:
        lib.cpn_set_lookback_spin_limit(prev)
    failed = bool(runtime._status_slots[: runtime._status_used].cpu().any())
    if failed:
        with pytest.raises(RuntimeError, match="failed on the device"):
            np.asarray(results[0])
    assert np.array_equal(np.asarray(num.argsort(a)), want)
    # eager: a reported failure is answered by one repeat with the single tile counter
    monkeypatch.setattr(runtime, "check_mode", "eager")
    real_check, real_sort = lib.cpn_local_sort_check, lib.cpn_local_sort_ex
    calls = {"n": 0, "options": [], "order_at_repeat": None}

    def failing_once(temp, stream):
        calls["n"] += 1
        if calls["n"] == 1:
            real_check(temp, stream)
            return _lib.CPN_ERR_DEVICE
        calls["order_at_repeat"] = lib.cpn_set_tile_order(0)  # returns the order in force
        return real_check(temp, stream)

    def recording_sort(*args):
        calls["options"].append(args[8])
        return real_sort(*args)

    monkeypatch.setattr(lib, "cpn_local_sort_check", failing_once)
    monkeypatch.setattr(lib, "cpn_local_sort_ex", recording_sort)
    got = num.argsort(a)
    monkeypatch.setattr(lib, "cpn_local_sort_check", real_check)
    monkeypatch.setattr(lib, "cpn_local_sort_ex", real_sort)
    # the repeat asks for the single counter per call; the process-wide order is never touched
    assert calls == {"n": 2, "options": [0, _lib.CPN_SORT_SINGLE_TICKET], "order_at_repeat": 0}
    assert np.array_equal(np.asarray(got), want)
    # an in-place sort cannot be repeated (its input is gone): the failure is raised
    calls["n"] = 0
    monkeypatch.setattr(lib, "cpn_local_sort_check", failing_once)
    b = num.array(x)
    with pytest.raises(RuntimeError):
        b.sort()
    monkeypatch.setattr(lib, "cpn_local_sort_check", real_check)


# ---- virtual digits: fewer passes for keys whose bytes take few distinct values ---------------------
def _few_values(rng, dtype, n, distinct):
    """n keys drawn from `distinct` arbitrary values of `dtype` (every byte position busy, few values each)."""
    dt = np.dtype(dtype)
    if dt.kind == "f":
        pool = rng.standard_normal(distinct).astype(dtype) * dtype(1000.0)
        pool[: min(3, distinct)] = [np.nan, -0.0, 0.0][: min(3, distinct)]
    else:
        info = np.iinfo(dtype)
        pool = rng.integers(info.min, info.max, distinct, dtype=dtype, endpoint=True)
    return pool[rng.integers(0, distinct, n)]


@pytest.fixture()
def virtual_digits_from_2_to_20(lib):
    """Virtual digits are considered from 2^26 elements on by default; the tests lower that."""
    prev = lib.cpn_set_virtual_digit_threshold(1 << 20)
    yield
    lib.cpn_set_virtual_digit_threshold(prev)


@pytest.mark.parametrize("dtype", [np.int64, np.uint64, np.float64, np.int32, np.float32])
def test_virtual_digits(lib, torch_cuda, virtual_digits_from_2_to_20, dtype):
    """One long row of 8-byte keys (4-byte keys run alongside: they never use virtual digits and must
    not be disturbed): with 16 distinct values every byte
    carries 4 bits and pairs of bytes are sorted in one pass; with 3 distinct values four bytes share a
    pass; with 300 values some bytes are too busy to share; random keys keep the ordinary passes.  Every
    output form is compared with the oracle bit for bit."""
    rng = np.random.default_rng(np.dtype(dtype).num)
    n = (1 << 21) + 1234
    for distinct in (16, 3, 300, 2):
        x = _few_values(rng, dtype, n, distinct)
        want_v = oracle.local_sort(x, argsort=False, threads=8)
        want_i = oracle.local_sort(x, argsort=True, threads=8)
        v, _ = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=False)
        assert_same_bits(v, want_v, f"{np.dtype(dtype)} {distinct} values, sort")
        _, i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
        assert_same_bits(i, want_i, f"{np.dtype(dtype)} {distinct} values, argsort")
        if distinct == 16:
            v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, in_place=True, offset=5)
            assert_same_bits(v, want_v, "in place + indices")
            assert_same_bits(i, want_i + 5, "in place + indices")
            v, _ = abi_sort(lib, torch_cuda, x, want_values=True, in_place=True)
            assert_same_bits(v, want_v, "in place")
    # bytes with few values next to bytes with all 256: only some positions share a pass
    if np.dtype(dtype).kind != "f":
        hi = rng.integers(0, 7, n).astype(np.uint64) << np.uint64(8 * (np.dtype(dtype).itemsize - 1) - 1)
        lo = rng.integers(0, 1 << 16, n).astype(np.uint64)
        x = (hi | lo).astype(np.dtype(dtype).str.replace("i", "u")).view(dtype)
        _, i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
        assert_same_bits(i, oracle.local_sort(x, argsort=True, threads=8), "mixed busy and quiet bytes")
    # more than 256 different keys whose bytes take 4 values each: bytes share passes (grouped digits)
    if np.dtype(dtype).kind != "f":
        width = np.dtype(dtype).itemsize
        x = np.zeros(n, dtype=np.uint64)
        for b in range(width):
            vals = rng.integers(0, 256, 4).astype(np.uint64)
            x |= vals[rng.integers(0, 4, n)] << np.uint64(8 * b)
        x = x.astype(np.dtype(dtype).str.replace("i", "u")).view(dtype)
        _, i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
        assert_same_bits(i, oracle.local_sort(x, argsort=True, threads=8), "4 values per byte")
        v, _ = abi_sort(lib, torch_cuda, x, want_values=True)
        assert_same_bits(v, oracle.local_sort(x, argsort=False, threads=8), "4 values per byte, sort")
    # short rows and several rows never use virtual digits; same answers
    x = _few_values(rng, dtype, 3 * 100_000, 16).reshape(3, 100_000)
    check_rows(lib, torch_cuda, x, f"{np.dtype(dtype)} short rows of few values")


@pytest.mark.parametrize("dtype", [np.int64, np.uint64, np.float64])
def test_rows_of_at_most_256_different_keys(lib, torch_cuda, virtual_digits_from_2_to_20, dtype):
    """A long row of 8-byte keys with at most 256 different values is sorted by one pass on the rank of
    each key among them; 257 and more fall back to the other plans.  The smallest key of the type (its
    ordered image is the marker of an empty table slot) and, for floats, NaNs of several payloads and both
    zeros take part."""
    rng = np.random.default_rng(7 + np.dtype(dtype).num)
    n = (1 << 20) + 4321
    dt = np.dtype(dtype)
    for distinct in (1, 2, 255, 256, 257, 1000):
        if dt.kind == "f":
            pool = rng.standard_normal(distinct) * 1e3
            bits = pool.view(np.uint64)
            if distinct >= 6:
                bits[:6] = [0x7FF8000000000000, 0x7FF8000000000123, 0xFFF8000000000000, 0x8000000000000000, 0,
                            0xFFF0000000000000]  # three NaNs (one key), -0.0 and 0.0 (one key), -inf
            pool = bits.view(np.float64)
        else:
            info = np.iinfo(dtype)
            pool = rng.integers(info.min, info.max, distinct, dtype=dtype, endpoint=True)
            if distinct >= 2:
                pool[0] = info.min
                pool[1] = info.max
        x = pool[rng.integers(0, distinct, n)]
        want_i = oracle.local_sort(x, argsort=True, threads=8)
        want_v = oracle.local_sort(x, argsort=False, threads=8)
        _, i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
        assert_same_bits(i, want_i, f"{dt} {distinct} different keys, argsort")
        v, i = abi_sort(lib, torch_cuda, x, want_values=True, want_indices=True, offset=3)
        assert_same_bits(v, want_v, f"{dt} {distinct} different keys, values")
        assert_same_bits(i, want_i + 3, f"{dt} {distinct} different keys, indices")
        v, _ = abi_sort(lib, torch_cuda, x, want_values=True, in_place=True)
        assert_same_bits(v, want_v, f"{dt} {distinct} different keys, in place")
    # few keys in most of the row, many in one corner: the workgroup that meets them reports it
    x = pool[:16][rng.integers(0, 16, n)]
    x[n // 3 : n // 3 + 5000] = pool[rng.integers(0, 1000, 5000)]
    _, i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
    assert_same_bits(i, oracle.local_sort(x, argsort=True, threads=8), f"{dt} crowded corner")
    # sorted input with long runs: every workgroup sees few keys, the row holds many
    x = np.sort(pool[rng.integers(0, 1000, n)])
    _, i = abi_sort(lib, torch_cuda, x, want_values=False, want_indices=True)
    assert_same_bits(i, oracle.local_sort(x, argsort=True, threads=8), f"{dt} sorted runs")


# ---- the streaming-rate probe of the benchmark ------------------------------------------------------
@pytest.mark.parametrize("nbytes", [0, 16, 4096 + 16, (1 << 22) + 48, 3 * (1 << 24)])
def test_stream_probe_copies_fills_and_leaves_the_source_alone(nbytes):
    """cpn_stream_probe: the copy moves every byte (sizes below, at and above one grid of 512-thread
    workgroups, and above the grid cap so that threads loop), the fill writes its constant, the read
    pass changes nothing, and bad arguments come back as status codes."""
    import torch

    lib = _lib.load()
    dev = torch.device("cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator(device="cpu").manual_seed(nbytes)
    host = torch.randint(0, 256, (max(nbytes, 16),), dtype=torch.uint8, generator=g)
    src = host.to(dev)
    dst = torch.full((max(nbytes, 16) + 32,), 0xEE, dtype=torch.uint8, device=dev)  # 32 guard bytes
    assert lib.cpn_stream_probe(1, src.data_ptr(), dst.data_ptr(), nbytes, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst[:nbytes].cpu(), host[:nbytes])
    assert bool((dst[nbytes:] == 0xEE).all()), "the copy wrote past its size"
    assert lib.cpn_stream_probe(0, src.data_ptr(), dst.data_ptr(), nbytes, stream) == 0
    assert lib.cpn_stream_probe(0, src.data_ptr(), None, nbytes, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(src.cpu(), host) and torch.equal(dst[:nbytes].cpu(), host[:nbytes])
    assert lib.cpn_stream_probe(2, None, dst.data_ptr(), nbytes, stream) == 0
    torch.cuda.synchronize()
    assert bool((dst[:nbytes] == 1).all()) and bool((dst[nbytes:] == 0xEE).all())
    # error paths: nothing is launched
    assert lib.cpn_stream_probe(3, src.data_ptr(), dst.data_ptr(), 16, stream) == -3
    assert lib.cpn_stream_probe(1, src.data_ptr(), dst.data_ptr(), 8, stream) == -3
    assert lib.cpn_stream_probe(1, None, dst.data_ptr(), 16, stream) == -2
    assert lib.cpn_stream_probe(2, None, None, 16, stream) == -2
    assert lib.cpn_stream_probe(1, src.data_ptr() + 4, dst.data_ptr(), 16, stream) == -5
