"""Consumers of sorted output: searchsorted, unique and the element casts they need
(src/cupynumeric/sort/searchsorted.cu, src/cupynumeric/set/unique.cu; reference tests
tests/integration/test_searchsorted.py, test_unique.py), through the public API and the C ABI."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
from conftest import ALL_REAL_DTYPES, COMPLEX_DTYPES, assert_same_bits

import cupynumeric_amd as num
from cupynumeric_amd import _lib
from oracle import sort_oracle as oracle

pytestmark = pytest.mark.gpu

SIDES = ["left", "right"]
# tests/integration/test_searchsorted.py:27-53
STANDARD_CASES = [
    (156, np.uint8), (123, np.uint16), (241, np.uint32), (1, np.uint64), (21, np.int8), (5, np.int16),
    (34, np.int32), (11, np.int64), (31, np.float32), (11, np.float64), (422, np.double), (220, np.double),
    (244, np.complex64), (24, np.complex128), (220, np.complex128), (0, np.uint32),
]
DTYPE_CASES = [
    (3, np.uint64, np.float32), (51, np.uint32, np.complex64), (23, np.uint32, np.float64),
    (51, np.complex64, np.float64), (21, np.complex64, np.int32), (22, np.complex128, np.float32),
]


def generate_random(rng, volume, datatype):
    """tests/integration/test_searchsorted.py:131-154, with a seeded generator."""
    if np.issubdtype(datatype, np.integer):
        info = np.iinfo(datatype)
        return rng.integers(info.min, info.max, size=volume, dtype=datatype)
    if np.issubdtype(datatype, np.floating):
        return rng.random(volume).astype(datatype)
    return (rng.random(volume) + rng.random(volume) * 1j).astype(datatype)


def check_api(a, v, side):
    """tests/integration/test_searchsorted.py:157-178: method and module form, with a sorter."""
    a_argsorted = np.argsort(a, kind="stable")
    a_num, v_num, s_num = num.array(a), num.array(v), num.array(a_argsorted)
    want = np.searchsorted(a, v, side=side, sorter=a_argsorted)
    got = a_num.searchsorted(v_num, side=side, sorter=s_num)
    assert got.dtype == np.int64 and got.shape == want.shape
    assert np.array_equal(np.asarray(got), want)
    got = num.searchsorted(a_num, v_num, side=side, sorter=s_num)
    assert np.array_equal(np.asarray(got), want)
    if a.size <= 64:
        assert np.array_equal(oracle.searchsorted(a, v, side, sorter=a_argsorted), want)


@pytest.mark.parametrize("side", SIDES)
def test_searchsorted_reference_cases(side):
    rng = np.random.default_rng(11)
    check_api(np.arange(25), np.arange(0), side)
    check_api(np.array([]), generate_random(rng, 10, np.float64), side)
    check_api(np.arange(0), np.arange(0), side)
    for volume, dtype in STANDARD_CASES:
        check_api(generate_random(rng, volume, dtype), generate_random(rng, 10, dtype), side)
    for volume, d1, d2 in DTYPE_CASES:
        check_api(generate_random(rng, volume, d1), generate_random(rng, 10, d2), side)
    for ndim in range(1, 5):
        a = rng.integers(-100, 100, size=100)
        v = rng.integers(-100, 100, size=2**ndim).reshape((2,) * ndim)
        check_api(a, v, side)
    # scalar value
    got = num.searchsorted(num.array(np.arange(10)), 4, side=side)
    assert got.shape == () and int(np.asarray(got)) == np.searchsorted(np.arange(10), 4, side=side)


def test_searchsorted_errors():
    rng = np.random.default_rng(1)
    with pytest.raises(ValueError):
        num.searchsorted(num.array(rng.random((5, 5, 5))), 5)
    with pytest.raises(TypeError):
        num.searchsorted(num.array([2, 3, 10, 9]), None)
    a = num.array(rng.integers(-100, 100, size=100))
    v = num.array(rng.integers(-100, 100, size=10))
    with pytest.raises(ValueError):
        num.searchsorted(a, v, sorter=num.array(rng.integers(0, 10, size=10)))
    with pytest.raises(ValueError):
        num.searchsorted(a, v, sorter=num.array(rng.random((5, 5, 5))))
    with pytest.raises(ValueError):
        num.searchsorted(a, v, sorter=num.array(rng.random(100)))


@pytest.mark.parametrize("dtype", ALL_REAL_DTYPES + COMPLEX_DTYPES)
@pytest.mark.parametrize("side", SIDES)
def test_searchsorted_special_values_and_pivot_table(dtype, side):
    """Duplicates, NaN / +-0 / inf, values outside the range; n large enough for the LDS pivot
    table (n >= 8192 with >= 2048 values) and n around its strides."""
    rng = np.random.default_rng(np.dtype(dtype).num + (side == "left"))
    kind = np.dtype(dtype).kind
    for n, m in [(5, 40), (300, 3000), (8192, 2048), (8193, 5000), (100_003, 20_000), (1 << 20, 1 << 16)]:
        if kind == "b":
            a = rng.integers(0, 2, n).astype(dtype)
            v = rng.integers(0, 2, m).astype(dtype)
        elif kind in "iu":
            info = np.iinfo(dtype)
            lo, hi = max(info.min, -(n // 3)), min(info.max, n // 3 + 1)
            a = rng.integers(lo, hi, n).astype(dtype)
            v = rng.integers(info.min, info.max, m, dtype=dtype, endpoint=True)
            v[: m // 2] = rng.integers(lo, hi, m // 2).astype(dtype)
        else:
            comp = {"e": np.float16, "f": np.float32, "d": np.float64, "F": np.float32, "D": np.float64}[np.dtype(dtype).char]
            def parts(k):
                x = np.round(rng.standard_normal(k) * (8 if comp == np.float16 else n / 8)).astype(comp)
                x[rng.random(k) < 0.02] = np.nan
                x[rng.random(k) < 0.02] = -0.0
                x[rng.random(k) < 0.01] = np.inf
                x[rng.random(k) < 0.01] = -np.inf
                return x
            if kind == "c":
                with np.errstate(invalid="ignore"):
                    a = (parts(n) + 1j * parts(n)).astype(dtype)
                    v = (parts(m) + 1j * parts(m)).astype(dtype)
            else:
                a, v = parts(n), parts(m)
        srt = np.sort(a, kind="stable")
        got = np.asarray(num.searchsorted(num.array(srt), num.array(v), side=side))
        assert np.array_equal(got, np.searchsorted(srt, v, side=side)), (n, m)


def test_searchsorted_follows_sort_output():
    """End to end on the device: sort, then search the sorted array for its own elements."""
    rng = np.random.default_rng(9)
    x = rng.standard_normal(500_000).astype(np.float32)
    x[::1000] = np.nan
    s = num.sort(num.array(x))
    v = num.array(x[:50_000])
    left = np.asarray(num.searchsorted(s, v, "left"))
    right = np.asarray(num.searchsorted(s, v, "right"))
    sx = np.sort(x)
    assert np.array_equal(left, np.searchsorted(sx, x[:50_000], "left"))
    assert np.array_equal(right, np.searchsorted(sx, x[:50_000], "right"))
    assert (right > left).all()  # every value is present


def test_searchsorted_presorted_values_path():
    """Array beyond the cache threshold (64 MiB) with many values: with a workspace the values are sorted
    first; without one they are searched as given.  Same answers, both sides, float and complex."""
    import torch

    lib = _lib.load()
    dev = torch.device("cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(12)
    for dtype, n, m in [(np.float32, (1 << 24) + 77, 200_001), (np.complex64, (1 << 23) + 5, 70_000), (np.uint8, 1 << 26, 1 << 16)]:
        if dtype == np.uint8:
            a = np.sort(rng.integers(0, 256, n).astype(dtype))
            v = rng.integers(0, 256, m).astype(dtype)
        elif dtype == np.float32:
            a = np.sort(rng.standard_normal(n).astype(dtype))
            a[-1000:] = np.nan
            v = rng.standard_normal(m).astype(dtype)
            v[::97] = np.nan
            v[1::97] = a[rng.integers(0, n - 1000, v[1::97].size)]  # values that are present
        else:
            a = np.sort((np.round(rng.standard_normal(n) * 1000) + 1j * np.round(rng.standard_normal(n) * 3)).astype(dtype))
            v = (np.round(rng.standard_normal(m) * 1000) + 1j * np.round(rng.standard_normal(m) * 3)).astype(dtype)
        code = _lib.DTYPE_CODES[np.dtype(dtype)]
        d_a = torch.from_numpy(a.view(np.uint8)).to(dev)
        d_v = torch.from_numpy(v.view(np.uint8)).to(dev)
        tb = lib.cpn_searchsorted_temp_bytes(code, n, m)
        assert tb > 0
        assert lib.cpn_searchsorted_temp_bytes(code, 1000, m) == 0 and lib.cpn_searchsorted_temp_bytes(code, n, 100) == 0
        temp = torch.empty(tb, dtype=torch.uint8, device=dev)
        for left in (1, 0):
            want = np.searchsorted(a, v, side="left" if left else "right")
            with_ws = torch.full((m,), -1, dtype=torch.int64, device=dev)
            rc = lib.cpn_searchsorted(code, d_a.data_ptr(), n, d_v.data_ptr(), m, left, with_ws.data_ptr(), temp.data_ptr(), tb, stream)
            assert rc == 0 and lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
            direct = torch.full((m,), -1, dtype=torch.int64, device=dev)
            assert lib.cpn_searchsorted(code, d_a.data_ptr(), n, d_v.data_ptr(), m, left, direct.data_ptr(), None, 0, stream) == 0
            assert np.array_equal(with_ws.cpu().numpy(), want), (dtype, left)
            assert np.array_equal(direct.cpu().numpy(), want), (dtype, left)
            assert np.array_equal(d_v.cpu().numpy(), v.view(np.uint8))  # values untouched


# ---- unique --------------------------------------------------------------------------------------------
def numpy_unique(x: np.ndarray) -> np.ndarray:
    """np.unique, except that float16 goes through float32 (exact and order preserving): the default
    float16 sort of NumPy 2.2.6 on AVX-512 machines leaves arrays holding -0.0 unsorted, and np.unique
    inherits that."""
    if x.dtype == np.float16:
        return np.unique(x.astype(np.float32)).astype(np.float16)
    return np.unique(x)


def test_unique_reference_cases():
    from conftest import UNIQUE_GOLDEN

    for values, shape, expected, dtype in UNIQUE_GOLDEN:  # tests/cpp/integration/test_unique.cc:34-68
        got = num.unique(num.array(np.array(values, dtype=dtype).reshape(shape)))
        assert got.dtype == np.dtype(dtype) and np.asarray(got).tolist() == expected
    # tests/integration/test_unique.py:23-39
    a = np.nonzero(np.array([1, 1, 0, 0]))[0]
    assert np.array_equal(np.asarray(num.unique(num.array(a))), np.unique(a))
    rng = np.random.default_rng(2)
    for ndim in range(1, 5):
        x = rng.integers(0, 3, size=(4,) * ndim)
        got = num.unique(num.array(x))
        want = np.unique(x)
        assert got.dtype == want.dtype and got.shape == want.shape
        assert np.array_equal(np.asarray(got), want)
    with pytest.raises(TypeError, match="cuPyNumeric does not support dtype"):
        num.unique(np.array(["apple", "banana", "apple"]))
    for kw in ({"return_index": True}, {"return_inverse": True}, {"return_counts": True}, {"axis": 0}):
        with pytest.raises(NotImplementedError):
            num.unique(num.array(np.arange(9).reshape(3, 3)), **kw)


@pytest.mark.parametrize("dtype", ALL_REAL_DTYPES + COMPLEX_DTYPES)
def test_unique_all_dtypes(dtype):
    """Sizes around the 4096-element compaction tile and the row-kernel / global-sort boundary; few and
    many distinct values; NaN, +-0, complex values with NaN parts."""
    rng = np.random.default_rng(np.dtype(dtype).num)
    kind = np.dtype(dtype).kind
    for n, distinct in [(1, 1), (2, 1), (7, 3), (4095, 50), (4096, 4096), (4097, 2), (12_289, 9000), (300_000, 70_000),
                        (300_000, 5)]:
        if kind == "b":
            x = rng.integers(0, 2, n).astype(dtype)
        elif kind in "iu":
            info = np.iinfo(dtype)
            x = rng.integers(max(info.min, -distinct // 2), min(info.max, distinct // 2 + 1), n).astype(dtype)
        else:
            comp = {"e": np.float16, "f": np.float32, "d": np.float64, "F": np.float32, "D": np.float64}[np.dtype(dtype).char]
            def parts(k, spread):
                p = np.round(rng.standard_normal(k) * spread).astype(comp)
                p[rng.random(k) < 0.03] = np.nan
                p[rng.random(k) < 0.03] = -0.0
                p[rng.random(k) < 0.03] = 0.0
                return p
            spread = max(1.0, min(distinct, 2000) / 4)
            with np.errstate(invalid="ignore"):
                x = (parts(n, spread) + 1j * parts(n, 2)).astype(dtype) if kind == "c" else parts(n, spread)
        got = num.unique(num.array(x))
        want = numpy_unique(x)
        assert got.dtype == want.dtype and got.shape == want.shape, (n, distinct, got.shape, want.shape)
        assert np.array_equal(np.asarray(got), want, equal_nan=True), (n, distinct)
        if n <= 20_000:
            assert_same_bits(np.asarray(got), oracle.unique(x), f"unique n={n}")  # which of -0.0 / +0.0, which NaN


def test_unique_c_abi_direct():
    """cpn_unique through ctypes on torch-owned buffers: count word, untouched input, temp size."""
    import torch

    lib = _lib.load()
    dev = torch.device("cuda")
    rng = np.random.default_rng(4)
    x = rng.integers(0, 1000, 100_000).astype(np.int32)
    d_in = torch.from_numpy(x.copy()).to(dev)
    d_out = torch.empty_like(d_in)
    count = torch.full((1,), -1, dtype=torch.int64, device=dev)
    code = _lib.DTYPE_CODES[np.dtype(np.int32)]
    tb = lib.cpn_unique_temp_bytes(code, x.size)
    assert tb >= lib.cpn_local_sort_temp_bytes(code, x.size, x.size, 1, 0, 0) + x.nbytes
    temp = torch.empty(tb, dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.cpn_unique(code, d_in.data_ptr(), d_out.data_ptr(), x.size, count.data_ptr(), temp.data_ptr(), tb, stream)
    assert rc == 0, _lib.status_string(rc)
    assert lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
    want = np.unique(x)
    assert int(count.item()) == want.size
    assert np.array_equal(d_out[: want.size].cpu().numpy(), want)
    assert np.array_equal(d_in.cpu().numpy(), x)
    assert lib.cpn_unique(code, d_in.data_ptr(), d_out.data_ptr(), x.size, count.data_ptr(), temp.data_ptr(), tb - 256, stream) == -4
    assert lib.cpn_unique(code, None, None, 0, count.data_ptr(), None, 0, stream) == 0
    assert int(count.item()) == 0


# ---- casts ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("src", ALL_REAL_DTYPES + COMPLEX_DTYPES)
def test_astype_matches_numpy(src):
    """Value-preserving casts (the ones `np.result_type` asks of searchsorted) and casts to bool."""
    rng = np.random.default_rng(np.dtype(src).num)
    kind = np.dtype(src).kind
    if kind == "b":
        x = rng.integers(0, 2, 1000).astype(src)
    elif kind in "iu":
        info = np.iinfo(src)
        x = rng.integers(info.min, info.max, 1000, dtype=src, endpoint=True)
        x[:4] = [info.min, info.max, 0, 1]
    elif kind == "f":
        x = (rng.standard_normal(1000) * 100).astype(src)
        x[:5] = [np.nan, np.inf, -np.inf, -0.0, 0.0]
    else:
        x = (rng.standard_normal(1000) * 100 + 1j * rng.standard_normal(1000)).astype(src)
        x[:3] = [complex(np.nan, 1), complex(0, np.inf), 0]
    a = num.array(x)
    for dst in ALL_REAL_DTYPES + COMPLEX_DTYPES:
        if not (np.can_cast(src, dst, casting="safe") or np.dtype(dst) == np.bool_):
            continue
        got = a.astype(dst)
        with np.errstate(all="ignore"):
            want = x.astype(dst)
        assert got.dtype == want.dtype and got.shape == want.shape
        assert_same_bits(np.asarray(got), want, f"{np.dtype(src)}->{np.dtype(dst)}")


# ---- seeded random sweep ------------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(6))
def test_random_consumers(seed):
    """Random dtypes, sizes and duplicate rates for unique and searchsorted (NumPy is the expectation) and
    random key sets for lexsort (the oracle, itself pinned on np.lexsort, is the expectation)."""
    rng = np.random.default_rng(2000 + seed)
    dtypes = ALL_REAL_DTYPES + COMPLEX_DTYPES
    for case in range(25):
        dtype = dtypes[int(rng.integers(len(dtypes)))]
        kind = np.dtype(dtype).kind
        n = int(rng.choice([1, 7, 300, 5000, 70_000]))
        spread = float(rng.choice([1, 5, 200, 1e6]))

        def draw(k):
            if kind == "b":
                return rng.integers(0, 2, k).astype(dtype)
            if kind in "iu":
                info = np.iinfo(dtype)
                return rng.integers(max(info.min, -int(spread)), min(info.max, int(spread)) + 1, k).astype(dtype)
            with np.errstate(all="ignore"):
                base = np.round(rng.standard_normal(k) * spread)
                if kind == "c":
                    base = base + 1j * np.round(rng.standard_normal(k) * 2)
                x = base.astype(dtype)
            x[rng.random(k) < 0.02] = np.nan
            return x

        x = draw(n)
        what = f"seed={seed} case={case} {np.dtype(dtype)} n={n} spread={spread}"
        got = num.unique(num.array(x))
        want = numpy_unique(x)
        assert got.shape == want.shape and np.array_equal(np.asarray(got), want, equal_nan=True), what + " unique"
        srt = np.sort(x, kind="stable")
        v = draw(int(rng.choice([1, 50, 3000])))
        side = "left" if rng.random() < 0.5 else "right"
        got = np.asarray(num.searchsorted(num.array(srt), num.array(v), side=side))
        assert np.array_equal(got, np.searchsorted(srt, v, side=side)), what + f" searchsorted {side}"
        # lexsort: 1-4 keys of random types over a random 1-3 dimensional shape
        ndim = int(rng.integers(1, 4))
        shape = tuple(int(rng.integers(1, 30)) for _ in range(ndim - 1)) + (int(rng.choice([1, 9, 400, 9000])),)
        axis = int(rng.integers(-ndim, ndim))
        keys = []
        for _ in range(int(rng.integers(1, 5))):
            kd = dtypes[int(rng.integers(len(dtypes)))]
            if np.dtype(kd).kind == "b":
                keys.append(rng.integers(0, 2, shape).astype(kd))
            elif np.dtype(kd).kind in "iu":
                keys.append(rng.integers(0, 6, shape).astype(kd))
            else:
                with np.errstate(all="ignore"):
                    k = np.round(rng.standard_normal(shape) * 2).astype(kd)
                k[rng.random(shape) < 0.05] = np.nan
                keys.append(k)
        got = np.asarray(num.lexsort(tuple(num.array(k) for k in keys), axis=axis))
        assert np.array_equal(got, oracle.lexsort(tuple(keys), axis=axis)), what + f" lexsort {shape} axis={axis}"
