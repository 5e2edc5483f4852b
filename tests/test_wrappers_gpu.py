"""Thin wrappers on the sort path: sort_complex, partition, argpartition
(cupynumeric/_module/ssc_sorting.py:124-268, tests/integration/test_sort_complex.py,
test_partition.py)."""
from __future__ import annotations

import numpy as np
import pytest
from conftest import ALL_REAL_DTYPES, make_input

import cupynumeric_amd as num

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ALL_REAL_DTYPES + [np.complex64, np.complex128])
def test_sort_complex_matches_numpy(dtype):
    for shape in [(12,), (3, 4), (2, 2, 3), (0,), (1,)]:
        x = make_input(dtype, shape, seed=3, special=False)
        if np.dtype(dtype).kind == "f":
            x = np.round(x * 4) / 4
        got = num.sort_complex(num.array(x))
        want = np.sort_complex(x)
        assert got.dtype == want.dtype, (dtype, got.dtype, want.dtype)
        assert got.shape == want.shape
        assert np.array_equal(np.asarray(got), want)


def test_sort_complex_reference_golden_vectors():
    # tests/cpp/integration/test_sort_complex.cc:27-195,257-345 through the public API; the
    # 10 000-element reversed input of :347-390 by its formula
    import json

    from conftest import ROOT, case_array

    from oracle import sort_oracle as oracle

    cases = json.loads((ROOT / "tests" / "golden" / "reference_vectors.json").read_text())["sort_complex_cases"]
    assert len(cases) == 43
    for c in cases:
        x = case_array(c["input"], c["in_dtype"], c["shape"])
        want = case_array(c["expect"], c["out_dtype"], c["shape"])
        got = num.sort_complex(num.array(x))
        assert got.dtype == want.dtype and got.shape == want.shape, c["where"]
        assert np.array_equal(np.asarray(got), want), (c["where"], c["shape"])
        assert np.array_equal(np.asarray(got), oracle.sort_complex(x)), c["where"]
    count = 10000
    for dt, out in ((np.int16, np.complex64), (np.int32, np.complex128), (np.complex64, np.complex64)):
        x = (count - np.arange(count)).astype(dt)
        got = num.sort_complex(num.array(x))
        assert got.dtype == out and np.array_equal(np.asarray(got), (np.arange(count) + 1).astype(out))


def partition_property(part: np.ndarray, original: np.ndarray, kth: int, axis: int) -> None:
    """tests/integration/test_partition.py:23-47: everything left of kth is <=, right is >=; and
    the element at kth is the one a full sort puts there."""
    p = np.moveaxis(part, axis, -1)
    s = np.moveaxis(np.sort(original, axis=axis, kind="stable"), axis, -1)
    assert np.array_equal(p[..., kth], s[..., kth])
    if kth > 0:
        assert (p[..., :kth].max(axis=-1) <= p[..., kth]).all()
    assert (p[..., kth:].min(axis=-1) >= p[..., kth]).all()
    assert np.array_equal(np.sort(p, axis=-1), s)  # same multiset per row


@pytest.mark.parametrize("dtype", [np.uint32, np.int8, np.float32, np.float64])
def test_partition_and_argpartition(dtype):
    for shape in [(30,), (7, 11), (3, 4, 5)]:
        x = make_input(dtype, shape, seed=9, special=False)
        a = num.array(x)
        for axis in range(-len(shape), len(shape)):
            for kth in (0, shape[axis] // 2, shape[axis] - 1):
                partition_property(np.asarray(num.partition(a, kth, axis=axis)), x, kth, axis)
                idx = np.asarray(num.argpartition(a, kth, axis=axis))
                assert idx.dtype == np.int64 and idx.shape == x.shape
                partition_property(np.take_along_axis(x, idx, axis=axis), x, kth, axis)
                assert np.array_equal(np.asarray(a.argpartition(kth, axis=axis)), idx)
                b = num.array(x)
                b.partition(kth, axis=axis)
                partition_property(np.asarray(b), x, kth, axis)
    flat = num.partition(num.array(make_input(np.int32, (4, 5), seed=1)), 3, axis=None)
    assert flat.shape == (20,)


def test_partition_validation():
    a = num.array(np.arange(6).reshape(2, 3))
    with pytest.raises(ValueError, match="invalid axis"):
        num.partition(a, 1, axis=2)
    with pytest.raises(NotImplementedError):
        num.argpartition(a, 1, order="x")


# ---- lexsort (cupynumeric/_module/ssc_sorting.py:271-444, tests/integration/test_lexsort.py) ---------
def test_lexsort_reference_cases():
    from lexsort_cases import cases, random_cases

    from oracle import sort_oracle as oracle

    for name, keys, axis in cases() + random_cases():
        want = oracle.lexsort(keys, axis=axis)
        assert np.array_equal(want, np.lexsort(keys, axis=axis)), name
        if isinstance(keys, np.ndarray):
            got = num.lexsort(num.array(keys), axis=axis)
        else:
            got = num.lexsort(tuple(num.array(k) for k in keys), axis=axis)
        assert got.dtype == np.int64 and got.shape == want.shape, name
        assert np.array_equal(np.asarray(got), want), name


def test_lexsort_large_rows_and_global_path():
    """Keys long enough for the global radix path, 1-D and along the first axis."""
    from oracle import sort_oracle as oracle

    rng = np.random.default_rng(5)
    n = 300_000
    k1 = rng.integers(0, 1000, n).astype(np.int32)
    k2 = rng.integers(0, 50, n).astype(np.float64)
    k3 = rng.integers(0, 7, n).astype(np.uint8)
    got = np.asarray(num.lexsort((num.array(k1), num.array(k2), num.array(k3))))
    assert np.array_equal(got, oracle.lexsort((k1, k2, k3), threads=8))
    a = rng.integers(0, 5, (20_000, 6)).astype(np.int16)
    b = rng.integers(0, 5, (20_000, 6)).astype(np.float32)
    got = np.asarray(num.lexsort((num.array(a), num.array(b)), axis=0))
    assert np.array_equal(got, np.lexsort((a, b), axis=0))


def test_take_along_last_axis_bounds():
    a = num.array(np.arange(12, dtype=np.float32).reshape(3, 4))
    idx = num.array(np.array([[0, -1], [3, 1], [-4, 2]], dtype=np.int64))
    got = a._thunk.take_along_last_axis(idx._thunk)
    assert np.array_equal(got.__numpy_array__(), np.take_along_axis(np.asarray(a), np.asarray(idx), axis=-1))
    bad = num.array(np.array([[0, 4], [0, 0], [0, 0]], dtype=np.int64))
    with pytest.raises(IndexError):
        a._thunk.take_along_last_axis(bad._thunk)


def test_lexsort_pack_c_abi():
    """cpn_lexsort_pack directly: the unsigned order of the packed words is the lexicographic order of
    the keys, with and without reading through a permutation; widths that do not fit are refused."""
    import ctypes

    import torch

    from cupynumeric_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda")
    rng = np.random.default_rng(8)
    rows, seg = 3, 1000
    k0 = rng.integers(-3, 3, (rows, seg)).astype(np.int8)
    k1 = np.round(rng.standard_normal((rows, seg)) * 2).astype(np.float16)
    k1[rng.random((rows, seg)) < 0.05] = np.nan
    k1[rng.random((rows, seg)) < 0.05] = -0.0
    k2 = rng.integers(0, 2, (rows, seg)).astype(np.bool_)
    k3 = rng.integers(-2, 2, (rows, seg)).astype(np.int32)
    keys = [k0, k1, k2, k3]  # 1 + 2 + 1 + 4 = 8 bytes
    d_keys = [torch.from_numpy(k.view(np.uint8).reshape(-1).copy()).to(dev) for k in keys]
    dtypes = (ctypes.c_int * 4)(*[_lib.DTYPE_CODES[k.dtype] for k in keys])
    ptrs = (ctypes.c_void_p * 4)(*[d.data_ptr() for d in d_keys])
    out = torch.zeros(rows * seg, dtype=torch.int64, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.cpn_lexsort_pack(4, dtypes, ptrs, None, 8, out.data_ptr(), rows, seg, stream) == 0
    packed = out.cpu().numpy().view(np.uint64).reshape(rows, seg)
    assert np.array_equal(np.argsort(packed, axis=-1, kind="stable"), np.lexsort(keys, axis=-1))
    perm = np.stack([rng.permutation(seg) for _ in range(rows)]).astype(np.int64)
    d_perm = torch.from_numpy(perm.reshape(-1)).to(dev)
    assert lib.cpn_lexsort_pack(4, dtypes, ptrs, d_perm.data_ptr(), 8, out.data_ptr(), rows, seg, stream) == 0
    assert np.array_equal(out.cpu().numpy().view(np.uint64).reshape(rows, seg), np.take_along_axis(packed, perm, axis=-1))
    assert lib.cpn_lexsort_pack(4, dtypes, ptrs, None, 4, out.data_ptr(), rows, seg, stream) == -3  # 8 bytes into 4
    cdt = (ctypes.c_int * 1)(_lib.DTYPE_CODES[np.dtype(np.complex64)])
    assert lib.cpn_lexsort_pack(1, cdt, ptrs, None, 8, out.data_ptr(), rows, seg, stream) == -1


def test_take_along_axis_public():
    """tests/integration/test_take_along_axis.py in the no-broadcast form: argsort indices reproduce the
    sort, every axis, negative indices, flattened form, error cases."""
    rng = np.random.default_rng(10)
    for shape in [(7,), (5, 9), (3, 4, 6), (2, 3, 4, 5)]:
        x = rng.standard_normal(shape).astype(np.float32)
        a = num.array(x)
        for axis in range(-len(shape), len(shape)):
            idx = num.argsort(a, axis=axis, kind="stable")
            got = num.take_along_axis(a, idx, axis)
            assert np.array_equal(np.asarray(got), np.sort(x, axis=axis))
            k = rng.integers(-shape[axis], shape[axis], shape).astype(np.int32)  # other integer type, negatives
            assert np.array_equal(np.asarray(num.take_along_axis(a, k, axis)), np.take_along_axis(x, k.astype(np.int64), axis))
        short = tuple(2 if d == len(shape) - 1 else s for d, s in enumerate(shape))  # fewer picks than elements
        k = rng.integers(0, shape[-1], short)
        assert np.array_equal(np.asarray(num.take_along_axis(a, k, -1)), np.take_along_axis(x, k, -1))
    x = rng.integers(0, 100, (4, 5))
    k = rng.integers(0, 20, 7)
    assert np.array_equal(np.asarray(num.take_along_axis(num.array(x), k, None)), np.take_along_axis(x, k, None))
    with pytest.raises(TypeError):
        num.take_along_axis(x, np.zeros((4, 5)), 0)
    with pytest.raises(ValueError):
        num.take_along_axis(x, np.zeros((4, 5), dtype=int), None)
    with pytest.raises(ValueError):
        num.take_along_axis(x, np.zeros(3, dtype=int), 0)
    with pytest.raises(IndexError):
        num.take_along_axis(x, np.full((4, 5), 5), 1)
    with pytest.raises(np.exceptions.AxisError):
        num.take_along_axis(x, np.zeros((4, 5), dtype=int), 2)


def test_take_along_axis_broadcasts_like_numpy():
    """Every dimension but the axis may be 1 on either side (`cupynumeric/_module/indexing.py:700-760`,
    where the reference gathers through coordinate arrays): against numpy.take_along_axis."""
    rng = np.random.default_rng(12)
    cases = [((4, 7), (1, 3), 1), ((1, 7), (5, 3), 1), ((4, 7), (2, 1), 0), ((4, 1), (3, 6), 0),
             ((3, 1, 5), (1, 4, 2), 2), ((3, 4, 5), (3, 1, 5), 1), ((1, 4, 1, 6), (2, 3, 5, 1), 1),
             ((2, 1, 3, 1, 2), (1, 3, 2, 4, 1), 2), ((6,), (9,), 0), ((3, 5), (3, 0), 1), ((1, 5), (0, 2), 1)]
    for a_shape, i_shape, axis in cases:
        for dtype in (np.float32, np.int16, np.complex128):
            x = (rng.standard_normal(a_shape) * 100).astype(dtype)
            k = rng.integers(-a_shape[axis], a_shape[axis], i_shape)
            want = np.take_along_axis(x, k, axis)
            got = np.asarray(num.take_along_axis(num.array(x), num.array(k), axis))
            assert got.shape == want.shape and np.array_equal(got, want), (a_shape, i_shape, axis, dtype)
    # shapes that do not broadcast: IndexError, as in NumPy (`tests/integration/test_take_along_axis.py:378-384`)
    with pytest.raises(IndexError, match="shape mismatch: indexing arrays could not be broadcast"):
        num.take_along_axis(num.array(np.ones((3, 3))), num.array(np.ones((3, 2), dtype=int)), 0)
    # out of bounds in the broadcast form is reported from the call too
    with pytest.raises(IndexError, match="out of bounds"):
        num.take_along_axis(num.array(np.ones((3, 3))), num.array(np.full((1, 3), 3)), 0)


def test_getitem_with_an_integer_array():
    """`arr.flatten()[argsort result]`, as `tests/integration/test_argsort.py:229-245` writes it, over that
    file's shapes; NumPy indices, lists and negative positions; an index out of range surfaces as
    IndexError with the next host read."""
    rng = np.random.default_rng(13)
    dim = 5
    sizes = [(0,), (1,), (dim,), (0, 1), (1, 0), (1, 1), (1, dim), (dim, 1), (dim, dim), (1, 0, 0), (1, 1, 0), (1, 0, 1),
             (1, 1, 1), (dim, 1, 1), (1, dim, 1), (1, 1, dim), (dim, dim, dim)]
    for size in sizes:
        arr_np = rng.integers(-100, 100, size)
        arr_num = num.array(arr_np)
        res_np = np.argsort(arr_np, axis=None)
        res_num = num.argsort(arr_num, axis=None)
        assert res_num.shape == (int(np.prod(size)),)
        sorted_np = arr_np.flatten()[res_np]
        sorted_num = arr_num.flatten()[res_num]
        assert np.array_equal(np.asarray(sorted_num), sorted_np), size
    x = rng.standard_normal(1000).astype(np.float32)
    a = num.array(x)
    k = rng.integers(-1000, 1000, 300)
    assert np.array_equal(np.asarray(a[k]), x[k])
    assert np.array_equal(np.asarray(a[k.astype(np.int32)]), x[k])
    assert np.array_equal(np.asarray(a[[5, -1, 0]]), x[[5, -1, 0]])
    assert np.asarray(a[[]]).shape == (0,)
    with pytest.raises(NotImplementedError):
        a[3]
    with pytest.raises(NotImplementedError):
        num.array(np.ones((2, 2)))[np.array([0])]
    bad = a[np.array([0, 1000])]  # issued without a host read ...
    with pytest.raises(IndexError, match="out of bounds"):
        np.asarray(bad)  # ... and reported with the first one
    assert np.array_equal(np.asarray(a[k]), x[k])  # the layer has recovered


def test_searchsorted_sorter_does_not_synchronise(monkeypatch):
    """The out-of-bounds flag of the gather behind `sorter` travels with the deferred status words: no
    host read happens inside the call."""
    from cupynumeric_amd.runtime import runtime

    rng = np.random.default_rng(14)
    x = rng.standard_normal(5000).astype(np.float32)
    order = np.argsort(x, kind="stable")
    v = rng.standard_normal(100).astype(np.float32)
    a, s = num.array(x), num.array(order)
    np.asarray(a), np.asarray(s)
    monkeypatch.setattr(runtime, "check_mode", "lazy")
    before = runtime._status_used
    got = num.searchsorted(a, v, sorter=s)
    assert runtime._status_used == before + 1 and runtime._status_kinds[-1] == "index"
    assert np.array_equal(np.asarray(got), np.searchsorted(x, v, sorter=order))
    assert runtime._status_used == 0


def test_astype_float16_rounds_once():
    """Casts to float16 from wider types must round to nearest even once, as NumPy does: values on and
    around the midpoints between neighbouring float16 numbers, where rounding to float32 first and to
    float16 afterwards lands on the other neighbour."""
    halves = np.array([1.0, 1.5, 1023.0, 2048.0, 6.1e-5, 5.96e-8, 3.0e-6, 65472.0, 0.333], dtype=np.float16)
    nxt = np.nextafter(halves, np.float16(np.inf))
    mid = (halves.astype(np.float64) + nxt.astype(np.float64)) / 2  # exact midpoints (representable in float64)
    eps = np.abs(mid) * 2.0**-40
    x = np.concatenate([mid, mid + eps, mid - eps, -mid, -(mid + eps), -(mid - eps),
                        [65519.99, 65520.0, 65520.01, 1e300, -1e300, 2.0**-25, 2.0**-25 * (1 + 2.0**-30), np.nan, np.inf]])
    got = np.asarray(num.array(x).astype(np.float16))
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    assert np.array_equal(got.view(np.uint16)[~np.isnan(want)], want.view(np.uint16)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()
    for dt in (np.int64, np.uint64, np.int32):
        v = np.array([0, 1, 2047, 2049, 4097, 4099, 65503, 65519, 65520, 70000, 2**30 + 1], dtype=dt)
        if np.dtype(dt).itemsize == 8:
            v = np.concatenate([v, np.array([2**40 + 1, 2**62 + 12345], dtype=dt)])
        if np.dtype(dt).kind == "i":
            v = np.concatenate([v, -v])
        with np.errstate(over="ignore"):
            want = v.astype(np.float16)
        assert np.array_equal(np.asarray(num.array(v).astype(np.float16)).view(np.uint16), want.view(np.uint16)), dt
