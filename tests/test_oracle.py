"""Pins the CPU oracle (oracle/sort_oracle.py + sort_oracle.c) before anything is checked
against it: the reference's golden vectors, NumPy's independent stable sort, closed forms and a
brute-force insertion sort on adversarial float alphabets.  CPU only."""
from __future__ import annotations

import itertools
import json

import numpy as np
import pytest
from conftest import ALL_REAL_DTYPES, COMPLEX_DTYPES, ROOT, assert_same_bits, case_array, make_input

from oracle import sort_oracle as oracle


# ---- golden vectors of the reference's own tests ------------------------------------------------
def test_reference_golden_vectors(reference_vectors):
    assert len(reference_vectors) == 390
    for case in reference_vectors:
        x = case_array(case["input"], case["dtype"], case["shape"])
        # kinds the reference runs the case with (tests/cpp/integration/test_argsort.cc:221-224)
        kinds = ["mergesort", "stable"] if case["stable_only"] else ["quicksort", "mergesort", "heapsort", "stable"]
        for kind in kinds:
            if case["op"] == "sort":
                got = oracle.sort(x, axis=case["axis"], kind=kind)
                want = case_array(case["expect"], case["dtype"], case["shape"])
            else:
                got = oracle.argsort(x, axis=case["axis"], kind=kind)
                want = np.array(case["expect"], dtype=np.int64).reshape(case["shape"])
            assert_same_bits(got, want, f"{case['where']} shape={case['shape']} axis={case['axis']} kind={kind}")


def test_reference_sort_complex_golden_vectors():
    # tests/cpp/integration/test_sort_complex.cc:27-195,257-345 (43 cases) and the formula case :347-390
    cases = json.loads((ROOT / "tests" / "golden" / "reference_vectors.json").read_text())["sort_complex_cases"]
    assert len(cases) == 43
    for c in cases:
        x = case_array(c["input"], c["in_dtype"], c["shape"])
        want = case_array(c["expect"], c["out_dtype"], c["shape"])
        got = oracle.sort_complex(x)
        assert got.dtype == want.dtype and got.shape == want.shape, c["where"]
        assert np.array_equal(got, want), (c["where"], c["shape"])
        assert np.array_equal(got, np.sort_complex(x).astype(want.dtype)), c["where"]
    count = 10000
    for dt, out in ((np.int16, np.complex64), (np.int32, np.complex128), (np.complex64, np.complex64)):
        x = (count - np.arange(count)).astype(dt)
        got = oracle.sort_complex(x)
        assert got.dtype == out and np.array_equal(got, (np.arange(count) + 1).astype(out))


def test_reference_large_reversed():
    # tests/cpp/integration/test_argsort.cc:379-410: 10 000 descending values -> N-1-j
    count = 10000
    want = count - 1 - np.arange(count, dtype=np.int64)
    assert np.array_equal(oracle.argsort(np.array([count - i for i in range(count)], dtype=np.int32)), want)
    assert np.array_equal(oracle.argsort(np.array([count * 1.1 - i for i in range(count)], dtype=np.float64)), want)


@pytest.mark.parametrize("shape", [(0,), (0, 1), (1, 0), (1, 0, 0), (1, 1, 0), (1, 0, 1)])
def test_reference_empty(shape):
    # tests/cpp/integration/test_argsort.cc:412-433, test_sort.cc:574-594
    x = np.zeros(shape, dtype=np.int32)
    for axis in range(-len(shape) + 1, len(shape)):
        assert oracle.sort(x, axis=axis).shape == shape
        assert oracle.argsort(x, axis=axis).shape == shape
        assert oracle.argsort(x, axis=axis).dtype == np.int64


@pytest.mark.parametrize("shape", [(1,), (1, 1), (1, 1, 1)])
def test_reference_single_item(shape):
    # tests/cpp/integration/test_argsort.cc:435-455, test_sort.cc:596-615
    x = np.full(shape, 12, dtype=np.int32)
    for axis in range(-len(shape) + 1, len(shape)):
        assert np.array_equal(oracle.sort(x, axis=axis), x)
        assert np.array_equal(oracle.argsort(x, axis=axis), np.zeros(shape, dtype=np.int64))


def test_reference_negative():
    # tests/cpp/integration/test_argsort.cc:457-467 (invalid axis); Python side raises ValueError
    # (cupynumeric/_thunk/deferred.py:5471-5472, tests/integration/test_sort.py:67-70)
    x = np.zeros((2, 3), dtype=np.int32)
    for axis in (2, -3):
        with pytest.raises(ValueError):
            oracle.argsort(x, axis=axis)
        with pytest.raises(ValueError):
            oracle.sort(x, axis=axis)
    with pytest.raises(NotImplementedError):
        oracle.sort(x, order="a")
    with pytest.raises(TypeError, match="cuPyNumeric does not support dtype="):
        oracle.sort(np.array(["a", "b"]))


# ---- NumPy's own stable sort as an independent implementation ------------------------------------
@pytest.mark.parametrize("dtype", ALL_REAL_DTYPES + COMPLEX_DTYPES)
@pytest.mark.parametrize("threads", [1, 4])
def test_against_numpy_1d(dtype, threads):
    for n in (1, 2, 3, 17, 24, 25, 1000, 70001):
        x = make_input(dtype, (n,), seed=n)
        assert np.array_equal(oracle.argsort(x, kind="stable", threads=threads), np.argsort(x, kind="stable"))
        assert_same_bits(oracle.sort(x, kind="stable", threads=threads), np.sort(x, kind="stable"), f"{dtype} n={n}")


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.float16, np.float64, np.uint8, np.complex64])
def test_against_numpy_axes(dtype):
    for shape in [(5, 5), (7, 1, 9), (3, 4, 5, 6), (33, 65)]:
        x = make_input(dtype, shape, seed=len(shape))
        for axis in list(range(-len(shape), len(shape))) + [None]:
            assert np.array_equal(oracle.argsort(x, axis=axis, kind="stable"), np.argsort(x, axis=axis, kind="stable"))
            assert_same_bits(oracle.sort(x, axis=axis), np.sort(x, axis=axis, kind="stable"), f"{shape} axis={axis}")


def test_parallel_segment_matches_serial():
    x = make_input(np.float32, (3, 200000), seed=5)
    assert np.array_equal(oracle.argsort(x, threads=1), oracle.argsort(x, threads=oracle.max_threads()))


# ---- closed forms ------------------------------------------------------------------------------
def test_closed_forms():
    n = 5003
    iota = np.arange(n, dtype=np.int64)
    assert np.array_equal(oracle.argsort(np.full(n, 7, dtype=np.int16)), iota)  # all equal -> identity
    assert np.array_equal(oracle.argsort(iota.astype(np.float32)), iota)  # sorted -> identity
    assert np.array_equal(oracle.argsort(-iota), iota[::-1])  # reversed distinct
    perm = np.random.default_rng(1).permutation(n)
    inv = np.empty(n, dtype=np.int64)
    inv[perm] = iota
    assert np.array_equal(oracle.argsort(perm.astype(np.uint32)), inv)  # argsort of a permutation = inverse
    # row-relative indices: every row of an N-D argsort is a permutation of 0..seg-1
    idx = oracle.argsort(make_input(np.int8, (11, 300), seed=2))
    assert np.array_equal(np.sort(idx, axis=-1), np.broadcast_to(np.arange(300), (11, 300)))


# ---- brute force over an adversarial float alphabet --------------------------------------------
def numpy_rule_less(a: float, b: float) -> bool:
    """a sorts strictly before b: a < b, or b is NaN and a is not."""
    return bool(a < b or (b != b and a == a))


def insertion_argsort(x: np.ndarray) -> list[int]:
    order: list[int] = []
    for i, v in enumerate(x):
        j = len(order)
        while j > 0 and numpy_rule_less(float(v), float(x[order[j - 1]])):
            j -= 1
        order.insert(j, i)
    return order


@pytest.mark.parametrize("dtype,ubits", [(np.float16, np.uint16), (np.float32, np.uint32), (np.float64, np.uint64)])
def test_bruteforce_float_alphabet(dtype, ubits):
    dt = np.dtype(dtype)
    nan = np.array(np.nan, dtype=dt).view(ubits)
    sign = ubits(1) << ubits(dt.itemsize * 8 - 1)
    alphabet_bits = [
        nan, nan | sign, nan | ubits(1),  # +NaN, -NaN, NaN with payload
        np.array(-np.inf, dtype=dt).view(ubits), np.array(np.inf, dtype=dt).view(ubits),
        np.array(-1.0, dtype=dt).view(ubits), np.array(1.0, dtype=dt).view(ubits),
        sign, ubits(0),  # -0.0, +0.0
        ubits(1), sign | ubits(1),  # smallest subnormals
    ]
    alphabet = np.array(alphabet_bits, dtype=ubits).view(dt)
    # all length-3 words over the alphabet, plus a long random word
    for word in itertools.product(range(len(alphabet)), repeat=3):
        x = alphabet[list(word)]
        got = oracle.argsort(x, kind="stable")
        assert got.tolist() == insertion_argsort(x), (dtype, word)
        assert_same_bits(oracle.sort(x), x[got])
    rng = np.random.default_rng(7)
    x = alphabet[rng.integers(0, len(alphabet), 400)]
    got = oracle.argsort(x, kind="stable")
    assert got.tolist() == insertion_argsort(x)
    assert_same_bits(oracle.sort(x), x[got])


# ---- complex: brute force with NumPy's rule written from its definition ----------------------------
def complex_rule_less(a: complex, b: complex) -> bool:
    """a sorts strictly before b: classes (no NaN) < (imag NaN) < (real NaN) < (both NaN); inside a
    class by real then imag, by real, by imag, none."""
    def key(z):
        rn, inn = z.real != z.real, z.imag != z.imag
        cls = 2 * rn + inn
        return cls, (z.real if not rn else (z.imag if not inn else 0.0)), (z.imag if cls == 0 else 0.0)
    (ca, pa, sa), (cb, pb, sb) = key(a), key(b)
    if ca != cb:
        return ca < cb
    if pa != pb:
        return pa < pb
    return sa < sb


@pytest.mark.parametrize("dtype", COMPLEX_DTYPES)
def test_bruteforce_complex_alphabet(dtype):
    part = [np.nan, -np.inf, -1.0, -0.0, 0.0, 1.0, np.inf]
    alphabet = np.empty(len(part) ** 2, dtype=dtype)
    alphabet.real = np.repeat(part, len(part))
    alphabet.imag = np.tile(part, len(part))
    rng = np.random.default_rng(11)
    for trial in range(40):
        x = alphabet[rng.integers(0, len(alphabet), 60)]
        order: list[int] = []
        for i, v in enumerate(x):
            j = len(order)
            while j > 0 and complex_rule_less(complex(v), complex(x[order[j - 1]])):
                j -= 1
            order.insert(j, i)
        got = oracle.argsort(x, kind="stable")
        assert got.tolist() == order, (dtype, trial)
        assert got.tolist() == np.argsort(x, kind="stable").tolist()
        assert_same_bits(oracle.sort(x), x[got])


# ---- lexsort (cupynumeric/_module/ssc_sorting.py:271-444) ------------------------------------------
def test_lexsort_matches_numpy_on_reference_cases():
    """Every input of the reference's tests/integration/test_lexsort.py, and random keys with ties
    and special values: the restated loop must agree with NumPy's independent lexsort."""
    from lexsort_cases import cases, random_cases

    for name, keys, axis in cases() + random_cases():
        want = np.lexsort(keys, axis=axis)
        got = oracle.lexsort(keys, axis=axis)
        assert got.dtype == np.int64 and got.shape == want.shape, name
        assert np.array_equal(got, want), name


def test_lexsort_errors():
    # tests/integration/test_lexsort.py:197-225,328-334,441-472,721-760
    with pytest.raises(TypeError):
        oracle.lexsort(None)
    with pytest.raises(TypeError):
        oracle.lexsort(())
    with pytest.raises(ValueError):
        oracle.lexsort((np.arange(100), np.arange(50)))
    with pytest.raises(ValueError):
        oracle.lexsort((np.arange(25).reshape(5, 5), np.arange(25)))
    for axis in (2, -3):
        with pytest.raises(np.exceptions.AxisError):
            oracle.lexsort((np.zeros((10, 100)), np.zeros((10, 100))), axis=axis)
    with pytest.raises(TypeError, match="'NoneType' object cannot be interpreted as an integer"):
        oracle.lexsort((np.arange(3), np.arange(3)), axis=None)
    with pytest.raises(TypeError, match="cuPyNumeric does not support dtype"):
        oracle.lexsort((("Heinrich", "Galileo", "Gustav"), ("Hertz", "Galilei", "Hertz")))


# ---- searchsorted / unique ---------------------------------------------------------------------------
def _consumer_inputs(dt, size, rng):
    if np.dtype(dt).kind == "c":
        a = (rng.integers(0, 5, size) + 1j * rng.integers(0, 5, size)).astype(dt)
        if size > 4:
            a[::7] = complex(np.nan, 1)
            a[3] = complex(2, np.nan)
            a[4] = complex(np.nan, np.nan)
        v = (rng.integers(-1, 6, 31) + 1j * rng.integers(-1, 6, 31)).astype(dt)
        v[5] = complex(np.nan, 0)
        v[6] = complex(1, np.nan)
    elif np.dtype(dt).kind == "f":
        a = np.round(rng.standard_normal(size) * 3).astype(dt)
        if size > 4:
            a[::5] = np.nan
            a[1], a[2], a[3] = -0.0, 0.0, np.inf
        v = np.round(rng.standard_normal(31) * 3).astype(dt)
        v[3], v[4], v[5] = np.nan, -0.0, -np.inf
    else:
        hi = 2 if dt == np.bool_ else 50
        a = rng.integers(0, hi, size).astype(dt)
        v = rng.integers(0, hi + (0 if dt == np.bool_ else 10), 31).astype(dt)
    return a, v


@pytest.mark.parametrize("dtype", ALL_REAL_DTYPES + COMPLEX_DTYPES)
def test_searchsorted_and_unique_match_numpy(dtype):
    """NumPy's own searchsorted / unique are the independent statement of the contract (NaN last and
    equal to itself, complex values with a NaN part one value for unique)."""
    rng = np.random.default_rng(np.dtype(dtype).num)
    for size in (0, 1, 2, 17, 200):
        a, v = _consumer_inputs(dtype, size, rng)
        srt = np.sort(a, kind="stable")
        order = np.argsort(a, kind="stable")
        for side in ("left", "right"):
            assert np.array_equal(oracle.searchsorted(srt, v, side), np.searchsorted(srt, v, side))
            v2 = v.reshape(-1, 1)
            assert np.array_equal(
                oracle.searchsorted(a, v2, side, sorter=order), np.searchsorted(a, v2, side, sorter=order)
            )
        # (float16 through float32, exact: NumPy 2.2.6's default float16 sort mis-sorts -0.0 on AVX-512)
        u, w = oracle.unique(a), (np.unique(a.astype(np.float32)).astype(a.dtype) if a.dtype == np.float16 else np.unique(a))
        assert u.dtype == w.dtype and u.shape == w.shape and np.array_equal(u, w, equal_nan=True)


def test_searchsorted_common_type_and_errors():
    # tests/integration/test_searchsorted.py:46-53 (dtype pairs), :79-128 (errors)
    rng = np.random.default_rng(3)
    for n, d1, d2 in [(3, np.uint64, np.float32), (51, np.uint32, np.complex64), (23, np.uint32, np.float64),
                      (51, np.complex64, np.float64), (21, np.complex64, np.int32), (22, np.complex128, np.float32)]:
        a = np.sort((rng.random(n) * 100).astype(d1))
        v = (rng.random(10) * 100).astype(d2)
        for side in ("left", "right"):
            assert np.array_equal(oracle.searchsorted(a, v, side), np.searchsorted(a, v, side))
    with pytest.raises(ValueError):
        oracle.searchsorted(rng.random((5, 5, 5)), 5)
    with pytest.raises(ValueError):
        oracle.searchsorted(np.arange(100), np.arange(10), sorter=np.arange(10))
    with pytest.raises(TypeError):
        oracle.searchsorted([2, 3, 10, 9], None)


def test_thrust_baseline_matches_numpy_on_plain_data():
    """The second CPU baseline of bench.py (the reference's per-row thrust calls over rocThrust's host
    backends) is only a timing baseline; on data without NaN and -0.0, where bit-pattern order and
    NumPy's order coincide, its output is checked here."""
    rng = np.random.default_rng(21)
    for dtype in (np.int32, np.int64, np.uint8, np.float32, np.float64):
        if np.dtype(dtype).kind == "f":
            x = rng.standard_normal((7, 3001)).astype(dtype)
        else:
            info = np.iinfo(dtype)
            x = rng.integers(info.min, info.max, (7, 3001), dtype=dtype, endpoint=True)
        for use_omp in (False, True):
            for transparent in (False, True):  # thrust::less<VAL> (radix sort) and thrust::less<> (merge sort)
                kw = dict(use_omp=use_omp, transparent=transparent)
                assert np.array_equal(oracle.thrust_local_sort(x, False, **kw), np.sort(x, axis=-1, kind="stable"))
                assert np.array_equal(oracle.thrust_local_sort(x, True, **kw), np.argsort(x, axis=-1, kind="stable"))


def test_unique_reference_golden_vectors():
    from conftest import UNIQUE_GOLDEN

    for values, shape, expected, dtype in UNIQUE_GOLDEN:
        got = oracle.unique(np.array(values, dtype=dtype).reshape(shape))
        assert got.dtype == np.dtype(dtype) and got.tolist() == expected


# ---- order statistics -------------------------------------------------------------------------------
QUANTILE_METHODS = ("inverted_cdf", "averaged_inverted_cdf", "closest_observation", "interpolated_inverted_cdf", "hazen",
                    "weibull", "linear", "median_unbiased", "normal_unbiased", "lower", "higher", "midpoint", "nearest")
# tests/integration/test_quantiles.py:44-73: the reference's own input
QUANTILE_REF_INPUT = np.array([1, 2, 2, 40, 1, 1, 2, 1, 0, 10, 3, 3, 40, 15, 3, 7, 5, 4, 7, 3, 5, 1, 0, 9], dtype=int).reshape(2, 3, 4)
QUANTILE_REF_QS = (0.5, [0.001, 0.37, 0.42, 0.67, 0.83, 0.99, 0.39, 0.49, 0.5])


@pytest.mark.parametrize("method", QUANTILE_METHODS)
def test_quantile_matches_numpy_on_the_reference_cases(method):
    """The oracle's quantile / percentile / median against numpy's on the inputs, axes, quantiles and
    keepdims of tests/integration/test_quantiles.py:36-111 and test_percentiles.py, to the reference's
    own tolerance (atol 1e-8: its interpolation formula is not NumPy's), exactly for methods that pick
    samples; plus float inputs, axis=None and 1-D."""
    eps = 1.0e-8
    rng = np.random.default_rng(44)
    inputs = [QUANTILE_REF_INPUT, QUANTILE_REF_INPUT.astype(np.float64) / 3, rng.standard_normal((2, 3, 4)).astype(np.float32),
              rng.integers(0, 100, (5, 7)).astype(np.uint8)]
    for arr in inputs:
        for axes in (None, 0, 1, (0,), (0, 1), (0, 2) if arr.ndim == 3 else (1,)):
            for qs in QUANTILE_REF_QS:
                for keepdims in (False, True):
                    want = np.quantile(arr, qs, axis=axes, method=method, keepdims=keepdims)
                    got = oracle.quantile(arr, qs, axis=axes, method=method, keepdims=keepdims)
                    assert got.shape == want.shape
                    if arr.dtype != np.float32:
                        assert got.dtype == want.dtype, (method, axes, got.dtype, want.dtype)
                    else:  # the reference gives float64 for every float narrower than that (stats_order.py:501-510), NumPy float32
                        assert got.dtype == (np.float32 if method in ("inverted_cdf", "closest_observation", "lower", "higher", "nearest") else np.float64)
                    if method in ("inverted_cdf", "closest_observation", "lower", "higher", "nearest"):
                        assert np.array_equal(got, want), (method, axes, qs)
                    else:
                        assert np.allclose(got, want, atol=eps if arr.dtype != np.float32 else 1e-6), (method, axes, qs)
                    p = oracle.percentile(arr, np.asarray(qs) * 100.0, axis=axes, method=method, keepdims=keepdims)
                    assert np.allclose(p, np.percentile(arr, np.asarray(qs) * 100.0, axis=axes, method=method, keepdims=keepdims),
                                       atol=1e-6)
    for arr in inputs:
        for axes in (None, 0, -1):
            assert np.allclose(oracle.median(arr, axis=axes), np.median(arr, axis=axes), atol=1e-6)
            assert oracle.median(arr, axis=axes, keepdims=True).shape == np.median(arr, axis=axes, keepdims=True).shape


def test_quantile_closed_forms():
    x = np.arange(101, dtype=np.float64)[::-1].copy()
    assert np.array_equal(oracle.quantile(x, [0.0, 0.25, 0.5, 1.0]), [0.0, 25.0, 50.0, 100.0])
    assert oracle.median(np.array([3, 1, 2, 10])) == 2.5
    assert oracle.quantile(np.array([7]), 0.3, method="weibull") == 7.0
    with pytest.raises(TypeError):
        oracle.quantile(np.array([1 + 2j, 3j]), 0.5)


# tests/integration/test_nanquantiles.py:47-58: the reference's own input
NANQUANTILE_REF_INPUT = np.asarray([[1.0, 2, 2, 40], [1, np.nan, 2, 1], [0, 10, np.nan, np.nan], [np.nan, np.nan, 0, 10],
                                    [np.nan, np.nan, np.nan, np.nan]])


@pytest.mark.parametrize("method", QUANTILE_METHODS)
def test_nanquantile_matches_numpy_on_the_reference_cases(method):
    """The oracle's nanquantile / nanpercentile / nanmedian against numpy's on the input, axes and
    quantiles of tests/integration/test_nanquantiles.py:41-103 and test_nanpercentiles.py (atol 1e-8,
    exactly for the methods that pick samples), on random float64 / float32 data with NaNs scattered
    and whole slices of NaN, every axis, keepdims, and axis=None (test_keepdims, :106-111)."""
    import warnings

    rng = np.random.default_rng(45)
    rnd = rng.standard_normal((4, 6, 5))
    rnd[rng.random(rnd.shape) < 0.3] = np.nan
    rnd[1, :, 2] = np.nan
    inputs = [NANQUANTILE_REF_INPUT, rnd, rnd.astype(np.float32)]
    picks = method in ("inverted_cdf", "closest_observation", "lower", "higher", "nearest")
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)  # NumPy warns about slices of NaN only
        for arr in inputs:
            axes_list = (0, 1, (0, 1), (0,), None) + (((0, 2), 2) if arr.ndim == 3 else ())
            for axes in axes_list:
                for qs in QUANTILE_REF_QS:
                    for keepdims in (False, True):
                        want = np.nanquantile(arr, qs, axis=axes, method=method, keepdims=keepdims)
                        got = oracle.nanquantile(arr, qs, axis=axes, method=method, keepdims=keepdims)
                        assert got.shape == want.shape, (method, axes, keepdims)
                        if arr.dtype == np.float64:
                            assert got.dtype == want.dtype
                        else:  # float64 unless the method picks samples (stats_order.py:893-903); NumPy keeps float32
                            assert got.dtype == (np.float32 if picks else np.float64)
                        if picks:
                            assert np.array_equal(got, want, equal_nan=True), (method, axes, qs)
                        else:
                            assert np.allclose(got, want, atol=1e-8 if arr.dtype == np.float64 else 1e-5, equal_nan=True), (method, axes, qs)
                        p = oracle.nanpercentile(arr, np.asarray(qs) * 100.0, axis=axes, method=method, keepdims=keepdims)
                        assert np.allclose(p, np.nanpercentile(arr, np.asarray(qs) * 100.0, axis=axes, method=method, keepdims=keepdims),
                                           atol=1e-5, equal_nan=True)
        for arr in inputs:
            for axes in (None, 0, -1):
                assert np.allclose(oracle.nanmedian(arr, axis=axes), np.nanmedian(arr, axis=axes), atol=1e-6, equal_nan=True)


def test_nanquantile_closed_forms_and_the_reference_quirks():
    # no NaN at all: the same positions as quantile (weights in the array's type make no difference for float64)
    x = np.arange(101, dtype=np.float64)[::-1].copy()
    assert np.array_equal(oracle.nanquantile(x, [0.0, 0.25, 0.5, 1.0]), [0.0, 25.0, 50.0, 100.0])
    # NaNs are dropped: the median of {1, 2, 10} and of {4}
    assert oracle.nanmedian(np.array([np.nan, 10.0, 1.0, np.nan, 2.0])) == 2.0
    assert np.array_equal(oracle.nanmedian(np.array([[np.nan, 4.0], [np.nan, np.nan]]), axis=1), [4.0, np.nan], equal_nan=True)
    # float32: the weight 0.3 is rounded to float32 and so is every step (stats_order.py:708-710,748-757)
    v = np.array([1.0, 2.0, np.nan], dtype=np.float32)
    g = np.float32(0.3)
    assert oracle.nanquantile(v, 0.3) == np.float64((np.float32(1) - g) * np.float32(1.0) + g * np.float32(2.0))
    # NaNs become the largest finite value BEFORE the sort (stats_order.py:886-887), so with +inf in the
    # same slice the position after the last finite element reads that value, where NumPy reads +inf
    w = np.array([1.0, np.inf, np.nan])
    assert oracle.nanquantile(w, 1.0, method="lower") == np.finfo(np.float64).max
    assert np.nanquantile(w, 1.0, method="lower") == np.inf
    with pytest.raises(TypeError):
        oracle.nanquantile(np.array([1 + 2j, np.nan + 0j]), 0.5)
    with pytest.raises(ValueError):
        oracle.nanquantile(np.array([1, 2, 3]), 0.5)  # numpy.finfo of an integer type, as in the reference
