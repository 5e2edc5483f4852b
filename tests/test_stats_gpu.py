"""quantile / percentile / median and their NaN-ignoring variants on top of the HIP sort (cupynumeric/_module/stats_order.py:358-650,
stats_avgs_vars.py:373-443) against the CPU oracle's restatement of the reference, bit for bit, and
against numpy.quantile to the reference's own tolerance (tests/integration/test_quantiles.py:36-111,
test_percentiles.py, test_median.py)."""
from __future__ import annotations

import numpy as np
import pytest
from conftest import assert_same_bits

import cupynumeric_amd as num
from oracle import sort_oracle as oracle

pytestmark = pytest.mark.gpu

METHODS = ("inverted_cdf", "averaged_inverted_cdf", "closest_observation", "interpolated_inverted_cdf", "hazen",
           "weibull", "linear", "median_unbiased", "normal_unbiased", "lower", "higher", "midpoint", "nearest")
REF_INPUT = np.array([1, 2, 2, 40, 1, 1, 2, 1, 0, 10, 3, 3, 40, 15, 3, 7, 5, 4, 7, 3, 5, 1, 0, 9], dtype=int).reshape(2, 3, 4)
REF_QS = (0.5, [0.001, 0.37, 0.42, 0.67, 0.83, 0.99, 0.39, 0.49, 0.5])


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("axes", (0, 1, (0,), (0, 1), (0, 2)))
def test_reference_quantile_cases(method, axes):
    # tests/integration/test_quantiles.py:36-111 (test_multi_axes), both quantile inputs, keepdims and overwrite_input
    for qs in REF_QS:
        for keepdims in (False, True):
            for overwrite in (False, True):
                got = num.quantile(num.array(REF_INPUT), qs, axis=axes, method=method, keepdims=keepdims, overwrite_input=overwrite)
                want_np = np.quantile(REF_INPUT, qs, axis=axes, method=method, keepdims=keepdims)
                assert got.shape == want_np.shape and got.dtype == want_np.dtype
                assert np.allclose(np.asarray(got), want_np, atol=1.0e-8)
                assert_same_bits(np.asarray(got), oracle.quantile(REF_INPUT, qs, axis=axes, method=method, keepdims=keepdims),
                                 f"{method} axes={axes}")


@pytest.mark.parametrize("dtype", [np.float64, np.float32, np.float16, np.int64, np.int16, np.uint8, np.bool_])
def test_quantile_all_dtypes_bit_exact_with_the_oracle(dtype):
    rng = np.random.default_rng(np.dtype(dtype).num)
    shape = (6, 50, 7)
    if np.dtype(dtype).kind == "f":
        x = (rng.standard_normal(shape) * 100).astype(dtype)
    elif np.dtype(dtype).kind == "b":
        x = rng.integers(0, 2, shape).astype(dtype)
    else:
        info = np.iinfo(dtype)
        x = rng.integers(max(info.min, -(2**40)), min(info.max, 2**40), shape, dtype=np.int64).astype(dtype)
    qs = np.array([[0.0, 0.013, 0.25], [0.5, 0.77, 1.0]])
    for method in METHODS:
        for axis in (None, 1, -1, (0, 2)):
            got = num.quantile(num.array(x), qs, axis=axis, method=method)
            want = oracle.quantile(x, qs, axis=axis, method=method)
            assert_same_bits(np.asarray(got), want, f"{np.dtype(dtype)} {method} axis={axis}")
    a = num.array(x)
    assert_same_bits(np.asarray(num.percentile(a, [5.0, 50.0, 99.5], axis=1)), oracle.percentile(x, [5.0, 50.0, 99.5], axis=1), "percentile")
    assert_same_bits(np.asarray(num.median(a, axis=0)), oracle.median(x, axis=0), "median")
    assert_same_bits(np.asarray(num.median(a)), oracle.median(x), "median of all")
    assert np.array_equal(np.asarray(a), x), "the input was modified"


def test_median_percentile_against_numpy():
    # tests/integration/test_median.py, test_percentiles.py: float64 data, every axis, keepdims
    rng = np.random.default_rng(9)
    x = rng.standard_normal((4, 9, 5))
    a = num.array(x)
    for axis in (None, 0, 1, 2, (0, 1), (1, 2)):
        for keepdims in (False, True):
            got = num.median(a, axis=axis, keepdims=keepdims)
            want = np.median(x, axis=axis, keepdims=keepdims)
            assert got.shape == want.shape and np.allclose(np.asarray(got), want, atol=1e-12)
            got = num.percentile(a, [10, 50, 90], axis=axis, keepdims=keepdims)
            want = np.percentile(x, [10, 50, 90], axis=axis, keepdims=keepdims)
            assert got.shape == want.shape and np.allclose(np.asarray(got), want, atol=1e-12)
    big = rng.standard_normal(1 << 20).astype(np.float32)
    assert np.allclose(float(np.asarray(num.median(num.array(big)))), np.median(big.astype(np.float64)), atol=1e-6)


def test_quantile_arguments():
    a = num.array(np.arange(12.0).reshape(3, 4))
    out = num.array(np.zeros(3))
    assert num.quantile(a, 0.5, axis=1, out=out) is out
    assert np.array_equal(np.asarray(out), [1.5, 5.5, 9.5])
    with pytest.raises(ValueError):
        num.quantile(a, 0.5, axis=1, out=num.array(np.zeros(4)))
    with pytest.raises(TypeError):
        num.quantile(num.array(np.array([1 + 2j, 3j])), 0.5)
    with pytest.raises(TypeError):
        num.median(None)
    b = num.array(np.array([[3.0, 1.0, 2.0]]))
    num.quantile(b, 0.5, axis=1, overwrite_input=True)
    assert np.array_equal(np.asarray(b), [[1.0, 2.0, 3.0]])  # sorted in place, as the reference does


# ---- the variants that ignore NaNs (stats_order.py:653-1080, stats_avgs_vars.py:445-512) ------------------
NAN_REF_INPUT = np.asarray([[1.0, 2, 2, 40], [1, np.nan, 2, 1], [0, 10, np.nan, np.nan], [np.nan, np.nan, 0, 10],
                            [np.nan, np.nan, np.nan, np.nan]])


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("axes", (0, 1, (0, 1), (0,), None))
def test_reference_nanquantile_cases(method, axes):
    # tests/integration/test_nanquantiles.py:41-103 (test_multi_axes) and :106-111 (test_keepdims)
    import warnings

    for qs in REF_QS:
        for keepdims in (False, True):
            got = num.nanquantile(num.array(NAN_REF_INPUT), qs, axis=axes, method=method, keepdims=keepdims)
            with warnings.catch_warnings():
                warnings.simplefilter("ignore", RuntimeWarning)
                want_np = np.nanquantile(NAN_REF_INPUT, qs, axis=axes, method=method, keepdims=keepdims)
            assert got.shape == want_np.shape and got.dtype == want_np.dtype
            assert np.allclose(np.asarray(got), want_np, atol=1.0e-8, equal_nan=True)
            assert_same_bits(np.asarray(got), oracle.nanquantile(NAN_REF_INPUT, qs, axis=axes, method=method, keepdims=keepdims),
                             f"{method} axes={axes}")


@pytest.mark.parametrize("dtype", [np.float64, np.float32, np.float16])
def test_nanquantile_bit_exact_with_the_oracle(dtype):
    """Every method, scattered NaNs, slices of NaN only, slices without any, -inf and +inf (with and
    without NaNs beside them: the reference reads the largest finite value after the last finite
    element of a slice that holds NaNs), -0.0, several axes, q as a 2-D array."""
    rng = np.random.default_rng(np.dtype(dtype).num + 100)
    shape = (5, 40, 6)
    x = (rng.standard_normal(shape) * 50).astype(dtype)
    x[rng.random(shape) < 0.25] = np.nan
    x[2, :, 3] = np.nan          # nothing left in these slices along axis 1
    x[4, :, :] = (rng.standard_normal((40, 6)) * 3).astype(dtype)  # no NaN at all
    x[0, 5, 0], x[0, 6, 0] = np.inf, -np.inf
    x[1, :3, 1] = np.inf
    x[3, 7, 2] = -0.0
    qs = np.array([[0.0, 0.013, 0.25], [0.5, 0.77, 1.0]])
    a = num.array(x)
    for method in METHODS:
        for axis in (None, 1, -1, 0, (0, 2)):
            got = num.nanquantile(a, qs, axis=axis, method=method)
            want = oracle.nanquantile(x, qs, axis=axis, method=method)
            assert_same_bits(np.asarray(got), want, f"{np.dtype(dtype)} {method} axis={axis}")
    assert_same_bits(np.asarray(num.nanpercentile(a, [5.0, 50.0, 99.5], axis=1)), oracle.nanpercentile(x, [5.0, 50.0, 99.5], axis=1),
                     "nanpercentile")
    assert_same_bits(np.asarray(num.nanmedian(a, axis=0)), oracle.nanmedian(x, axis=0), "nanmedian")
    assert_same_bits(np.asarray(num.nanmedian(a)), oracle.nanmedian(x), "nanmedian of all")
    assert_same_bits(np.asarray(a), x, "the input was modified")


def test_nanquantile_arguments():
    # tests/integration/test_nanquantiles.py:114-141
    arr = np.array([[10.0, np.nan, 4.0], [4.0, 2.0, 2]])
    out = num.array(np.zeros(2))
    assert num.nanquantile(num.array(arr), 0.5, axis=1, out=out) is out
    assert np.array_equal(np.asarray(out), np.nanquantile(arr, 0.5, axis=1))
    with pytest.raises(ValueError, match="wrong shape on output array"):
        num.nanquantile(num.array(arr), 0.5, axis=1, out=num.array(np.zeros((2, 2))))
    with pytest.raises(TypeError, match="input array cannot be of complex type"):
        num.nanquantile(num.array(np.array([1 + 2j, np.nan + 0j, 5 + 6j])), 0.5)
    with pytest.raises(ValueError):
        num.nanquantile(num.array(np.array([1, 2, 3])), 0.5)
    with pytest.raises(TypeError):
        num.nanmedian(None)
    for axes in (1, None):
        want = np.nanquantile(arr, 0.5, axis=axes, keepdims=True)
        assert np.array_equal(np.asarray(num.nanquantile(num.array(arr), 0.5, axis=axes, keepdims=True)), want)
    # a long axis: counts by binary search over 2^20 elements, a third of them NaN
    rng = np.random.default_rng(12)
    big = rng.standard_normal(1 << 20)
    big[rng.random(big.size) < 1 / 3] = np.nan
    got = np.asarray(num.nanquantile(num.array(big), [0.1, 0.5, 0.9]))
    assert np.allclose(got, np.nanquantile(big, [0.1, 0.5, 0.9]), atol=1e-12)
