"""Inputs of the reference's lexsort tests (tests/integration/test_lexsort.py), as data: each case
is (name, keys, axis).  The expected result of every case is `np.lexsort(keys, axis)`, which is
what the reference's own tests compare against."""
from __future__ import annotations

import numpy as np

DTYPES = [
    np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64,
    np.float16, np.float32, np.float64, np.complex64, np.complex128,
]
DIM = 5
SIZES = [
    (0,), (1,), (DIM,), (0, 1), (1, 0), (1, 1), (1, DIM), (DIM, 1), (DIM, DIM), (1, 0, 0), (1, 1, 0), (1, 0, 1),
    (1, 1, 1), (DIM, 1, 1), (1, DIM, 1), (1, 1, DIM), (DIM, DIM, DIM),
]


def seq(shape) -> np.ndarray:
    """Sequential integers from 1 in C order (tests/integration/utils/generators.py:51-62)."""
    size = int(np.prod(shape))
    return np.arange(1, size + 1).reshape(shape)


def cases():
    out = []
    out.append(("three_keys", (seq(100), seq(100), seq(100)), -1))  # :62-74
    for dt in DTYPES:  # :77-87
        out.append((f"dtype_{np.dtype(dt)}", (seq(100).astype(dt), seq(100).astype(dt)), -1))
    for da in [np.int32, np.uint32, np.int8, np.uint64, np.int16, np.float32, np.float64, np.complex64]:  # :90-126
        for db in [np.int64, np.int32, np.uint64, np.float32, np.float64, np.float16, np.complex64, np.complex128]:
            out.append((f"mixed_{np.dtype(da)}_{np.dtype(db)}", (seq(500).astype(da), seq(500).astype(db)), -1))
    for size in SIZES:  # :129-139
        out.append((f"size_{size}", (seq(size), seq(size)), -1))
    for mod in (10, 50, 100):  # :142-154
        out.append((f"dups_{mod}", (seq(1000) % mod, seq(1000) % (mod * 2)), -1))
    for g in (5, 20, 100):  # :157-169
        out.append((f"groups_{g}", (seq(1000) // g, (seq(1000) * 3) % (g * 2)), -1))
    out.append(("stability", (np.array([10000000] * 3 + [20000000] * 3), np.array([30000000] * 3 + [40000000] * 3)), -1))
    out.append(("all_equal", (np.array([50000000] * 4), np.array([10000000] * 4)), -1))
    out.append(("priority", (np.array([20000000, 10000000, 30000000]), np.array([10000000, 20000000, 10000000])), -1))
    out.append(("negative", (np.array([-10000000, -20000000, 0, 10000000, 20000000]),
                             np.array([50000000, -30000000, 0, -10000000, 40000000])), -1))
    for axis in (0, -1):  # :227-241
        out.append((f"axis1d_{axis}", (seq(1000), seq(1000), seq(1000)), axis))
    for axis in (0, 1, -1, -2):  # :244-259
        out.append((f"axis2d_{axis}", (seq((10, 100)), seq((10, 100)), seq((10, 100))), axis))
    out.append(("bool", (np.array([True, False, True, False]), np.array([False, True, False, True])), -1))
    nan, inf = np.nan, np.inf
    ar1 = [[nan, 1e6, 2e6, 3e6], [nan, 1e6, nan, 3e6], [inf, -inf, 1e6, 2e6], [nan, inf, -inf, 1e6]]  # :273-300
    ar2 = [[1e6, 2e6, 3e6, 4e6], [1e6, nan, 3e6, 4e6], [3e6, 4e6, inf, -inf], [inf, -inf, nan, 3e6]]
    for i, a in enumerate(ar1):
        for j, b in enumerate(ar2):
            out.append((f"special_{i}_{j}", (np.array(a), np.array(b)), -1))
    out.append(("complex", (np.array([1e6 + 2e6j, 3e6 + 4e6j, 1e6 + 2e6j, 5e6 + 6e6j]),
                            np.array([7e6 + 8e6j, 9e6 + 1e7j, 1.1e7 + 1.2e7j, 1.3e7 + 1.4e7j])), -1))
    out.append(("single_key", (seq(1000),), -1))
    out.append(("zero_d", (np.array(42),), -1))
    out.append(("zero_d_3", (np.array(42), np.array(17), np.array(99)), -1))
    out.append(("ten_keys", tuple(seq(100) for _ in range(10)), -1))
    out.append(("i64_u64", (np.array([-1, -2, 3, 4], dtype=np.int64), np.array([10, 20, 30, 40], dtype=np.uint64)), -1))
    out.append(("i8_u32", (np.array([-1, 10, -5, 5], dtype=np.int8), np.array([1000, 10, 1000, 20], dtype=np.uint32)), -1))
    out.append(("all_nan_primary", (np.array([1e6, 2e6, 3e6]), np.array([nan, nan, nan])), -1))
    out.append(("all_inf_primary", (np.array([1e6, 2e6, 3e6]), np.array([inf, inf, inf])), -1))
    out.append(("complex_real", (np.array([1 + 1j, 2 + 2j, 1 + 1j, 3 + 3j]), np.array([4, 3, 5, 2])), -1))
    out.append(("real_complex", (np.array([4, 3, 5, 2]), np.array([1 + 1j, 2 + 2j, 1 + 1j, 3 + 3j])), -1))
    out.append(("single_elem", (np.array([42], dtype=np.int32), np.array([3.14]), np.array([1 + 2j])), -1))
    out.append(("three_d", (seq((2, 3, 4)), seq((2, 3, 4)), seq((2, 3, 4))), 1))
    for n in (1, 2, 3):
        out.append((f"small_{n}", (seq(n), seq(n)), -1))
    out.append(("long", (seq(50000), seq(50000)), -1))
    for axis in (0, 1, 2, -1, -2, -3):  # :535-549
        out.append((f"axes3d_{axis}", (seq((5, 10, 15)), seq((5, 10, 15))), axis))
    out.append(("empty", (np.array([]), np.array([])), -1))
    out.append(("empty_single", (np.array([]),), -1))
    out.append(("identical", (np.array([1, 1, 1, 1]), np.array([2, 2, 2, 2]), np.array([3, 3, 3, 3])), -1))
    out.append(("neg_inf", (np.array([1, 2, 3, 4]), np.array([-inf, -inf, 1, 2])), -1))
    out.append(("inf_nan", (np.array([1, 2, 3, 4, 5]), np.array([inf, -inf, nan, 1, 2])), -1))
    out.append(("complex_nan", (np.array([1 + 1j, 2 + 2j, complex(nan, 1), 4 + 4j]), np.array([1, 2, 3, 4])), -1))
    out.append(("tiny_values", (np.array([1e-10, 1e-20, 1e-30, 1e-40]), np.array([1, 2, 3, 4])), -1))
    out.append(("huge_values", (np.array([1e10, 1e20, 1e30, 1e40]), np.array([1, 2, 3, 4])), -1))
    # a single ndarray: its first axis runs over the keys (:637-679)
    out.append(("nd_1d", np.array([3, 1, 2]), -1))
    out.append(("nd_2d", np.array([[3, 1, 2], [1, 2, 3]]), -1))
    out.append(("nd_2d_b", np.array([[3, 1, 2, 4], [1, 2, 3, 1], [2, 1, 1, 3]]), -1))
    out.append(("nd_3d", np.array([[[1, 2], [3, 4]], [[5, 6], [7, 8]]]), -1))
    out.append(("nd_2d_axis0", np.array([[3, 1, 2], [1, 2, 3]]), 0))
    for dt in (np.int32, np.float64, np.complex128):
        out.append((f"nd_{np.dtype(dt)}", seq((3, 4)).astype(dt), -1))
    return out


def random_cases():
    """Beyond the reference's cases: random keys with many ties, special values, several rows."""
    rng = np.random.default_rng(77)
    out = []
    for shape, axis in [((3000,), -1), ((40, 700), -1), ((40, 700), 0), ((6, 50, 9), 1), ((20000,), 0)]:
        k1 = rng.integers(0, 4, shape).astype(np.int8)
        k2 = np.round(rng.standard_normal(shape) * 2).astype(np.float32)
        k2[rng.random(shape) < 0.05] = np.nan
        k2[rng.random(shape) < 0.05] = -0.0
        k3 = rng.integers(0, 3, shape).astype(np.uint64)
        k4 = (rng.integers(0, 2, shape) + 1j * rng.integers(0, 2, shape)).astype(np.complex64)
        out.append((f"random_{shape}_{axis}", (k1, k2, k3, k4), axis))
        out.append((f"random2_{shape}_{axis}", (k2, k1), axis))
    return out
