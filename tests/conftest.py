"""Test configuration.  Tests marked `gpu` need an MI355X and the built libcpnsort.so; all the
others run on a CPU-only machine (oracle, host logic, ABI symbol checks)."""
from __future__ import annotations

import json
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X) and the built libcpnsort.so")


@pytest.fixture(scope="session")
def reference_vectors():
    """Golden vectors transcribed from the reference's tests/cpp/integration/test_sort.cc and
    test_argsort.cc (see tests/golden/extract_reference_vectors.py)."""
    return json.loads((ROOT / "tests" / "golden" / "reference_vectors.json").read_text())["cases"]


def bits(a: np.ndarray) -> np.ndarray:
    """Unsigned-integer view of an array, so that NaN payloads and zero signs are compared."""
    a = np.ascontiguousarray(a)
    if a.dtype.itemsize == 16:  # complex128: two words per element
        return a.reshape(-1).view(np.uint64)
    return a.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize])


def assert_same_bits(got: np.ndarray, want: np.ndarray, what: str = "") -> None:
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    assert got.dtype == want.dtype, f"{what}: dtype {got.dtype} != {want.dtype}"
    if got.size == 0:
        return
    if not np.array_equal(bits(got), bits(want)):
        bad = np.flatnonzero(bits(got).reshape(-1) != bits(want).reshape(-1)) // (2 if got.dtype.itemsize == 16 else 1)
        raise AssertionError(
            f"{what}: {bad.size} of {got.size} elements differ, first at flat index {bad[0]}: "
            f"got {got.reshape(-1)[bad[0]]!r}, want {want.reshape(-1)[bad[0]]!r}"
        )


def case_array(values, dtype, shape=None) -> np.ndarray:
    """Array of a golden-vector case; complex values are stored as [real, imag] pairs."""
    dt = np.dtype(dtype)
    if dt.kind == "c" :
        pairs = np.array(values, dtype=np.float64).reshape(-1, 2)
        out = np.empty(len(pairs), dtype=dt)
        out.real = pairs[:, 0]
        out.imag = pairs[:, 1]
    else:
        out = np.array(values, dtype=dt)
    return out if shape is None else out.reshape(shape)


COMPLEX_DTYPES = [np.complex64, np.complex128]

ALL_REAL_DTYPES = [
    np.bool_, np.int8, np.int16, np.int32, np.int64,
    np.uint8, np.uint16, np.uint32, np.uint64,
    np.float16, np.float32, np.float64,
]


def make_input(dtype, shape, seed: int, special: bool = True, duplicates: bool = True) -> np.ndarray:
    """Seeded test input.  Floats: normal values with NaN (both signs, payloads), +-0, +-inf and
    subnormals mixed in; integers: full range with a block of duplicates."""
    rng = np.random.default_rng(seed)
    dt = np.dtype(dtype)
    n = int(np.prod(shape, dtype=np.int64))
    if dt.kind == "c":
        # few distinct real parts so that the imaginary part decides often; specials in both parts
        part = np.float32 if dt == np.complex64 else np.float64
        re = make_input(part, (n,), seed * 2 + 1, special)
        im = make_input(part, (n,), seed * 2 + 2, special)
        if n:
            re = np.where(rng.random(n) < 0.6, np.round(re * 2) / 2, re).astype(part)
        x = np.empty(n, dtype=dt)
        x.real = re
        x.imag = im
        return x.reshape(shape)
    if dt.kind == "f":
        x = rng.standard_normal(n).astype(dt)
        if special and n:
            u = rng.random(n)
            ub = {2: np.uint16, 4: np.uint32, 8: np.uint64}[dt.itemsize]
            xb = x.view(ub)
            nan_pos = np.array(np.nan, dtype=dt).view(ub)
            sign = ub(1) << ub(dt.itemsize * 8 - 1)
            m = u < 0.03
            xb[m] = nan_pos | (rng.integers(0, 8, int(m.sum())).astype(ub))  # payload bits
            m = (u >= 0.03) & (u < 0.05)
            xb[m] = nan_pos | sign  # negative NaN
            x[(u >= 0.05) & (u < 0.08)] = 0.0
            x[(u >= 0.08) & (u < 0.11)] = -0.0
            x[(u >= 0.11) & (u < 0.12)] = np.inf
            x[(u >= 0.12) & (u < 0.13)] = -np.inf
            m = (u >= 0.13) & (u < 0.15)
            xb[m] = rng.integers(1, 4, int(m.sum())).astype(ub)  # positive subnormals
            m = (u >= 0.15) & (u < 0.17)
            xb[m] = sign | rng.integers(1, 4, int(m.sum())).astype(ub)  # negative subnormals
    elif dt.kind == "b":
        x = rng.integers(0, 2, n).astype(dt)
    else:
        info = np.iinfo(dt)
        x = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
        if duplicates and n > 8:
            x[rng.integers(0, n, n // 3)] = x[0]
            x[rng.integers(0, n, max(n // 50, 1))] = info.min
            x[rng.integers(0, n, max(n // 50, 1))] = info.max
    return x.reshape(shape)


# tests/cpp/integration/test_unique.cc:34-68: (input, shape, expected distinct values)
UNIQUE_GOLDEN = [
    ([1, 1, 2, 2, 3, 3], (6,), [1, 2, 3], np.int32),
    ([1, 1, 2, 3], (2, 2), [1, 2, 3], np.int32),
    ([1, 2, 1, 1, 3, 3, 3, 4, 5, 4], (10,), [1, 2, 3, 4, 5], np.int32),
    ([99], (1,), [99], np.int64),
]
