"""Host-side random inputs wrapped as device arrays: the one `cupynumeric.random` call the
reference's sort tests use (`tests/integration/test_sort.py`, `num.random.randint`)."""
from __future__ import annotations

from typing import Any

import numpy as np


def seed(value: int | None = None) -> None:
    np.random.seed(value)


def randint(low: int, high: int | None = None, size: Any = None, dtype: Any = int):
    from . import array

    return array(np.random.randint(low, high, size=size, dtype=dtype))
