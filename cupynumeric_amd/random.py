"""Host-side random inputs wrapped as device arrays: the `cupynumeric.random` calls that the
reference's sort tests and its sort example make (`tests/integration/test_sort.py`:
`num.random.randint`; `examples/sort.py:52-71`: `seed`, `randint`, `random`)."""
from __future__ import annotations

from typing import Any

import numpy as np


def seed(value: int | None = None) -> None:
    np.random.seed(value)


def randint(low: int, high: int | None = None, size: Any = None, dtype: Any = int):
    from . import array

    return array(np.random.randint(low, high, size=size, dtype=dtype))


def random(size: Any = None):
    from . import array

    return array(np.random.random(size))
