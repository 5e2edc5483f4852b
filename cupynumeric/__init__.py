"""`import cupynumeric` for the sort path on MI355X.

The reference's users write `import cupynumeric as np` (`examples/sort.py`, `tests/integration/test_sort.py`);
this package gives that name to `cupynumeric_amd`, which holds the implementation: `sort`, `argsort`,
`ndarray.sort`, `ndarray.argsort` and the callers and consumers next to them.  Everything else
of cuPyNumeric is out of scope and absent.
"""
import sys as _sys

import cupynumeric_amd as _impl
from cupynumeric_amd import *  # noqa: F401,F403
from cupynumeric_amd import __all__, __version__, random  # noqa: F401

# `import cupynumeric.random` and `from cupynumeric import random` name the same module
_sys.modules[__name__ + ".random"] = _impl.random
