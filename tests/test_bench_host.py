"""Host-side checks of bench.py that need no GPU: the byte accounting behind the roofline figures, the
shrunken workloads, and the refusal of more than one GPU."""
from __future__ import annotations

import subprocess
import sys

import numpy as np
from conftest import ROOT

sys.path.insert(0, str(ROOT))
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused():
    res = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


def test_algorithmic_bytes_of_the_headline_workload():
    cfg = bench.make_config("c2", log2n=16)
    n = cfg["x"].size
    alg = bench.algorithmic_bytes(cfg, lds_limit_rows=False)
    # fp32 keys, 4-byte row positions between passes, int64 on the last write
    assert alg["onesweep_per_pass"] == [n * 12, n * 16, n * 16, n * 16]
    assert alg["onesweep"] == n * 15 and alg["histogram"] == n * 4
    total = alg["histogram"] + sum(alg["onesweep_per_pass"])
    assert total == n * 64
    # the baseline's own accounting (8-byte payload in every pass): N*88 for this workload
    assert alg["whole_baseline_formula"] == n * 88 and alg["onesweep_baseline_formula"] == n * 21
    # keys-only int32 sort: every pass reads and writes the key
    alg1 = bench.algorithmic_bytes(bench.make_config("c1", log2n=16), lds_limit_rows=False)
    assert alg1["onesweep_per_pass"] == [(1 << 16) * 8] * 4


def test_row_and_transpose_workloads():
    c3 = bench.make_config("c3", rows=4)
    assert c3["x"].shape == (4, 1024) and c3["x"].dtype == np.float64
    assert bench.algorithmic_bytes(c3, lds_limit_rows=True)["lds_row_sort"] == 4 * 1024 * 16
    c5 = bench.make_config("c5", rows=64)
    alg = bench.algorithmic_bytes(c5, lds_limit_rows=True)
    assert c5["axis"] == 0 and alg["transpose_last"] == 64 * 64 * 4 and alg["lds_row_sort"] == 64 * 64 * 4


def test_workloads_are_seeded():
    a = bench.make_config("c2", log2n=12)["x"]
    b = bench.make_config("c2", log2n=12)["x"]
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.isnan(a).any() and (a == 0).any()
    c4 = bench.make_config("c4", log2n=12)["x"]
    assert np.unique(c4).size <= 16
