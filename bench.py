#!/usr/bin/env python3
"""Benchmark of the sort hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--log2n L] [--no-cpu-baseline]

A step is one pass of the hot path (one `cpn_local_sort` call, plus the two transposes for the
axis-0 config) over one batch of synthetic input that already sits in HBM.  The default
workload is the one the headline metric is quoted on: stable argsort of 2^28 float32 keys with
1 % NaN and 1 % signed zeros (seed 1), int64 indices out.  One JSON line is printed.

Timing follows the reference's microbenchmark loop (`examples/_benchmark/timer.py:199-241`,
`examples/microbenchmarks/sort_bench.py:104-130`): warm-up calls, then K calls between two
device synchronisations.  The `roofline` object is for the dominant kernel (the onesweep scatter
pass, or the per-row LDS sort): algorithmic bytes per launch divided by its average launch
duration, measured with HIP events that the library records on its own stream.  The
`cpu_baseline` object times the CPU restatement of the reference's CPU/OpenMP variant
(oracle/sort_oracle.c) on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_BYTES_PER_S = 8.0e12  # MI355X HBM3E

def measured_traffic_bytes(config: str, kernel: str) -> float | None:
    """HBM bytes per launch of `kernel` on workload `config`, as measured with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE and scaled by a plain copy of known size: read from the summary line
    of profiles/<kernel>_<config>_traffic.txt ("<kernel>: X GB of HBM traffic per launch"), so the
    figure changes with the committed profile and is null where none exists."""
    import re

    path = ROOT / "profiles" / f"{kernel}_{config}_traffic.txt"
    if not path.exists():
        return None
    m = re.search(rf"^{re.escape(kernel)}: ([0-9.]+) GB of HBM traffic per launch", path.read_text(), flags=re.M)
    return float(m.group(1)) * 1e9 if m else None


# -------------------------------------------------------------------------------------------------
# workloads (the five configurations of the baseline; `log2n` / `rows` shrink them for tests)
# -------------------------------------------------------------------------------------------------
def make_config(name: str, log2n: int | None = None, rows: int | None = None) -> dict:
    """Seeded synthetic input of one workload as a host array plus what to do with it."""
    if name == "c1":
        n = 1 << (24 if log2n is None else log2n)
        rng = np.random.default_rng(0)
        x = rng.integers(-(2**31), 2**31, size=n, dtype=np.int64).astype(np.int32)
        return dict(name=name, x=x, op="sort", axis=-1,
                    workload=f"c1: np.sort int32 1-D N=2^{int(np.log2(n))}, uniform over int32, seed 0")
    if name == "c2":
        n = 1 << (28 if log2n is None else log2n)
        rng = np.random.default_rng(1)
        x = rng.standard_normal(n, dtype=np.float32)
        u = rng.random(n)
        x[u < 0.01] = np.nan
        m = (u >= 0.01) & (u < 0.02)
        x[m] = np.where(rng.random(int(m.sum())) < 0.5, np.float32(-0.0), np.float32(0.0))
        return dict(name=name, x=x, op="argsort", axis=-1,
                    workload=f"c2: stable argsort float32 1-D N=2^{int(np.log2(n))}, normal + 1% NaN + 1% +-0, "
                             "seed 1, int64 indices out")
    if name == "c3":
        r = 65536 if rows is None else rows
        rng = np.random.default_rng(2)
        x = rng.random((r, 1024))
        return dict(name=name, x=x, op="sort", axis=-1,
                    workload=f"c3: np.sort float64 ({r},1024) last axis, uniform [0,1), seed 2")
    if name == "c4":
        n = 1 << (27 if log2n is None else log2n)
        rng = np.random.default_rng(3)
        vals = rng.integers(-(2**63), 2**63 - 1, size=16, dtype=np.int64)
        x = vals[rng.integers(0, 16, size=n)]
        return dict(name=name, x=x, op="argsort", axis=-1,
                    workload=f"c4: stable argsort int64 1-D N=2^{int(np.log2(n))}, 16 distinct keys, seed 3, "
                             "int64 indices out")
    if name == "c5":
        r = 8192 if rows is None else rows
        rng = np.random.default_rng(4)
        x = rng.standard_normal((r, r)).astype(np.float16)
        return dict(name=name, x=x, op="sort", axis=0,
                    workload=f"c5: np.sort float16 ({r},{r}) axis 0, normal, seed 4")
    if name in ("flat", "skinny"):
        # examples/microbenchmarks/sort_bench.py:54-68 at size s: ceil(s^1/4) x ceil(s^3/4) ("2D-flat") and
        # its transpose ("2D-skinny"), float32 from rng.random (examples/_benchmark/random_array.py:43-49)
        import math

        s_total = 1 << (28 if log2n is None else log2n)
        a, b = math.ceil(math.pow(s_total, 1 / 4)), math.ceil(math.pow(s_total, 3 / 4))
        shape = (a, b) if name == "flat" else (b, a)
        rng = np.random.default_rng(8 if name == "flat" else 9)
        x = rng.random(size=shape, dtype=np.float32)
        return dict(name=name, x=x, op="sort", axis=-1,
                    workload=f"sort-2D-{name}: np.sort float32 {shape} last axis, uniform [0,1), seed "
                             f"{8 if name == 'flat' else 9} (the reference's sort_bench.py shape at s=2^{int(math.log2(s_total))})")
    if name.startswith("rows:"):
        # rows:<dtype>:<rows>:<row length>:<sort|argsort> -- batched rows of any length, e.g. on either
        # side of the row length at which the library changes kernels
        _, dt, r, seg, op = name.split(":")
        r, seg, dtype = int(r), int(seg), np.dtype(dt)
        rng = np.random.default_rng(10)
        if dtype == np.float64:
            x = rng.random((r, seg))
        elif dtype.kind == "f":
            x = rng.standard_normal((r, seg), dtype=np.float32).astype(dtype)
        else:
            info = np.iinfo(dtype)
            x = rng.integers(info.min, info.max, size=(r, seg), dtype=dtype, endpoint=True)
        if op not in ("sort", "argsort"):
            raise ValueError(f"rows config: op must be sort or argsort, not {op}")
        return dict(name=name, x=x, op=op, axis=-1,
                    workload=f"np.{op} {dtype.name} ({r},{seg}) last axis, "
                             f"{'uniform [0,1)' if dtype == np.float64 else 'normal' if dtype.kind == 'f' else 'uniform'}, seed 10")
    raise ValueError(f"unknown config {name}")


# Row lengths on either side of every length at which the library changes kernels (--edges): key type,
# operation, lengths whose successor is timed too; 2^26 keys per run.
EDGE_LENGTHS = (
    ("float32", "sort", (32, 40, 64, 96, 128, 256, 512, 768, 1024, 1536, 2048, 3072, 4096, 6144, 8192, 12288, 16384, 32768, 65536)),
    ("float64", "sort", (32, 40, 64, 96, 128, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096, 6144, 8192, 16384, 32768, 65536, 1048576)),
    ("float16", "sort", (32, 40, 64, 96, 128, 256, 512, 768, 4096, 8192, 16384, 32768, 57344)),
    ("float32", "argsort", (32, 40, 64, 96, 128, 256, 512, 1024, 2048, 4096, 6144, 8192, 16384, 32768, 65536)),
    ("float64", "argsort", (32, 40, 64, 96, 128, 256, 512, 2048, 4096, 6144, 8192, 14336, 28672, 57344, 458752)),
)


def run_edges() -> dict:
    """Times batched rows of length n and n + 1 for every n of EDGE_LENGTHS (fastest and median of 7
    single steps through the C ABI, launch timing off) and says which kernel path each took."""
    import torch

    table = []
    for dt, op, lengths in EDGE_LENGTHS:
        for n in lengths:
            rows = (1 << 26) // n
            pair = []
            for seg in (n, n + 1):
                f, _, job = run_sort_workload(f"rows:{dt}:{rows}:{seg}:{op}", steps=7, warmup=2, profile_steps=1)
                pair.append({"row_length": seg, "ms_min": round(f["ms_per_step_min"], 4),
                             "ms_median": round(f["ms_per_step_median"], 4),
                             "ps_per_key": round(f["ms_per_step_min"] * 1e9 / (rows * seg), 2),
                             "path": f["config"]["path"], "verify": f["verify"]})
                del job
                torch.cuda.empty_cache()
            table.append({"dtype": dt, "op": op, "rows": rows, "below": pair[0], "above": pair[1],
                          "step": round(pair[1]["ms_min"] / pair[0]["ms_min"], 2)})
    return {"metric": "row-length edges of the per-row kernels, ms per sort of rows x row_length keys",
            "unit": "ms", "n_gpus": 1, "data": "synthetic", "edges": table}


def run_edges_compact() -> dict:
    """The same row lengths as --edges on input generated on the device (normal float32 / float16, uniform
    float64), fastest of 7 single steps through the C ABI, every result checked against torch's stable sort;
    reports, per key type and operation, the largest step between a row length and its successor and every
    step above 1.5."""
    import torch

    out = {}
    ok = True
    for dt, op, lengths in EDGE_LENGTHS:
        kb = np.dtype(dt).itemsize
        data = device_random(torch, (1 << 26) + (1 << 21), dt, seed=10, law="uniform" if dt == "float64" else "normal")
        steps = []
        for n in lengths:
            rows = (1 << 26) // n
            ms = []
            for seg in (n, n + 1):
                job = GpuJob(dict(x_dev=data[: rows * seg * kb], shape=(rows, seg), dtype=dt, op=op, axis=-1))
                for _ in range(2):
                    job.step()
                best = float("inf")
                for _ in range(7):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    job.step()
                    e1.record()
                    torch.cuda.synchronize()
                    best = min(best, e0.elapsed_time(e1))
                job.check_status()
                got = job.d_idx.view(torch.uint8) if op == "argsort" else job.d_val
                ok = ok and verify_against_torch(torch, got, job.d_in, (rows, seg), dt, op, -1) == "ok"
                ms.append(best)
                del job, got
                torch.cuda.empty_cache()
            steps.append({"row_length": n, "ms_below": round(ms[0], 4), "ms_above": round(ms[1], 4),
                          "step": round((ms[1] / (rows * (n + 1))) / (ms[0] / (rows * n)), 2)})
        worst = max(steps, key=lambda e: e["step"])
        out[f"{dt} {op}"] = {"worst": worst, "above_1.5": [e for e in steps if e["step"] > 1.5 and e is not worst],
                             "edges_timed": len(steps)}
        del data
        torch.cuda.empty_cache()
    out["verify"] = "ok" if ok else "FAILED"
    out["what"] = ("rows of n and n + 1 keys for every n at which the library changes kernels, 2^26 keys per sort; "
                   "step = time per key above / time per key below")
    return out


def algorithmic_bytes(cfg: dict, lds_limit_rows: bool, passes_run: int | None = None) -> dict:
    """Bytes the algorithm has to move, per kernel kind.  `kb` key bytes, `ib` = 4-byte row
    positions between passes (rows shorter than 2^30) and 8-byte int64 on the final write.
    `passes_run`: how many scatter passes actually ran (passes on a digit that is the same for every key
    are skipped, and keys whose bytes take few values share passes: virtual digits); default one per
    key byte."""
    x = cfg["x"]
    n = x.size
    kb = x.dtype.itemsize
    argsort = cfg["op"] == "argsort"
    out = {"n": n, "kb": kb}
    if lds_limit_rows:
        # one read of the keys, one write of values or of int64 indices
        out["lds_row_sort"] = n * (kb + (8 if argsort else kb))
    else:
        passes = kb if passes_run is None else max(1, passes_run)
        per_pass = []
        for p in range(passes):
            first, last = p == 0, p == passes - 1
            r = kb + (0 if (first or not argsort) else 4)
            if argsort:
                w = (0 if last else kb) + (8 if last else 4)
            else:
                w = kb
            per_pass.append(n * (r + w))
        out["onesweep_per_pass"] = per_pass
        out["onesweep"] = sum(per_pass) / passes  # average launch
        out["histogram"] = n * kb
        out["virtual_histogram"] = n * kb
        out["distinct_sweep"] = n * kb
        # the same passes counted with the baseline's formula, which carries the payload at its final
        # width (vb = 8) through every pass: r_1 = kb, r_p = w_p = kb + vb, w_P = vb for index-only output
        vb = 8 if argsort else 0
        formula = []
        for p in range(kb):  # the formula always runs one pass per key byte
            first, last = p == 0, p == kb - 1
            r = kb if first else kb + vb
            w = vb if (last and argsort) else kb + vb
            formula.append(n * (r + w))
        out["onesweep_baseline_formula"] = sum(formula) / kb
        out["whole_baseline_formula"] = n * kb + sum(formula)
    if cfg["axis"] == 0:
        out["transpose_last"] = n * 2 * kb
    return out


# -------------------------------------------------------------------------------------------------
# GPU side
# -------------------------------------------------------------------------------------------------
def measure_device_rates(torch) -> dict:
    """Streaming rates of the device on 1 GiB buffers, outside the timed region: a device-to-device
    copy (bytes read + written), a read-only sweep and a write-only fill, each once with the
    library's own probe kernels (cpn_stream_probe: 128-bit nontemporal accesses, many short
    workgroups) and once with torch's copy_/sum/zero_.  Reported beside the roofline so that the
    fraction of the published HBM peak can be read against what plain passes reach on the same box."""
    n = 1 << 28
    src = torch.empty(n, dtype=torch.float32, device="cuda:0").normal_()
    dst = torch.empty_like(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best_ms(fn, reps=5, inner=5):
        fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(reps):
            e0.record()
            for _ in range(inner):
                fn()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) / inner)
        return best

    nbytes = 4 * n
    from cupynumeric_amd import _lib

    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def probe(mode):
        rc = lib.cpn_stream_probe(mode, src.data_ptr(), dst.data_ptr(), nbytes, stream)
        if rc != 0:
            raise RuntimeError(f"cpn_stream_probe: {_lib.status_string(rc)}")

    rates = {
        "copy_GBps": 2 * nbytes / best_ms(lambda: probe(1)) / 1e6,
        "read_GBps": nbytes / best_ms(lambda: probe(0)) / 1e6,
        "fill_GBps": nbytes / best_ms(lambda: probe(2)) / 1e6,
        "torch_copy_GBps": 2 * nbytes / best_ms(lambda: dst.copy_(src)) / 1e6,
        "torch_sum_GBps": nbytes / best_ms(lambda: src.sum()) / 1e6,
        "torch_zero_GBps": nbytes / best_ms(lambda: dst.zero_()) / 1e6,
        "buffer_bytes": nbytes,
    }
    del src, dst
    return rates


class GpuJob:
    """Device buffers and the call sequence of one workload, through the C ABI: a sort or argsort
    along any axis of a dense array (other axes than the last: transposed copy, last-axis sort,
    transposed copy back, as `sort_swapped` does).  `cfg["x"]` is the host input, or `cfg["x_dev"]`
    a device byte tensor that already holds it (then `cfg["shape"]` and `cfg["dtype"]` describe it)."""

    def __init__(self, cfg: dict):
        import torch

        from cupynumeric_amd import _lib

        self.torch = torch
        self.lib = _lib.load()
        self._lib_mod = _lib
        if not torch.cuda.is_available():
            raise RuntimeError("bench.py needs a HIP device")
        dev = torch.device("cuda:0")
        self.cfg = cfg
        if cfg.get("x_dev") is not None:
            self.d_in = cfg["x_dev"]
            self.shape = tuple(cfg["shape"])
            self.np_dtype = np.dtype(cfg["dtype"])
        else:
            x = cfg["x"]
            self.shape = x.shape
            self.np_dtype = x.dtype
            self.d_in = torch.from_numpy(x.reshape(-1).view(np.uint8)).to(dev)
        self.code = _lib.DTYPE_CODES[self.np_dtype]
        self.kb = self.np_dtype.itemsize
        self.argsort = cfg["op"] == "argsort"
        ndim = len(self.shape)
        self.axis = cfg["axis"] % ndim
        self.transposed = self.axis != ndim - 1
        self.volume = int(np.prod(self.shape, dtype=np.int64))
        self.seg = self.shape[self.axis]
        self.d_val = None if self.argsort else torch.empty_like(self.d_in)
        self.d_idx = torch.empty(self.volume, dtype=torch.int64, device=dev) if self.argsort else None
        self.d_tr = torch.empty_like(self.d_in) if self.transposed else None
        self.d_idx_tr = torch.empty_like(self.d_idx) if (self.transposed and self.argsort) else None
        in_place = self.transposed and not self.argsort  # the transposed copy is sorted in place, as sort_swapped does
        self.temp_bytes = self.lib.cpn_local_sort_temp_bytes(
            self.code, self.volume, self.seg, int(not self.argsort), int(self.argsort), int(in_place)
        )
        self.temp = torch.empty(self.temp_bytes, dtype=torch.uint8, device=dev)
        self.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        # rows that fit the per-row LDS kernel need nothing but the workspace header
        self.uses_lds_rows = self.temp_bytes == self.lib.cpn_local_sort_temp_bytes(self.code, 0, 0, 1, 0, 0)
        if self.transposed:
            moved = list(self.shape)
            moved[self.axis], moved[-1] = moved[-1], moved[self.axis]
            self.c_shape = (ctypes.c_int64 * ndim)(*self.shape)
            self.c_shape_moved = (ctypes.c_int64 * ndim)(*moved)

    def step(self) -> None:
        lib, ck = self.lib, self._lib_mod.check
        if self.transposed:
            ndim, last = len(self.shape), len(self.shape) - 1
            ck(lib.cpn_swapaxes_copy(self.kb, self.d_in.data_ptr(), self.d_tr.data_ptr(), self.c_shape, ndim, self.axis,
                                     last, self.stream), "cpn_swapaxes_copy")
            if self.argsort:
                ck(lib.cpn_local_sort(self.code, self.d_tr.data_ptr(), None, self.d_idx_tr.data_ptr(), self.volume,
                                      self.seg, 0, 1, self.temp.data_ptr(), self.temp_bytes, self.stream), "cpn_local_sort")
                ck(lib.cpn_swapaxes_copy(8, self.d_idx_tr.data_ptr(), self.d_idx.data_ptr(), self.c_shape_moved, ndim,
                                         self.axis, last, self.stream), "cpn_swapaxes_copy")
            else:
                ck(lib.cpn_local_sort(self.code, self.d_tr.data_ptr(), self.d_tr.data_ptr(), None, self.volume, self.seg,
                                      0, 1, self.temp.data_ptr(), self.temp_bytes, self.stream), "cpn_local_sort")
                ck(lib.cpn_swapaxes_copy(self.kb, self.d_tr.data_ptr(), self.d_val.data_ptr(), self.c_shape_moved, ndim,
                                         self.axis, last, self.stream), "cpn_swapaxes_copy")
        else:
            ck(lib.cpn_local_sort(
                self.code, self.d_in.data_ptr(), None if self.argsort else self.d_val.data_ptr(),
                self.d_idx.data_ptr() if self.argsort else None, self.volume, self.seg, 0, 1,
                self.temp.data_ptr(), self.temp_bytes, self.stream), "cpn_local_sort")

    def check_status(self) -> None:
        self._lib_mod.check(self.lib.cpn_local_sort_check(self.temp.data_ptr(), self.stream), "cpn_local_sort")

    def result(self) -> np.ndarray:
        if self.argsort:
            return self.d_idx.cpu().numpy().reshape(self.shape)
        return self.d_val.cpu().numpy().view(self.np_dtype).reshape(self.shape)


def verify_sample(job: GpuJob, cfg: dict) -> str:
    """Cheap end-of-run sanity check on the device result (full parity lives in tests/)."""
    torch = job.torch
    if cfg["op"] == "argsort" and cfg["x"].ndim == 1:
        idx = job.d_idx
        keys = job.d_in.view(torch.float32 if cfg["x"].dtype == np.float32 else torch.int64)[idx]
        a, b = keys[:-1], keys[1:]
        if keys.dtype.is_floating_point:
            ordered = bool(((a <= b) | torch.isnan(b)).all())
            tie = (a == b) | (torch.isnan(a) & torch.isnan(b))
        else:
            ordered = bool((a <= b).all())
            tie = a == b
        stable = bool((idx[1:][tie] > idx[:-1][tie]).all())
        seen = torch.zeros(idx.numel(), dtype=torch.bool, device=idx.device)
        seen[idx] = True
        perm = bool(seen.all())
        return "ok" if (ordered and stable and perm) else f"FAILED ordered={ordered} stable={stable} permutation={perm}"
    tdt = {np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64, np.dtype(np.int32): torch.int32,
           np.dtype(np.int64): torch.int64}.get(cfg["x"].dtype)
    if cfg["op"] == "argsort" and cfg["x"].ndim == 2 and tdt is not None and not np.isnan(cfg["x"][:1]).any():
        # batched rows without NaN: the stable argsort is unique, torch's stable sort must give the same indices
        x = job.d_in.view(tdt).view(job.shape)
        ref = torch.sort(x, dim=-1, stable=True).indices
        same = job.d_idx.view(job.shape) == ref
        return "ok" if bool(same.all()) else f"FAILED: {int((~same).sum())} indices differ from torch.sort(stable=True)"
    return "not checked here"


# -------------------------------------------------------------------------------------------------
# CPU baseline: restatement of the reference's CPU / OpenMP variant on a bounded sample
# -------------------------------------------------------------------------------------------------
# The CPU variants and how much of the workload each sorts, so that the whole baseline stays within
# about half a minute: the fast ones take the whole workload, the one-core comparison sorts a prefix.
CPU_FULL_KEYS = 1 << 28
CPU_ONE_CORE_MERGE_KEYS = 1 << 25


def cpu_baseline(cfg: dict) -> dict:
    from oracle import sort_oracle as oracle

    x = cfg["x"]
    argsort = cfg["op"] == "argsort"

    def take(limit: int):
        """(sample, description): at most `limit` keys of the workload, whole rows."""
        if x.ndim == 1:
            part = x[: min(x.size, limit)]
            return part, ("the whole workload" if part.size == x.size else f"first 2^{int(np.log2(part.size))} keys")
        if cfg["axis"] == 0:
            cols = min(x.shape[1], max(1, limit // x.shape[0]))
            return np.ascontiguousarray(x[:, :cols].T), f"{cols} columns (transposes not timed)"
        r = min(x.shape[0], max(1, limit // x.shape[1]))
        return x[:r], ("the whole workload" if r == x.shape[0] else f"first {r} rows")

    threads = min(oracle.max_threads(), os.cpu_count() or 1, 16)
    variants = {}

    def timed(label, cores, limit, algorithm, fn):
        sample, what = take(limit)
        t0 = time.perf_counter()
        fn(sample)
        dt = time.perf_counter() - t0
        variants[label] = {"keys_per_s": sample.size / dt, "cores": cores, "seconds": round(dt, 2),
                           "sample": what, "algorithm": algorithm}

    # the C restatement of the reference's CPU / OpenMP variant (oracle/sort_oracle.c): serial loop over
    # the rows, a stable merge sort per row under NumPy's comparison, OpenMP inside a row
    timed("oracle_c_1", 1, CPU_ONE_CORE_MERGE_KEYS, "stable merge sort, NumPy order",
          lambda a: oracle.local_sort(a, argsort=argsort, stable=True, threads=1))
    if threads > 1:
        timed(f"oracle_c_{threads}", threads, CPU_FULL_KEYS, "stable merge sort, NumPy order, OpenMP inside a row",
              lambda a: oracle.local_sort(a, argsort=argsort, stable=True, threads=threads))
    # the reference's own per-row thrust calls (oracle/thrust_baseline.cpp) over rocThrust's host backends:
    # policy thrust::host = its CPU variant, thrust::omp::par = its OpenMP variant; comparator typed
    # (thrust::less<VAL>: rocThrust runs a radix sort) or transparent as the reference writes it
    # (`::cuda::std::less{}`, sort_cpu.inl:62-83: rocThrust runs a merge sort).  Output order differs
    # from NumPy's on NaN / -0.0 in every one of them; only the time is used.
    if x.dtype != np.float16:
        timed("thrust_host_less_typed_1", 1, CPU_FULL_KEYS, "thrust::host, thrust::less<VAL>: rocThrust host radix sort",
              lambda a: oracle.thrust_local_sort(a, argsort, stable=True, use_omp=False, transparent=False))
        timed("thrust_host_less_transparent_1", 1, CPU_ONE_CORE_MERGE_KEYS,
              "thrust::host, thrust::less<>: rocThrust host merge sort",
              lambda a: oracle.thrust_local_sort(a, argsort, stable=True, use_omp=False, transparent=True))
        if threads > 1:
            timed(f"thrust_omp_less_typed_{threads}", threads, CPU_FULL_KEYS,
                  "thrust::omp::par, thrust::less<VAL>: rocThrust OpenMP sort",
                  lambda a: oracle.thrust_local_sort(a, argsort, stable=True, use_omp=True, transparent=False))
            timed(f"thrust_omp_less_transparent_{threads}", threads, CPU_FULL_KEYS,
                  "thrust::omp::par, thrust::less<>: rocThrust OpenMP merge sort",
                  lambda a: oracle.thrust_local_sort(a, argsort, stable=True, use_omp=True, transparent=True))
    best = max(variants, key=lambda k: variants[k]["keys_per_s"])
    b = variants[best]
    return {
        "value": b["keys_per_s"],
        "unit": "keys/s",
        "cores": b["cores"],
        "kind": "port",
        "sample": f"fastest of the CPU variants timed: {best} ({b['algorithm']}) on {b['sample']}, {b['seconds']} s.  "
                  "oracle_c = oracle/sort_oracle.c; thrust_* = oracle/thrust_baseline.cpp, the reference's per-row "
                  "thrust::stable_sort[_by_key] calls over rocThrust (not the CCCL the reference pins): the reference "
                  "passes the transparent comparator, which rocThrust sorts by merging and which CCCL may or may not "
                  "hand to its radix sort, so both comparators are timed; each variant names its sample",
        "variants": variants,
    }


# -------------------------------------------------------------------------------------------------
# callers and consumers of the sort path: lexsort, searchsorted, unique
# -------------------------------------------------------------------------------------------------
class LexsortJob:
    """np.lexsort((k0, k1)): int32 secondary key with 1000 distinct values, float32 primary key with
    about 2^16 distinct values.  Both keys packed into one 64-bit word per element, one argsort."""

    name = "lexsort"

    def __init__(self, torch, lib, log2n):
        n = 1 << (26 if log2n is None else log2n)
        rng = np.random.default_rng(5)
        self.k0 = rng.integers(0, 1000, n).astype(np.int32)
        self.k1 = np.round(rng.standard_normal(n, dtype=np.float32) * 8192).astype(np.float32)
        self.n = n
        self.workload = f"lexsort((int32 1000 distinct, float32 ~2^16 distinct)) N=2^{int(np.log2(n))}, seed 5"
        dev = "cuda:0"
        self.torch, self.lib = torch, lib
        self.d_k0 = torch.from_numpy(self.k0).to(dev)
        self.d_k1 = torch.from_numpy(self.k1).to(dev)
        self.d_packed = torch.empty(n, dtype=torch.int64, device=dev)
        self.d_out = torch.empty(n, dtype=torch.int64, device=dev)
        self.tb = lib.cpn_local_sort_temp_bytes(8, n, n, 0, 1, 0)
        self.temp = torch.empty(self.tb, dtype=torch.uint8, device=dev)
        self.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.dtypes = (ctypes.c_int * 2)(3, 10)
        self.ptrs = (ctypes.c_void_p * 2)(self.d_k0.data_ptr(), self.d_k1.data_ptr())
        # pack: read 4+4, write 8; histogram: read 8; the passes that run (digits that vary): first reads
        # 8 and writes 8+4, middle ones move 8+4 both ways, the last reads 8+4 and writes 8
        self.alg = {"lexsort_pack": n * 16, "histogram": n * 8, "onesweep": n * 24}
        self.alg["total"] = None  # filled in from the number of passes that ran
        self.dominant = "onesweep"
        self.dtype = "u64"

    def step(self):
        lib, n, s = self.lib, self.n, self.stream
        rc = lib.cpn_lexsort_pack(2, self.dtypes, self.ptrs, None, 8, self.d_packed.data_ptr(), 1, n, s)
        rc |= lib.cpn_local_sort(8, self.d_packed.data_ptr(), None, self.d_out.data_ptr(), n, n, 0, 1,
                                 self.temp.data_ptr(), self.tb, s)
        assert rc == 0, rc

    def verify(self):
        idx = self.d_out
        a0, a1 = self.d_k0[idx], self.d_k1[idx]
        ordered = bool(((a1[:-1] < a1[1:]) | ((a1[:-1] == a1[1:]) & (a0[:-1] <= a0[1:]))).all())
        tie = (a1[:-1] == a1[1:]) & (a0[:-1] == a0[1:])
        stable = bool((idx[1:][tie] > idx[:-1][tie]).all())
        seen = self.torch.zeros(self.n, dtype=self.torch.bool, device=idx.device)
        seen[idx] = True
        return "ok" if ordered and stable and bool(seen.all()) else "FAILED"

    def cpu(self, oracle, threads):
        m = min(self.n, 1 << 24)
        t0 = time.perf_counter()
        oracle.lexsort((self.k0[:m], self.k1[:m]), threads=threads)
        return m, time.perf_counter() - t0, f"first 2^{int(np.log2(m))} elements of both keys; oracle.lexsort over oracle/sort_oracle.c"


class SearchsortedJob:
    """np.searchsorted(a, v, 'left'): a = 2^28 sorted float32, v = 2^24 float32 drawn from the same law."""

    name = "searchsorted"

    def __init__(self, torch, lib, log2n):
        n = 1 << (28 if log2n is None else log2n)
        m = max(n >> 4, 1)
        rng = np.random.default_rng(6)
        self.v = rng.standard_normal(m, dtype=np.float32)
        self.n, self.m = n, m
        self.workload = (f"searchsorted(sorted float32 N=2^{int(np.log2(n))}, float32 values M=2^{int(np.log2(m))}, "
                         "side=left), normal, seed 6")
        dev = "cuda:0"
        self.torch, self.lib = torch, lib
        g = torch.Generator(device=dev)
        g.manual_seed(6)
        self.d_a = torch.randn(n, dtype=torch.float32, device=dev, generator=g).sort().values  # input preparation only
        self.d_v = torch.from_numpy(self.v).to(dev)
        self.d_out = torch.empty(m, dtype=torch.int64, device=dev)
        self.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.tb = 0 if os.environ.get("CPN_BENCH_SEARCH_DIRECT") else lib.cpn_searchsorted_temp_bytes(10, n, m)
        self.temp = torch.empty(max(self.tb, 1), dtype=torch.uint8, device=dev)
        self.alg = {"total": m * (4 + 8), "searchsorted": m * (4 + 8)}
        self.dominant = "searchsorted"
        self.dtype = "u32"
        self.n_keys = m

    def step(self):
        rc = self.lib.cpn_searchsorted(10, self.d_a.data_ptr(), self.n, self.d_v.data_ptr(), self.m, 1,
                                       self.d_out.data_ptr(), self.temp.data_ptr() if self.tb else None, self.tb,
                                       self.stream)
        assert rc == 0, rc

    def verify(self):
        p = self.d_out
        a, v = self.d_a, self.d_v
        n = self.n
        right_ok = (p == n) | (a[p.clamp(max=n - 1)] >= v)
        left_ok = (p == 0) | (a[(p - 1).clamp(min=0)] < v)
        return "ok" if bool((right_ok & left_ok).all()) else "FAILED"

    def cpu(self, oracle, threads):
        a = self.d_a[: min(self.n, 1 << 26)].cpu().numpy()
        t0 = time.perf_counter()
        np.searchsorted(a, self.v, side="left")
        return self.m, time.perf_counter() - t0, (f"all {self.m} values against the first 2^{int(np.log2(a.size))} sorted elements; "
                                                  "numpy.searchsorted on one core (the oracle's own search is a Python loop)")


class UniqueJob:
    """np.unique(x): int32, 2^26 elements, about 2^20 distinct values."""

    name = "unique"

    def __init__(self, torch, lib, log2n):
        n = 1 << (26 if log2n is None else log2n)
        rng = np.random.default_rng(7)
        self.x = rng.integers(0, max(n >> 6, 2), n).astype(np.int32)
        self.n = n
        self.workload = f"unique(int32 N=2^{int(np.log2(n))}, values below N/64), seed 7"
        dev = "cuda:0"
        self.torch, self.lib = torch, lib
        self.d_in = torch.from_numpy(self.x).to(dev)
        self.d_out = torch.empty_like(self.d_in)
        self.count = torch.zeros(1, dtype=torch.int64, device=dev)
        self.tb = lib.cpn_unique_temp_bytes(3, n)
        self.temp = torch.empty(self.tb, dtype=torch.uint8, device=dev)
        self.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        distinct = min(n, max(n >> 6, 2))
        self.alg = {"total": n * 4 + 4 * n * 8 + 2 * n * 4 + distinct * 4, "onesweep": n * 8,
                    "unique_count": n * 4, "unique_scatter": n * 4 + distinct * 4, "histogram": n * 4}
        self.dominant = "onesweep"
        self.dtype = "u32"

    def step(self):
        rc = self.lib.cpn_unique(3, self.d_in.data_ptr(), self.d_out.data_ptr(), self.n, self.count.data_ptr(),
                                 self.temp.data_ptr(), self.tb, self.stream)
        assert rc == 0, rc

    def verify(self):
        c = int(self.count.item())
        u = self.d_out[:c]
        strictly = bool((u[1:] > u[:-1]).all())
        present = self.torch.zeros(max(self.n >> 6, 2), dtype=self.torch.bool, device=u.device)
        present[self.d_in.long()] = True
        return "ok" if strictly and c == int(present.sum()) and bool(present[u.long()].all()) else "FAILED"

    def cpu(self, oracle, threads):
        t0 = time.perf_counter()
        oracle.unique(self.x, threads=threads)
        return self.n, time.perf_counter() - t0, "the whole workload; oracle.unique over oracle/sort_oracle.c"


CONSUMERS = {"lexsort": LexsortJob, "searchsorted": SearchsortedJob, "unique": UniqueJob}


def run_consumer(args) -> dict:
    import torch

    from cupynumeric_amd import _lib

    if not torch.cuda.is_available():
        raise RuntimeError("bench.py needs a HIP device")
    lib = _lib.load()
    job = CONSUMERS[args.config](torch, lib, args.log2n)
    for _ in range(args.warmup):
        job.step()
    torch.cuda.synchronize()
    lib.cpn_profile_enable(1)
    _lib.profile_collect()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        job.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.cpn_profile_enable(0)
    by_label: dict[str, list[float]] = {}
    for label, ms in _lib.profile_collect():
        by_label.setdefault(label, []).append(ms)
    n_keys = getattr(job, "n_keys", job.n)
    step_s = elapsed / args.steps
    dom = job.dominant
    if dom == "onesweep":  # launches of skipped passes exit at once: keep the ones that moved data
        longest = max(by_label[dom])
        by_label["onesweep_skipped"] = [t for t in by_label[dom] if t < 0.1 * longest]
        by_label[dom] = [t for t in by_label[dom] if t >= 0.1 * longest]
        if not by_label["onesweep_skipped"]:
            del by_label["onesweep_skipped"]
    if job.alg.get("total") is None:
        ran = len(by_label["onesweep"]) / args.steps
        job.alg["total"] = job.alg["lexsort_pack"] + job.alg["histogram"] + ran * job.alg["onesweep"]
    avg_ms = float(np.mean(by_label[dom]))
    achieved = job.alg[dom] / (avg_ms * 1e-3)
    line = {
        "metric": f"elements/sec, {job.name}, 1 GPU",
        "value": n_keys / step_s,
        "unit": "keys/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_s * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": job.dtype,
        "data": "synthetic",
        "config": {"workload": job.workload, "keys": int(n_keys), "op": job.name},
        "roofline": {"kernel": dom, "bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK_BYTES_PER_S / 1e9,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_BYTES_PER_S, "traffic": None,
                     "bytes_per_launch": job.alg[dom], "avg_launch_ms": avg_ms,
                     "launches_per_step": len(by_label[dom]) / args.steps},
        "whole_step": {"algorithmic_bytes": job.alg["total"], "GBps": job.alg["total"] / step_s / 1e9,
                       "frac_of_hbm_peak": job.alg["total"] / step_s / HBM_PEAK_BYTES_PER_S},
        "kernels": {label: {"launches_per_step": len(v) / args.steps, "avg_ms": float(np.mean(v))}
                    for label, v in by_label.items()},
        "verify": job.verify(),
    }
    if not args.no_cpu_baseline:
        from oracle import sort_oracle as oracle

        threads = min(oracle.max_threads(), os.cpu_count() or 1, 16)
        count, dt, what = job.cpu(oracle, threads)
        line["cpu_baseline"] = {"value": count / dt, "unit": "keys/s", "cores": 1 if job.name == "searchsorted" else threads,
                                "kind": "port", "sample": f"{what}, {dt:.2f} s"}
    return line


# -------------------------------------------------------------------------------------------------
ROW_KERNELS = ("bitonic_row_sort", "tiny_row_sort", "wave_row_sort", "lds_row_sort", "count16_row_sort")


def verify_result(job: GpuJob, cfg: dict) -> str:
    """End-of-run check of the device result, on the device (full parity lives in tests/): 1-D
    argsorts through permutation, order and stability, which together fix the stable argsort; value
    sorts against torch.sort of the same input, element for element (equal or both NaN)."""
    torch = job.torch
    if cfg["op"] == "argsort":
        return verify_sample(job, cfg)
    tdt = {np.dtype(np.int32): torch.int32, np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64,
           np.dtype(np.float16): torch.float16, np.dtype(np.int64): torch.int64}.get(cfg["x"].dtype)
    if tdt is None:
        return "not checked here"
    x = job.d_in.view(tdt).view(job.shape)
    got = job.d_val.view(tdt).view(job.shape)
    ref = torch.sort(x, dim=0 if job.transposed else -1).values
    same = (got == ref) | ((got != got) & (ref != ref))
    return "ok" if bool(same.all()) else f"FAILED: {int((~same).sum())} elements differ from torch.sort"


def run_sort_workload(name: str, steps: int, warmup: int, log2n=None, rows=None, profile_steps: int = 5,
                      calibrate_copy: bool = False) -> tuple[dict, dict, GpuJob]:
    """One sort workload: `steps` timed steps between two device synchronisations with the library's
    launch timing off (that is `ms_per_step`), the same steps timed one by one with events on the
    stream (median and min), then a separate short loop with launch timing on for the per-kernel
    durations.  Returns (result fields, config, job)."""
    from cupynumeric_amd import _lib

    cfg = make_config(name, log2n, rows)
    job = GpuJob(cfg)
    torch, lib = job.torch, job.lib
    if calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB (shows up as the runtime's copyBuffer kernel)
        torch.cuda.synchronize()
        del src, dst

    lib.cpn_profile_enable(0)
    for _ in range(warmup):
        job.step()
    torch.cuda.synchronize()
    job.check_status()

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        job.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    job.check_status()

    # the same step, one at a time, between events on the stream the library launches on
    per_step = []
    for _ in range(steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        job.step()
        e1.record()
        torch.cuda.synchronize()
        per_step.append(e0.elapsed_time(e1))

    # per-kernel launch durations: the library's own HIP events, in a loop of their own (recording
    # them costs a few microseconds per launch, which the timed loop above does not pay)
    lib.cpn_profile_enable(1)
    _lib.profile_collect()  # drop anything recorded earlier
    torch.cuda.synchronize()
    for _ in range(profile_steps):
        job.step()
    torch.cuda.synchronize()
    lib.cpn_profile_enable(0)
    records = _lib.profile_collect()
    job.check_status()

    step_s = elapsed / steps
    by_label: dict[str, list[float]] = {}
    for label, ms in records:
        by_label.setdefault(label, []).append(ms)
    passes_run = None
    if "onesweep_distinct" in by_label:  # the one pass of an index-only sort on few different keys: a launch of its own shape
        by_label.setdefault("onesweep", []).extend(by_label.pop("onesweep_distinct"))
    if "onesweep" in by_label:  # launches of skipped passes exit at once: keep the ones that moved data
        longest = max(by_label["onesweep"])
        skipped = [t for t in by_label["onesweep"] if t < 0.1 * longest]
        by_label["onesweep"] = [t for t in by_label["onesweep"] if t >= 0.1 * longest]
        if skipped:
            by_label["onesweep_skipped"] = skipped
        passes_run = round(len(by_label["onesweep"]) / profile_steps)
    # sweeps whose launch exits at once because the device-side plan has no use for them
    for label in ("histogram", "virtual_histogram", "distinct_sweep"):
        if label in by_label and cfg["x"].nbytes >= (1 << 26) and max(by_label[label]) < 0.02:
            by_label[label + "_skipped"] = by_label.pop(label)
    merged_halves = "merge_halves" in by_label  # rows longer than the LDS capacity: sorted pieces, merged level by level
    alg = algorithmic_bytes(cfg, job.uses_lds_rows or merged_halves, passes_run)
    merge_levels = 0
    if merged_halves:
        n, kb, pos = cfg["x"].size, cfg["x"].dtype.itemsize, (8 if cfg["op"] == "argsort" else 0)
        merge_levels = round(len(by_label["merge_halves"]) / profile_steps)
        dominant = "lds_row_sort"
        alg[dominant] = n * (kb + kb + pos)  # every piece read, written with its positions
        # per launch, averaged over the levels: all but the last read and write keys and positions, the
        # last one writes the requested output only
        alg["merge_halves"] = ((2 * merge_levels - 1) * n * (kb + pos) + n * (pos if pos else kb)) / merge_levels
    elif job.uses_lds_rows:  # whichever of the per-row kernels the row length selects
        dominant = next(k for k in ROW_KERNELS if k in by_label)
        alg[dominant] = alg["lds_row_sort"]
    else:
        dominant = "onesweep"
    avg_ms = float(np.mean(by_label[dominant]))
    achieved = alg[dominant] / (avg_ms * 1e-3)
    kernels = {
        label: {"launches_per_step": len(v) / profile_steps, "avg_ms": float(np.mean(v)),
                "algorithmic_GBps": (alg[label] / (float(np.mean(v)) * 1e-3) / 1e9) if label in alg else None}
        for label, v in by_label.items()
    }
    roofline = {
        "kernel": dominant,
        "bound": "hbm",
        "achieved": achieved / 1e9,
        "peak": HBM_PEAK_BYTES_PER_S / 1e9,
        "unit": "GB/s",
        "frac": achieved / HBM_PEAK_BYTES_PER_S,
        "traffic": measured_traffic_bytes(name, dominant) if (log2n is None and rows is None) else None,
        "bytes_per_launch": alg[dominant],
        "avg_launch_ms": avg_ms,
        "launches_per_step": len(by_label[dominant]) / profile_steps,
    }
    if "onesweep_baseline_formula" in alg and dominant == "onesweep":
        # for comparison only: the baseline's accounting moves an 8-byte payload in every pass, this
        # build moves 4-byte row positions, so `achieved` above is the smaller, real figure
        fb = alg["onesweep_baseline_formula"]
        roofline["baseline_formula"] = {"bytes_per_launch": fb, "achieved": fb / (avg_ms * 1e-3) / 1e9,
                                        "frac": fb / (avg_ms * 1e-3) / HBM_PEAK_BYTES_PER_S}
    step_bytes = sum(alg.get(k, 0) * len(v) / profile_steps for k, v in by_label.items() if k in alg)
    fields = {
        "value": cfg["x"].size / step_s,
        "ms_per_step": step_s * 1e3,
        "ms_per_step_median": float(np.median(per_step)),
        "ms_per_step_min": float(np.min(per_step)),
        "dtype": {1: "u8", 2: "u16", 4: "u32", 8: "u64"}[cfg["x"].dtype.itemsize],
        "config": {"workload": cfg["workload"], "keys": int(cfg["x"].size), "op": cfg["op"],
                   "path": (f"lds_row_sort on {1 << merge_levels} pieces of a row + {merge_levels} x merge_halves" if merged_halves else dominant)
                   if (job.uses_lds_rows or merged_halves) else f"onesweep, 8-bit digits, {passes_run} passes ran",
                   "workspace_bytes": int(job.temp_bytes)},
        "roofline": roofline,
        "whole_step": {"algorithmic_bytes": step_bytes, "GBps": step_bytes / step_s / 1e9,
                       "frac_of_hbm_peak": step_bytes / step_s / HBM_PEAK_BYTES_PER_S,
                       **({"baseline_formula_bytes": alg["whole_baseline_formula"],
                           "baseline_formula_frac": alg["whole_baseline_formula"] / step_s / HBM_PEAK_BYTES_PER_S}
                          if "whole_baseline_formula" in alg else {})},
        "kernels": kernels,
        "verify": verify_result(job, cfg),
    }
    return fields, cfg, job


# -------------------------------------------------------------------------------------------------
# the reference's own sort microbenchmark, through the public API and through the C ABI
# -------------------------------------------------------------------------------------------------
TORCH_DTYPES = {"float16": "float16", "float32": "float32", "float64": "float64", "int32": "int32", "int64": "int64"}

# examples/microbenchmarks/sort_bench.py:44-51: the six variants; :104-105: the two dtypes
MICRO_VARIANTS = ("sort-1D", "argsort-1D", "sort-2D-flat", "argsort-2D-flat", "sort-2D-skinny", "argsort-2D-skinny")
MICRO_DTYPES = ("float32", "float64")


def micro_shape(variant: str, size: int) -> tuple[int, ...]:
    """Array shape of a variant at `size` (examples/microbenchmarks/sort_bench.py:54-68)."""
    import math

    if variant.endswith("-1D"):
        return (size,)
    a, b = math.ceil(math.pow(size, 1 / 4)), math.ceil(math.pow(size, 3 / 4))
    return (a, b) if variant.endswith("-2D-flat") else (b, a)


def device_random(torch, count: int, dtype: str, seed: int, law: str = "uniform"):
    """`count` seeded random elements of `dtype` generated on the device, as a byte tensor: uniform in
    [0, 1) (what the reference's benchmarks sort, examples/_benchmark/random_array.py:43-49) or
    standard normal."""
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    tdt = getattr(torch, TORCH_DTYPES[dtype])
    gen_dt = torch.float32 if tdt == torch.float16 else tdt
    x = torch.empty(count, dtype=gen_dt, device="cuda:0")
    if law == "uniform":
        x.uniform_(0.0, 1.0, generator=g)
    else:
        x.normal_(generator=g)
    return x.to(tdt).view(torch.uint8)


def verify_against_torch(torch, result_bytes, input_bytes, shape, dtype: str, op: str, axis: int) -> str:
    """Element for element against torch's stable sort of the same device input along `axis` (values equal
    or both NaN; indices equal: the stable argsort is unique)."""
    tdt = getattr(torch, TORCH_DTYPES[dtype])
    x = input_bytes.view(tdt).view(shape)
    ref = torch.sort(x, dim=axis, stable=True)
    if op == "argsort":
        same = result_bytes.view(torch.int64).view(shape) == ref.indices
    else:
        got = result_bytes.view(tdt).view(shape)
        same = (got == ref.values) | ((got != got) & (ref.values != ref.values))
    bad = int((~same).sum())
    del ref
    return "ok" if bad == 0 else f"FAILED: {bad} elements differ from torch.sort(stable=True)"


def timed_calls(torch, fn, runs: int, warmup: int) -> float:
    """The reference's timed loop (examples/_benchmark/timer.py:199-241): `warmup` untimed calls, then
    `runs` calls between a start and a stop that waits for the device; calls are ordered by the stream
    they are issued on (the reference's fence), the host does not wait between them.  Returns
    milliseconds per call, host wall clock."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(runs):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / runs


def time_case(torch, num, input_bytes, shape, dtype: str, op: str, axis: int, runs: int, warmup: int,
              verify: bool = True) -> dict:
    """One case both ways: through the public API (`cupynumeric.sort(x, axis)` / `argsort`: result and
    workspace allocated per call, status bookkeeping included) and through the C ABI (`cpn_local_sort`
    and `cpn_swapaxes_copy` with outputs and workspace allocated beforehand)."""
    from cupynumeric_amd._thunk import DeviceArray

    a = num.ndarray(shape, np.dtype(dtype), thunk=DeviceArray.from_device(input_bytes, shape, dtype))
    api_fn = (lambda: num.argsort(a, axis)) if op == "argsort" else (lambda: num.sort(a, axis))
    api_ms = timed_calls(torch, api_fn, runs, warmup)
    out = {"shape": list(shape), "api_ms": round(api_ms, 5)}
    if verify:
        res = api_fn()
        out["verify"] = verify_against_torch(torch, res._thunk.base.device(), input_bytes, shape, dtype, op, axis)
        del res
    torch.cuda.empty_cache()
    job = GpuJob(dict(x_dev=input_bytes, shape=shape, dtype=dtype, op=op, axis=axis))
    abi_ms = timed_calls(torch, job.step, runs, warmup)
    job.check_status()
    if verify:
        got = job.d_idx.view(torch.uint8) if op == "argsort" else job.d_val
        v = verify_against_torch(torch, got, input_bytes, shape, dtype, op, axis)
        if v != "ok" or out["verify"] != "ok":
            out["verify"] = f"api: {out['verify']}; abi: {v}"
    out["abi_ms"] = round(abi_ms, 5)
    out["api_over_abi"] = round(api_ms / abi_ms, 3)
    out["keys_per_s_api"] = int(np.prod(shape, dtype=np.int64)) / (api_ms * 1e-3)
    del job
    torch.cuda.empty_cache()
    return out


def run_reference_microbenchmarks(log2size: int = 28, runs: int = 5, warmup: int = 2) -> dict:
    """The plan of the reference's sort microbenchmark (examples/microbenchmarks/sort_bench.py:44-68,
    104-130) at size 2^log2size: six variants x float32 / float64, `np.sort(x, -1)` / `np.argsort(x, -1)`
    on uniform [0, 1) input, each through the public API and through the C ABI; sort-1D / argsort-1D of
    float32 for sizes 2^10 ... 2^26 (the regime of examples/sort.py and of the reference's CI, which runs
    the suite at size 1000); and two sorts along other axes than the last."""
    import torch

    import cupynumeric as num

    size = 1 << log2size
    cases = {}
    for k, dtype in enumerate(MICRO_DTYPES):
        data = device_random(torch, size, dtype, seed=11 + k)
        for variant in MICRO_VARIANTS:
            op = variant.split("-")[0]
            cases[f"{variant}:{dtype}"] = time_case(torch, num, data, micro_shape(variant, size), dtype, op, -1, runs, warmup)
        del data
        torch.cuda.empty_cache()
    sweep = {}
    data = device_random(torch, 1 << 26, "float32", seed=13)
    for log2s in range(10, 27, 2):
        n = 1 << log2s
        reps = 200 if log2s <= 18 else (50 if log2s <= 22 else 10)
        for op in ("sort", "argsort"):
            part = data[: 4 * n]
            r = time_case(torch, num, part, (n,), "float32", op, -1, reps, 5, verify=True)
            sweep[f"{op}-1D:2^{log2s}"] = {"api_us": round(r["api_ms"] * 1e3, 2), "abi_us": round(r["abi_ms"] * 1e3, 2),
                                          "api_over_abi": r["api_over_abi"], "verify": r["verify"]}
    del data
    torch.cuda.empty_cache()
    axes = {}
    data = device_random(torch, 1 << 28, "float32", seed=14)
    axes["argsort axis 0 of (8192, 8192) float32"] = time_case(
        torch, num, data[: 4 * 8192 * 8192], (8192, 8192), "float32", "argsort", 0, runs, warmup)
    axes["sort axis 1 of (256, 512, 2048) float32"] = time_case(
        torch, num, data, (256, 512, 2048), "float32", "sort", 1, runs, warmup)
    del data
    torch.cuda.empty_cache()
    ok = all(c["verify"] == "ok" for group in (cases, sweep, axes) for c in group.values())
    return {"size": f"2^{log2size}", "runs": runs, "warmup": warmup, "input": "uniform [0, 1), generated on the device, seeded",
            "timing": "host wall clock around `runs` calls, device synchronised before the first and after the last",
            "cases": cases, "sizes_1d_float32": sweep, "other_axes": axes, "verify": "ok" if ok else "FAILED"}


# the other workloads reported beside the headline: the baseline's configs and the reference's own
# 2-D microbenchmark shapes
ALL_CONFIGS = ("c1", "c3", "c4", "c5", "flat", "skinny")


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    known = ["c1", "c2", "c3", "c4", "c5", "flat", "skinny", "lexsort", "searchsorted", "unique"]

    def config_name(text: str) -> str:
        if text in known or text.startswith("rows:"):
            return text
        raise argparse.ArgumentTypeError(f"one of {', '.join(known)} or rows:<dtype>:<rows>:<row length>:<sort|argsort>")

    ap.add_argument("--config", default="c2", type=config_name,
                    help="c1..c5: the sort workloads of the baseline; flat / skinny: the 2-D shapes of the "
                         "reference's sort microbenchmark; lexsort / searchsorted / unique: the callers and "
                         "consumers of the sort path, on workloads of this file's own choosing; "
                         "rows:<dtype>:<rows>:<row length>:<sort|argsort>: batched rows of any length")
    ap.add_argument("--edges", action="store_true",
                    help="instead of a workload: time rows of length n and n + 1 for every n at which the "
                         "library changes kernels (EDGE_LENGTHS), one JSON line")
    ap.add_argument("--micro", action="store_true",
                    help="instead of a workload: the reference's sort microbenchmark matrix (six variants x float32 / "
                         "float64), the 1-D sizes 2^10 ... 2^26 and two sorts along other axes, each through the public "
                         "API and through the C ABI; one JSON line")
    ap.add_argument("--micro-log2size", type=int, default=28, help="size of the microbenchmark matrix, 2^L elements")
    ap.add_argument("--log2n", type=int, default=None, help="shrink a 1-D workload to 2^L keys")
    ap.add_argument("--rows", type=int, default=None, help="shrink a 2-D workload to this many rows")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-all-configs", action="store_true",
                    help="the default run (c2 at full size) also times the other workloads, 10 steps each "
                         "(all_configs), the reference's microbenchmark matrix through the public API and the C ABI "
                         "(sort_bench) and the row-length edges (edges); this switch leaves them out")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy, the known-size kernel that "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build sorts on one GPU; --gpus must be 1 (no multi-GPU sample sort is built)")

    if args.edges:
        print(json.dumps(run_edges()))
        return
    if args.micro:
        print(json.dumps({"metric": "ms per call, the reference's sort microbenchmark, public API and C ABI", "unit": "ms",
                          "n_gpus": 1, "data": "synthetic", "sort_bench": run_reference_microbenchmarks(args.micro_log2size)}))
        return
    if args.config in CONSUMERS:
        print(json.dumps(run_consumer(args)))
        return

    fields, cfg, job = run_sort_workload(args.config, args.steps, args.warmup, args.log2n, args.rows,
                                         calibrate_copy=args.calibrate_copy)
    torch = job.torch
    device_rates = measure_device_rates(torch)
    # what this device sustains on plain streaming kernels, measured in this run: the published peak
    # is not reached by a copy either
    fields["roofline"]["device_rates"] = device_rates
    fields["roofline"]["frac_of_device_copy"] = fields["roofline"]["achieved"] / device_rates["copy_GBps"]
    headline = args.config == "c2" and args.log2n is None
    line = {
        "metric": "sorted keys/sec, stable argsort fp32 N=2^28, 1 GPU" if headline
        else f"sorted keys/sec, config {args.config}, 1 GPU",
        "value": fields["value"],
        "unit": "keys/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": fields["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": fields["dtype"],
        "data": "synthetic",
        "config": fields["config"],
        "roofline": fields["roofline"],
        "ms_per_step_median": fields["ms_per_step_median"],
        "ms_per_step_min": fields["ms_per_step_min"],
        "whole_step": fields["whole_step"],
        "kernels": fields["kernels"],
        "verify": fields["verify"],
    }
    del job
    torch.cuda.empty_cache()
    if headline and not args.no_all_configs:
        others = {}
        for name in ALL_CONFIGS:
            f, _, j = run_sort_workload(name, steps=10, warmup=2)
            r = f["roofline"]
            others[name] = {
                "workload": f["config"]["workload"], "keys": f["config"]["keys"], "path": f["config"]["path"],
                "ms_per_step": f["ms_per_step"], "ms_per_step_median": f["ms_per_step_median"],
                "ms_per_step_min": f["ms_per_step_min"], "keys_per_s": f["value"],
                "dominant_kernel": r["kernel"], "kernel_avg_ms": r["avg_launch_ms"],
                "kernel_launches_per_step": r["launches_per_step"], "algorithmic_bytes_per_launch": r["bytes_per_launch"],
                "frac": r["frac"], "traffic": r["traffic"],
                "whole_step_frac": f["whole_step"]["frac_of_hbm_peak"],
                "kernels_ms": {k: round(v["avg_ms"] * v["launches_per_step"], 4) for k, v in f["kernels"].items()},
                "verify": f["verify"],
            }
            del j
            torch.cuda.empty_cache()
        line["all_configs"] = others
        line["sort_bench"] = run_reference_microbenchmarks()
        line["edges"] = run_edges_compact()
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
