"""The five baseline workloads on the GPU: exact parity with the CPU oracle at a size the oracle
finishes in seconds, and size-independent properties (permutation, order, stability) at full size,
checked on the device."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
from conftest import assert_same_bits

import bench
from oracle import sort_oracle as oracle

pytestmark = pytest.mark.gpu

REDUCED = {"c1": dict(log2n=20), "c2": dict(log2n=20), "c3": dict(rows=256), "c4": dict(log2n=20), "c5": dict(rows=512)}


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_config_matches_oracle_at_reduced_size(name):
    cfg = bench.make_config(name, **REDUCED[name])
    job = bench.GpuJob(cfg)
    job.step()
    job.torch.cuda.synchronize()
    job.check_status()
    got = job.result()
    x = cfg["x"]
    if cfg["op"] == "argsort":
        want = oracle.argsort(x, axis=cfg["axis"], kind="stable", threads=4)
    else:
        want = oracle.sort(x, axis=cfg["axis"], kind="stable", threads=4)
    assert_same_bits(got, want, cfg["workload"])


def ordered_key_torch(torch, raw, np_dtype):
    """NumPy-order integer key of raw bit patterns (a torch restatement used only as a checker):
    floats: NaN -> max, -0 -> +0, negative -> ~bits, positive -> bits | sign; computed in int64
    arithmetic so that comparisons are signed-safe."""
    dt = np.dtype(np_dtype)
    if dt.kind == "i":
        return raw.to(torch.int64)
    bits = dt.itemsize * 8
    v = raw.to(torch.int64) & ((1 << bits) - 1) if bits < 64 else raw
    if dt.kind in "ub":
        return v
    assert bits < 64
    sign = 1 << (bits - 1)
    inf = {16: 0x7C00, 32: 0x7F800000}[bits]
    mag = v & (sign - 1)
    key = torch.where((v & sign) != 0, (~v) & ((1 << bits) - 1), v | sign)
    key = torch.where(mag == 0, torch.full_like(v, sign), key)
    key = torch.where(mag > inf, torch.full_like(v, (1 << bits) - 1), key)
    return key


def test_c1_full_size_sorted_permutation():
    cfg = bench.make_config("c1")
    job = bench.GpuJob(cfg)
    torch = job.torch
    job.step()
    torch.cuda.synchronize()
    job.check_status()
    out = job.d_val.view(torch.int32)
    inp = job.d_in.view(torch.int32)
    assert bool((out[:-1] <= out[1:]).all())
    # same multiset: compare against an independent device sort of the input
    assert bool((out == torch.sort(inp).values).all())


def test_c2_full_size_stable_argsort_properties():
    """permutation + keys non-decreasing under the NumPy order + indices increasing inside ties
    characterise the stable argsort uniquely, so they prove bit-exactness at 2^28."""
    cfg = bench.make_config("c2")
    job = bench.GpuJob(cfg)
    torch = job.torch
    job.step()
    torch.cuda.synchronize()
    job.check_status()
    assert bench.verify_sample(job, cfg) == "ok"
    idx = job.d_idx
    raw = job.d_in.view(torch.int32)
    key = ordered_key_torch(torch, raw, np.float32)[idx]
    assert bool((key[:-1] <= key[1:]).all())
    tie = key[:-1] == key[1:]
    assert bool((idx[1:][tie] > idx[:-1][tie]).all())
    assert int(idx.min()) == 0 and int(idx.max()) == idx.numel() - 1
    # exact comparison with the oracle on the head of the result: the first positions of the
    # output are the most negative keys; their original indices must agree with a CPU sort of
    # exactly those elements
    head = idx[:100000].cpu().numpy()
    x = cfg["x"]
    sub = x[np.sort(head)]
    order = oracle.argsort(sub, kind="stable")
    assert np.array_equal(np.sort(head)[order], head)


def test_c4_full_size_heavy_duplicates():
    cfg = bench.make_config("c4")
    job = bench.GpuJob(cfg)
    torch = job.torch
    job.step()
    torch.cuda.synchronize()
    job.check_status()
    assert bench.verify_sample(job, cfg) == "ok"
    # closed form: with 16 distinct keys the stable argsort is the concatenation, in key order,
    # of the ascending positions of each key
    x = cfg["x"]
    idx = job.d_idx.cpu().numpy()
    pos = 0
    for v in np.sort(np.unique(x)):
        where = np.flatnonzero(x == v)
        assert np.array_equal(idx[pos : pos + where.size], where)
        pos += where.size
    assert pos == x.size


def test_c3_full_size_rows_sorted():
    cfg = bench.make_config("c3")
    job = bench.GpuJob(cfg)
    torch = job.torch
    job.step()
    torch.cuda.synchronize()
    job.check_status()
    out = job.d_val.view(torch.float64).view(65536, 1024)
    inp = job.d_in.view(torch.float64).view(65536, 1024)
    assert bool((out[:, :-1] <= out[:, 1:]).all())
    assert bool((out == torch.sort(inp, dim=1).values).all())  # distinct finite keys: any correct sort agrees
    rows = [0, 1, 32767, 65535]
    assert_same_bits(out[rows].cpu().numpy(), oracle.sort(cfg["x"][rows]), "c3 sample rows")


def test_c5_full_size_axis0():
    cfg = bench.make_config("c5")
    job = bench.GpuJob(cfg)
    torch = job.torch
    job.step()
    torch.cuda.synchronize()
    job.check_status()
    out = job.d_val.view(torch.float16).view(8192, 8192)
    inp = job.d_in.view(torch.float16).view(8192, 8192)
    assert bool((out[:-1, :] <= out[1:, :]).all())
    # the whole result, element for element: an independent sort of every column must agree in
    # value everywhere (no NaN in this workload; a -0.0 and a +0.0 of one column may stand in either
    # order in torch's result, hence equality of values, and the exact bits on the sample below)
    ref = torch.sort(inp, dim=0).values
    assert bool((out == ref).all()), "columns differ from an independent sort of the input"
    not_zero = ref != 0
    assert bool((out.view(torch.int16)[not_zero] == ref.view(torch.int16)[not_zero]).all())
    del ref, not_zero
    cols = [0, 1, 4097, 8191]
    got = out[:, cols].cpu().numpy()
    want = oracle.sort(np.ascontiguousarray(cfg["x"][:, cols]), axis=0)
    assert_same_bits(got, want, "c5 sample columns")
    # idempotence: sorting the sorted array changes nothing
    job2 = bench.GpuJob(dict(cfg, x=job.result()))
    job2.step()
    torch.cuda.synchronize()
    assert bool((job2.d_val == job.d_val).all())


def test_more_than_2_to_31_elements():
    """One row of 2^31 + 12345 uint16 keys: element counts and offsets beyond 32 bits, the 64-bit row
    kernels at their real size.  Checked on the device through the properties that characterise a
    stable argsort (permutation, order, ties in input order) and a sort (order, same histogram)."""
    import ctypes

    import torch

    from cupynumeric_amd import _lib

    free, _total = torch.cuda.mem_get_info()
    if free < 90 * (1 << 30):
        pytest.skip("needs about 80 GiB of free device memory")
    lib = _lib.load()
    dev = torch.device("cuda")
    n = (1 << 31) + 12345
    g = torch.Generator(device=dev)
    g.manual_seed(31)
    keys = torch.randint(0, 1 << 16, (n,), dtype=torch.int32, device=dev, generator=g).to(torch.int16)  # uint16 bit patterns
    code = _lib.DTYPE_CODES[np.dtype(np.uint16)]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    # argsort
    idx = torch.empty(n, dtype=torch.int64, device=dev)
    tb = lib.cpn_local_sort_temp_bytes(code, n, n, 0, 1, 0)
    temp = torch.empty(tb, dtype=torch.uint8, device=dev)
    rc = lib.cpn_local_sort(code, keys.data_ptr(), None, idx.data_ptr(), n, n, 0, 1, temp.data_ptr(), tb, stream)
    assert rc == 0, _lib.status_string(rc)
    assert lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
    del temp
    assert int(idx.min()) == 0 and int(idx.max()) == n - 1
    seen = torch.zeros(n, dtype=torch.bool, device=dev)
    seen[idx] = True
    assert bool(seen.all()), "indices are not a permutation"
    del seen
    k = (keys[idx].to(torch.int32) & 0xFFFF)
    assert bool((k[1:] >= k[:-1]).all()), "keys[idx] is not ascending"
    out_of_order_tie = (k[1:] == k[:-1]) & (idx[1:] <= idx[:-1])  # (no mask indexing: 2^31 elements overflow it)
    assert not bool(out_of_order_tie.any()), "ties are not in input order"
    del out_of_order_tie, idx

    # sort (values only): ascending and the same multiset
    out = torch.empty_like(keys)
    tb = lib.cpn_local_sort_temp_bytes(code, n, n, 1, 0, 0)
    temp = torch.empty(tb, dtype=torch.uint8, device=dev)
    rc = lib.cpn_local_sort(code, keys.data_ptr(), out.data_ptr(), None, n, n, 0, 1, temp.data_ptr(), tb, stream)
    assert rc == 0, _lib.status_string(rc)
    assert lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
    assert bool(((out.to(torch.int32) & 0xFFFF) == k).all()), "sorted values differ from keys[argsort]"


def test_more_rows_than_a_grid_has_blocks():
    """(2^31 + 7, 1) int8: rows of one element, more of them than one launch can take; the row kernels
    are launched in chunks.  Sorting rows of one element is the identity, their argsort is the offset."""
    import ctypes

    import torch

    from cupynumeric_amd import _lib

    free, _total = torch.cuda.mem_get_info()
    if free < 30 * (1 << 30):
        pytest.skip("needs about 22 GiB of free device memory")
    lib = _lib.load()
    dev = torch.device("cuda")
    n = (1 << 31) + 7
    g = torch.Generator(device=dev)
    g.manual_seed(32)
    keys = torch.randint(-128, 128, (n,), dtype=torch.int8, device=dev, generator=g)
    code = _lib.DTYPE_CODES[np.dtype(np.int8)]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tb = lib.cpn_local_sort_temp_bytes(code, n, 1, 1, 1, 0)
    assert tb > 0
    temp = torch.empty(tb, dtype=torch.uint8, device=dev)
    out = torch.zeros_like(keys)
    idx = torch.full((n,), -7, dtype=torch.int64, device=dev)
    rc = lib.cpn_local_sort(code, keys.data_ptr(), out.data_ptr(), idx.data_ptr(), n, 1, 3, 1, temp.data_ptr(), tb, stream)
    assert rc == 0, _lib.status_string(rc)
    assert lib.cpn_local_sort_check(temp.data_ptr(), stream) == 0
    assert bool((out == keys).all())
    assert bool((idx == 3).all())
