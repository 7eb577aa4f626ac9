#!/usr/bin/env python3
"""Headline benchmark: batched hashmap get / set at 64M int64 keys -> float32 values on one
MI355X, load factors 0.5 and 0.9 (synthetic data).

One "step" is one `get` of a 64M-query batch (50% hits drawn Zipf(1.1) over the stored keys,
50% uniform misses) against the load-factor-0.5 table.  The JSON line also carries set
throughput, the load-factor-0.9 figures, mean probe lengths, the HBM roofline of the get kernel
(`roofline.achieved` / `frac`: the bytes that crossed the HBM interface, from profiler counters,
over the kernel's live duration), the other four benchmark configurations, the multi-word layout
and the DOK indexing kernels at scale (`roofline.other_legs`), and a CPU baseline (the reference
algorithm restated in C, timed on this machine's cores on the benchmark's own keys and queries).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--keys N] [--no-cpu] [--headline-only]
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per measured leg (everything the leg launches, per repetition), from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of `bench.py --markers --no-cpu --calibrate --steps 10`, the counter
# units scaled against a table scan and a table clear of known size (the files under profiles/ hold
# the runs).  The figures belong to one state of the kernel sources, named by `csrc_sha16` (see
# csrc_sha16()): when the sources have changed since, nothing measured is reported.
# PROFILED-BEGIN
PROFILED = {
    "csrc_sha16": "aa601f8a2352ca93",
    "bytes": {
        "get_lf05": 6.657e+09,
        "line_gather_lf05": 8.877e+09,
        "set_cas_lf05": 1.599e+10,
        "set_bulk_lf05": 7.69e+09,
        "build_lf05": 5.971e+09,
        "overwrite_cas_lf05": 1.177e+10,
        "update_existing_lf05": 1.157e+10,
        "remove_lf05": 5.688e+09,
        "remove_cas_lf05": 6.769e+09,
        "remove_bulk_lf05": 3.561e+09,
        "get_lf09": 7.065e+09,
        "set_cas_lf09": 1.923e+10,
        "set_bulk_lf09": 6.144e+09,
        "build_lf09": 5.188e+09,
        "cfg1_set_65536": 1.639e+07,
        "cfg1_get_131072": 1.352e+07,
        "cfg1_remove_32768": 5.211e+06,
        "cfg2_set_1M_f32x3_i64x5": 4.802e+08,
        "cfg2_upsert_1M": 5.45e+08,
        "cfg2_get_2M": 3.722e+08,
        "cfg2_remove_250K": 4.348e+07,
        "cfg4_construct_50M": 4.421e+09,
        "cfg4_getitem_4096x256": 1.406e+08,
        "cfg4_setitem_10M_with_growth": 7.219e+09,
        "cfg4_setitem_10M_overwrite": 1.865e+09,
        "cfg4_readout": 4.207e+09,
        "cfg5_construct_100M": 1.07e+10,
        "cfg5_64_getitems": 1.06e+09,
        "cfg5_remove_20M": 4.717e+09,
        "cfg5_reinsert_20M": 4.396e+09,
        "tagged_set_lf05": 1.184e+10,
        "tagged_build_lf05": 1.492e+10,
        "tagged_overwrite_lf05": 1.165e+10,
        "tagged_get_lf05": 6.068e+09,
        "tagged_remove_lf05": 1.518e+09,
        "tagged_set_lf075": 1.403e+10,
        "tagged_build_lf075": 1.575e+10,
        "tagged_overwrite_lf075": 1.362e+10,
        "tagged_get_lf075": 6.433e+09,
        "tagged_remove_lf075": 1.682e+09,
        "dok_getitem_2p26": 1.161e+10,
        "dok_setitem_10M": 2.192e+09,
        "dok_setitem_10M_overwrite": 1.865e+09,
        "dok_readout": 4.25e+09,
        "dok_lin_construct_10M": 9.805e+08,
        "dok_lin_getitem_4M": 6.526e+08,
        "dok_lin_setitem_4M": 8.994e+08,
        "dok_wide_construct_10M": 3.174e+09,
        "dok_wide_getitem_4M": 6.207e+08,
        "dok_wide_setitem_4M": 9.103e+08,
    },
}
# PROFILED-END
# algorithmic bytes per op for 8-byte keys and 4-byte values: one 128-byte bucket line per op,
# plus the batch row and the outputs
B_GET = 8 + 128 + 4 + 1           # key in, bucket line, value out, flag out


def csrc_sha16():
    """First 16 hex digits of the SHA-256 over the kernel sources, in name order."""
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "doksparse_amd", "csrc")
    for name in sorted(os.listdir(d)):
        with open(os.path.join(d, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def measured(leg, kernel_ms):
    """Roofline figures of a leg from its profiled HBM bytes and the live duration; None where no
    profile of the current sources exists."""
    nbytes = PROFILED["bytes"].get(leg) if PROFILED["csrc_sha16"] == csrc_sha16() else None
    if nbytes is None or kernel_ms is None:
        return None
    gbs = nbytes / (kernel_ms * 1e-3) / 1e9
    return {"traffic": nbytes, "gbs": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4)}


def leg_entry(leg, ms, ops, level):
    """One entry of roofline.other_legs."""
    m = measured(leg, ms)
    return {"ms": ms, "mops": round(ops / ms / 1e3, 1), "level": level,
            "traffic": m and m["traffic"], "bytes_per_op": m and round(m["traffic"] / ops, 1),
            "measured_gbs": m and m["gbs"], "frac_measured": m and m["frac"]}


def make_unique_keys(n, gen, device):
    k = torch.randint(0, 2**62, (int(n * 1.002) + 1024,), generator=gen, device=device, dtype=torch.long)
    k = torch.unique(k)
    assert k.shape[0] >= n
    perm = torch.randperm(k.shape[0], generator=gen, device=device)[:n]
    return k[perm].contiguous()


def make_queries(keys, n_q, gen, device, zipf_s=1.1):
    """50% hits with rank ~ r^-s over the stored keys (rank -> key through the keys' own random
    order), 50% uniform misses, shuffled."""
    n = keys.shape[0]
    n_hit = n_q // 2
    w = torch.arange(1, n + 1, device=device, dtype=torch.float64).pow_(-zipf_s)
    cdf = torch.cumsum(w, 0)
    del w
    u = torch.rand(n_hit, generator=gen, device=device, dtype=torch.float64) * cdf[-1]
    rank = torch.searchsorted(cdf, u).clamp_(max=n - 1)
    del cdf, u
    hits = keys[rank]
    del rank
    misses = torch.randint(0, 2**62, (n_q - n_hit,), generator=gen, device=device, dtype=torch.long)
    q = torch.cat([hits, misses])
    del hits, misses
    q = q[torch.randperm(n_q, generator=gen, device=device)].contiguous()
    return q, n_hit


class LegMarks:
    """--markers (profiling runs): every measured leg is bracketed by two tiny launches of the
    library's clear kernel on a scratch table, whose grid sizes say which leg begins (leg number
    x 256 threads, numbers from 3) and that it ends (256 threads), so that a kernel trace or a counter
    run can be cut into legs without knowing the launch sequence.  The numbers are printed at the end
    (`{"leg_ids": ...}`).  The markers sit outside the timed regions."""
    ids = {}
    state = None

    @classmethod
    def enable(cls, device):
        from doksparse_amd import CudaClosedHashmap
        hm = CudaClosedHashmap(n_buckets=1 << 17, device=device)
        hm.set(torch.arange(8, device=device)[:, None], torch.zeros(8, 1, device=device))
        cls.state = (hm, device)

    @classmethod
    def _launch(cls, number):
        from doksparse_amd import _lib
        from doksparse_amd.closed_hashmap import _stream_ptr
        hm, device = cls.state
        desc = _lib.DokTable.from_buffer_copy(hm._desc)
        desc.n_phys_buckets = 64 * number                  # (the clear kernel: one workgroup per 64 buckets)
        assert desc.n_phys_buckets <= hm._n_phys
        _lib.check(_lib.load().dok_table_clear(ctypes.byref(desc), _stream_ptr(device)), "marker")

    @classmethod
    def begin(cls, leg):
        if cls.state is not None and leg is not None:
            cls._launch(cls.ids.setdefault(leg, 3 + len(cls.ids)))

    @classmethod
    def end(cls, leg):
        if cls.state is not None and leg is not None:
            cls._launch(1)


def time_kernel(fn, reps, prep=None, leg=None):
    """Average / min milliseconds of fn() over reps, measured with events on the current stream
    (the stream the library launches on).  prep() runs untimed before each rep.  leg: the name
    the measurement goes by in a profile (see LegMarks)."""
    times = []
    for _ in range(reps):
        if prep is not None:
            prep()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        LegMarks.begin(leg)
        e0.record()
        fn()
        e1.record()
        LegMarks.end(leg)
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    return float(np.mean(times)), float(np.min(times))


def build_map(keys, values, capacity, device):
    from doksparse_amd import CudaClosedHashmap
    hm = CudaClosedHashmap(n_buckets=capacity, device=device, rehash_threshold=1.0, seed=12345)
    hm.set(keys[:, None], values[:, None])
    return hm


def raw_calls(hm):
    """Closures that launch the get / set / clear kernels through the C ABI on preallocated
    buffers, so that a timed region holds nothing but the kernel."""
    from doksparse_amd import _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    desc = ctypes.byref(hm._desc)
    dev = hm.device

    def get(q, out_v, out_f):
        _lib.check(lib.dok_map_get(desc, q.data_ptr(), q.shape[0], out_v.data_ptr(), None,
                                   out_f.data_ptr(), _stream_ptr(dev)), "get")

    def set_(k, v):
        _lib.check(lib.dok_map_set(desc, k.data_ptr(), v.data_ptr(), k.shape[0], None, _stream_ptr(dev)), "set")

    def clear():
        _lib.check(lib.dok_table_clear(desc, _stream_ptr(dev)), "clear")

    return get, set_, clear


def raw_bulk_set(hm, n, build=False):
    """Closure launching the bulk insert (partition + merge) of n rows on a preallocated
    workspace; None if the library has no bulk path for this table.  build=True: the variant
    that takes the table as uninitialised memory (clear + insert in one pass)."""
    from doksparse_amd import _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    desc = ctypes.byref(hm._desc)
    nbytes = int(lib.dok_bulk_workspace_bytes(desc, n))
    if nbytes <= 0:
        return None
    ws = torch.empty(nbytes, device=hm.device, dtype=torch.uint8)

    fn = lib.dok_map_build_bulk if build else lib.dok_map_set_bulk

    def bulk(k, v):
        _lib.check(fn(desc, k.data_ptr(), v.data_ptr(), k.shape[0], ws.data_ptr(), nbytes,
                      _stream_ptr(hm.device)), "set_bulk")

    return bulk


def cpu_baseline(keys, vals, q, n_hit, seed, what):
    """The reference algorithm (oracle/closed_hashmap_ref.c) on the host cores: set of `keys`
    (unique int64) -> `vals` into a table at load factor 0.5, then get of the batch `q`
    (numpy arrays; n_hit = hits expected in q)."""
    from oracle.ref_hashmap import RefClosedHashmap, _rows
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    n_keys = keys.shape[0]
    ref = RefClosedHashmap(n_buckets=2 * n_keys, rehash_threshold=1.0, rng=np.random.default_rng(seed + 1),
                           n_threads=cores)
    ref._allocate(keys[:, None], vals[:, None])
    ref._keys.fill(0)          # touch the pages before timing
    ref._values.fill(0)
    kr, vr, qr = _rows(keys[:, None]), _rows(vals[:, None]), _rows(q[:, None])
    t0 = time.perf_counter()
    ref._kernel_set(kr, vr)
    t_set = time.perf_counter() - t0
    best_get = 1e30
    for _ in range(3):
        t0 = time.perf_counter()
        _, found = ref._kernel_get(qr)
        best_get = min(best_get, time.perf_counter() - t0)
    assert abs(int(found.sum()) - n_hit) <= 64, "oracle get disagrees with the workload"
    return {
        "value": round(q.shape[0] / best_get / 1e6, 2),
        "unit": "Mops/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{what}: {n_keys} unique int64 keys -> f32 at load factor 0.5 (a "
                  f"{round(2 * n_keys * 20 / 1e9, 2)} GB host table), get of {q.shape[0]} queries "
                  f"(50% Zipf(1.1) hits, 50% misses), best of 3; set of the same keys "
                  f"{round(n_keys / t_set / 1e6, 2)} Mops/s",
        "set_mops": round(n_keys / t_set / 1e6, 2),
    }


def timed(fn, leg=None):
    """Milliseconds of fn() (everything it enqueues on the current stream), by events."""
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    LegMarks.begin(leg)
    e0.record()
    out = fn()
    e1.record()
    LegMarks.end(leg)
    e1.synchronize()
    return e0.elapsed_time(e1), out


def other_configs(device):
    """Timings of the four non-headline configurations (API level, inputs resident in HBM)."""
    from doksparse_amd import CudaClosedHashmap, SparseDOKTensor
    res = {}
    gen = torch.Generator(device=device)

    def uniq_lin(n, volume):
        lin = torch.unique(torch.randint(0, volume, (n,), generator=gen, device=device))
        return lin[torch.randperm(lin.numel(), generator=gen, device=device)]

    # cfg1: 65,536 int64 keys -> int64, capacity 131,072
    gen.manual_seed(1001)
    k = make_unique_keys(131072, gen, device)
    v = torch.randint(-2**62, 2**62, (65536, 1), generator=gen, device=device)
    # (the configuration's set is the first large one of a map; one call is a few tens of
    # microseconds, so it is taken as the best of five maps)
    k1 = k[:65536, None]
    best = None
    for _ in range(5):
        hm = CudaClosedHashmap(n_buckets=131072, device=device)
        hm.set(k[:8, None], v[:8]); hm.get(k[:8, None]); hm.remove(k[:8, None])   # warm-up (allocation, first launches)
        ms = timed(lambda: hm.set(k1, v), leg="cfg1_set_65536")[0]
        best = ms if best is None else min(best, ms)
    res["cfg1_set_ms"] = round(best, 4)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(50):
        hm.set(k[:65536, None], v)
    res["cfg1_set_host_us_per_call"] = round((time.perf_counter() - t0) / 50 * 1e6, 1)
    torch.cuda.synchronize()
    hm.get(k[:, None])                  # (the first call of a size pays for the allocation of its outputs)
    res["cfg1_get_ms"] = round(timed(lambda: hm.get(k[:, None]), leg="cfg1_get_131072")[0], 4)
    res["cfg1_remove_ms"] = round(timed(lambda: hm._remove_rows(k[:32768, None].contiguous(), unique=True), leg="cfg1_remove_32768")[0], 4)

    # cfg2: 1M float32[3] keys -> int64[5], capacity 2^21 (tagged layout)
    gen.manual_seed(1002)
    k2 = torch.rand(1_000_000, 3, generator=gen, device=device)
    v2 = torch.randint(0, 2**63 - 1, (1_000_000, 5), generator=gen, device=device)
    q2 = torch.cat([k2, torch.rand(1_000_000, 3, generator=gen, device=device) + 1.0])
    # warm-up on a map of its own (first launches; its table and workspace go back to torch's caching
    # allocator), then the configuration's batch as the first `set` of a new map - which is how the
    # configuration states it - and once more as an upsert of the same keys
    warm = CudaClosedHashmap(n_buckets=2**21, device=device)
    warm.set(k2, v2); warm.get(k2[:8]); warm._remove_rows(k2[:8].contiguous()); warm.set(k2[:8], v2[:8])
    del warm
    best = None
    for _ in range(3):                  # (best of three new maps, like configuration 1's first set)
        hm2 = CudaClosedHashmap(n_buckets=2**21, device=device)
        ms = timed(lambda: hm2.set(k2, v2), leg="cfg2_set_1M_f32x3_i64x5")[0]
        best = ms if best is None else min(best, ms)
        assert hm2.n_elements == 1_000_000
    res["cfg2_set_ms"] = round(best, 4)
    res["cfg2_upsert_ms"] = round(timed(lambda: hm2.set(k2, v2), leg="cfg2_upsert_1M")[0], 4)
    hm2.get(q2)
    res["cfg2_get_ms"] = round(timed(lambda: hm2.get(q2), leg="cfg2_get_2M")[0], 4)
    res["cfg2_remove_ms"] = round(timed(lambda: hm2._remove_rows(k2[:250_000].contiguous(), unique=True), leg="cfg2_remove_250K")[0], 4)
    del hm, hm2, k2, v2, q2

    # cfg4: 2-D 1e6 x 1e6 float32, 50M entries
    gen.manual_seed(1004)
    lin = uniq_lin(50_000_000, 10**12)
    coords = torch.stack([lin // 10**6, lin % 10**6])
    vals = torch.randn(lin.numel(), generator=gen, device=device)
    # (a first construction is made and dropped, so that the timed one takes its table and workspace
    # from torch's caching allocator instead of hipMalloc: allocation is not part of the path)
    del_me = SparseDOKTensor((10**6, 10**6), coords, vals, device=device)
    del del_me
    ms, dok = timed(lambda: SparseDOKTensor((10**6, 10**6), coords, vals, device=device), leg="cfg4_construct_50M")
    res["cfg4_construct_50M_ms"] = round(ms, 3)
    res["cfg4_entries"] = int(lin.numel())
    rows = torch.randint(0, 10**6, (4096, 1), generator=gen, device=device)
    cols = torch.randint(0, 10**6, (1, 256), generator=gen, device=device)
    dok[rows, cols]
    res["cfg4_getitem_4096x256_ms"] = round(min(timed(lambda: dok[rows, cols], leg="cfg4_getitem_4096x256")[0] for _ in range(5)), 4)
    sc = torch.cat([coords[:, :5_000_000], torch.randint(0, 10**6, (2, 5_000_000), generator=gen, device=device)], dim=1)
    sv = torch.randn(sc.shape[1], generator=gen, device=device)
    def scatter():
        dok[sc[0], sc[1]] = sv
    res["cfg4_setitem_10M_ms"] = round(timed(scatter, leg="cfg4_setitem_10M_with_growth")[0], 3)           # includes the growth to 120M slots
    res["cfg4_setitem_10M_again_ms"] = round(timed(scatter, leg="cfg4_setitem_10M_overwrite")[0], 3)     # all overwrites, no growth
    res["cfg4_readout_ms"] = round(timed(lambda: dok.storage().items(), leg="cfg4_readout")[0], 3)
    del dok, coords, vals, lin, sc, sv

    # cfg5: 4-D (4096, 4096, 64, 8) float16, 100M entries at load factor 0.85
    gen.manual_seed(1005)
    size, strides = (4096, 4096, 64, 8), (4096 * 64 * 8, 64 * 8, 8, 1)
    lin = uniq_lin(100_000_000, 2**33)
    coords = torch.stack([(lin // st) % s for st, s in zip(strides, size)])
    vals = torch.randn(lin.numel(), generator=gen, device=device).half()
    def new_store():
        return CudaClosedHashmap(n_buckets=int(np.ceil(lin.numel() / 0.85)), device=device, rehash_threshold=0.9,
                                 coord_dims=size)
    del_me = SparseDOKTensor(size, coords, vals, device=device, storage=new_store())    # (as for cfg4)
    del del_me
    store = new_store()
    ms, dok = timed(lambda: SparseDOKTensor(size, coords, vals, device=device, storage=store), leg="cfg5_construct_100M")
    res["cfg5_construct_100M_ms"] = round(ms, 3)
    res["cfg5_entries"] = int(lin.numel())
    i_list = torch.randint(0, 4096, (64,), generator=gen, device=device).tolist()
    idx = torch.randint(0, 64, (128, 1), generator=gen, device=device)
    mask = torch.tensor([True, False, True, True, False, False, True, False], device=device)
    def gets():
        for i in i_list:
            dok[i, :512, idx, mask]
    gets()
    res["cfg5_lookups_per_64_getitems"] = 64 * 512 * 128 * int(mask.sum().item())
    res["cfg5_64_getitems_ms"] = round(timed(gets, leg="cfg5_64_getitems")[0], 3)
    # the host's share: time to enqueue the 64 calls (selector normalisation, descriptor, launch),
    # without waiting for the GPU
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    gets()
    res["cfg5_64_getitems_host_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
    torch.cuda.synchronize()
    n_gone = lin.numel() // 5
    gone = coords[:, :n_gone].T.contiguous()
    # (`del storage[keys]`: no per-row flags asked for, so the partitioned removal runs)
    res["cfg5_remove_20M_ms"] = round(timed(lambda: dok.storage().__delitem__(gone), leg="cfg5_remove_20M")[0], 3)
    fresh = torch.stack([torch.randint(0, s, (n_gone,), generator=gen, device=device) for s in size], dim=1)
    fv = torch.randn(n_gone, 1, generator=gen, device=device).half()
    res["cfg5_reinsert_20M_ms"] = round(timed(lambda: dok.storage().set(fresh, fv), leg="cfg5_reinsert_20M")[0], 3)
    res["cfg5_64_getitems_after_churn_ms"] = round(timed(gets)[0], 3)
    return res


def tagged_scale(device, n=32_000_000):
    """The tagged layout (keys / values wider than 8 bytes) at scale: n float32[3] keys -> int64[5]
    values, the row shape of the reference README's hashmap example, at load factors 0.5 and 0.75.
    Kernel-level timings through the C ABI on preallocated buffers."""
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    res = {}
    gen = torch.Generator(device=device)
    gen.manual_seed(1002)
    k = torch.rand(n, 3, generator=gen, device=device)
    v = torch.randint(0, 2**63 - 1, (n, 5), generator=gen, device=device)
    q = torch.cat([k[: n // 2], torch.rand(n - n // 2, 3, generator=gen, device=device) + 1.0])
    q = q[torch.randperm(n, generator=gen, device=device)].contiguous()
    out_v = torch.empty(n, 5, device=device, dtype=torch.long)
    out_f = torch.empty(n, device=device, dtype=torch.bool)
    quarter = k[: n // 4].contiguous()
    stream = _stream_ptr(device)
    for lf, tag in ((0.5, "lf05"), (0.75, "lf075")):
        hm = CudaClosedHashmap(n_buckets=int(n / lf), device=device, rehash_threshold=1.0, seed=4242)
        hm.set(k[:8], v[:8])
        desc = ctypes.byref(hm._desc)
        clear = lambda: _lib.check(lib.dok_table_clear(desc, stream), "clear")
        set_ = lambda: _lib.check(lib.dok_map_set(desc, k.data_ptr(), v.data_ptr(), n, None, stream), "set")
        get = lambda: _lib.check(lib.dok_map_get(desc, q.data_ptr(), n, out_v.data_ptr(), None,
                                                 out_f.data_ptr(), stream), "get")
        rem = lambda: _lib.check(lib.dok_map_remove_unique(desc, quarter.data_ptr(), n // 4, out_f.data_ptr(), stream), "remove")
        s_avg, _ = time_kernel(set_, 3, prep=clear, leg=f"tagged_set_{tag}")
        assert hm.n_elements == n
        # the same rows as the first batch of a new map takes them: clear + insert with one
        # compare-and-swap per row, in one call (dok_map_build_bulk)
        nws = int(lib.dok_bulk_workspace_bytes(desc, n))
        ws = torch.empty(nws, device=device, dtype=torch.uint8)
        build = lambda: _lib.check(lib.dok_map_build_bulk(desc, k.data_ptr(), v.data_ptr(), n, ws.data_ptr(), nws, stream), "build")
        b_avg, _ = time_kernel(build, 3, leg=f"tagged_build_{tag}")
        assert hm.n_elements == n
        del ws
        o_avg, _ = time_kernel(set_, 3, leg=f"tagged_overwrite_{tag}")
        get()
        assert int(out_f.sum().item()) == n // 2
        g_avg, _ = time_kernel(get, 5, leg=f"tagged_get_{tag}")
        probe = hm.probe_stats(q)
        r_avg, _ = time_kernel(rem, 1, leg=f"tagged_remove_{tag}")
        assert hm.n_elements == n - n // 4
        res[f"tagged_build_mops_{tag}"] = round(n / b_avg / 1e3, 1)
        for nm, ms in (("set", s_avg), ("build", b_avg), ("overwrite", o_avg), ("get", g_avg), ("remove", r_avg)):
            res[f"tagged_{nm}_ms_{tag}"] = round(ms, 4)
        res[f"tagged_set_mops_{tag}"] = round(n / s_avg / 1e3, 1)
        res[f"tagged_overwrite_mops_{tag}"] = round(n / o_avg / 1e3, 1)
        res[f"tagged_get_mops_{tag}"] = round(n / g_avg / 1e3, 1)
        res[f"tagged_remove_mops_{tag}"] = round((n // 4) / r_avg / 1e3, 1)
        res[f"tagged_probe_len_{tag}"] = round(probe, 4)
        res[f"tagged_table_bytes_{tag}"] = hm._n_phys * 128
        del hm
    res["tagged_keys"] = n
    return res


def dok_scale(device):
    """The DOK indexing kernels at scale, kernel-level through the C ABI on preallocated buffers:
    a 2-D 1e6 x 1e6 float32 tensor of 50M entries (the fourth benchmark configuration); gather of 2^26
    stored coordinates through `__getitem__`'s kernel, scatter of 10M coordinates (half present,
    half new) through `__setitem__`'s, and the read-out of all entries."""
    from doksparse_amd import SparseDOKTensor, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    res = {}
    gen = torch.Generator(device=device)
    gen.manual_seed(1004)
    lin = torch.unique(torch.randint(0, 10**12, (50_000_000,), generator=gen, device=device))
    lin = lin[torch.randperm(lin.numel(), generator=gen, device=device)]
    coords = torch.stack([lin // 10**6, lin % 10**6])
    vals = torch.randn(lin.numel(), generator=gen, device=device)
    dok = SparseDOKTensor((10**6, 10**6), coords, vals, device=device)
    hm = dok.storage()
    hm.rehash(120_000_000)                       # room for the scatter below without a growth
    nnz = hm.n_elements
    stream = _stream_ptr(device)
    # gather: 2^26 stored coordinates, in random order
    n_g = 1 << 26
    pick = torch.randint(0, lin.numel(), (n_g,), generator=gen, device=device)
    r, c = coords[0][pick].contiguous(), coords[1][pick].contiguous()
    plan, keep = dok._plan((r, c))
    ix = plan.ix
    out = torch.empty(n_g, device=device, dtype=torch.float32)
    gather = lambda: _lib.check(lib.dok_getitem_dense(ctypes.byref(hm._desc), ctypes.byref(ix), out.data_ptr(), stream), "getitem")
    gather()
    assert torch.equal(out, vals[pick])
    g_avg, _ = time_kernel(gather, 5, leg="dok_getitem_2p26")
    res["dok_getitem_2p26_ms"] = round(g_avg, 4)
    res["dok_getitem_2p26_mops"] = round(n_g / g_avg / 1e3, 1)
    del pick, r, c, out, ix, keep, plan
    # scatter: 5M present + 5M new coordinates
    sc = torch.cat([coords[:, :5_000_000], torch.randint(0, 10**6, (2, 5_000_000), generator=gen, device=device)], dim=1)
    sc = sc[:, torch.randperm(sc.shape[1], generator=gen, device=device)].contiguous()
    sv = torch.randn(sc.shape[1], generator=gen, device=device)
    plan, keep = dok._plan((sc[0], sc[1]))
    ix = plan.ix
    view = _lib.DokView()
    view.data = sv.data_ptr()
    view.strides[0] = 1
    scatter = lambda: _lib.check(lib.dok_setitem_dense(ctypes.byref(hm._desc), ctypes.byref(ix), ctypes.byref(view), stream), "setitem")
    s_first, _ = timed(scatter, leg="dok_setitem_10M")    # half of the rows are new
    s_avg, _ = time_kernel(scatter, 3, leg="dok_setitem_10M_overwrite")            # every row present
    res["dok_setitem_10M_ms"] = round(s_first, 4)
    res["dok_setitem_10M_overwrite_ms"] = round(s_avg, 4)
    assert hm.n_elements > nnz
    # read-out of every entry as [ndim, nnz] coordinates + values
    ro, _ = timed(lambda: hm.items_coo())
    ro, _ = timed(lambda: hm.items_coo(), leg="dok_readout")
    res["dok_readout_ms"] = round(ro, 4)
    res["dok_entries"] = hm.n_elements
    del dok, hm, coords, vals, lin, sc, sv, ix, keep, plan
    torch.cuda.empty_cache()
    res.update(dok_wide_scale(device))
    return res


def gather_scale(device, n):
    """Uniformly random, naturally aligned granules of 128, 64 and 32 bytes of the default workload's
    load-factor-0.5 table (n keys, 13.4M buckets = 1.72 GB at n = 2^26), n granules per launch: what
    a lookup could cost at most if a probe needed only half or a quarter of a bucket line."""
    from doksparse_amd import _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    gen = torch.Generator(device=device)
    gen.manual_seed(1003)
    keys = make_unique_keys(n, gen, device)
    values = torch.randn(n, generator=gen, device=device, dtype=torch.float32)
    hm = build_map(keys, values, 2 * n, device)
    out = torch.empty(n, device=device, dtype=torch.int32)
    res = {"gather_table_bytes": hm._n_phys * 128, "gather_granules_per_launch": n}
    for gb in (128, 64, 32):
        fn = lambda: _lib.check(lib.dok_line_gather_granule(ctypes.byref(hm._desc), n, 12345, gb, out.data_ptr(),
                                                            _stream_ptr(device)), "gather")
        fn()
        avg, _ = time_kernel(fn, 10, leg=f"gather_{gb}B")
        res[f"gather_{gb}B_ms"] = round(avg, 4)
        res[f"gather_{gb}B_ggranules_s"] = round(n / avg / 1e6, 2)
        res[f"gather_{gb}B_payload_gbs"] = round(n * gb / avg / 1e6, 1)
    return res


def dok_wide_scale(device, nnz=10_000_000, n_q=1 << 22):
    """A tensor whose coordinates do not fit one 8-byte key, (2^40, 2^40), beside one of the same
    content whose do, (2^20, 2^20): the same 10M entries (the small tensor's coordinates, spread
    over 2^40 by a shift), construction, gather of 4M elements (half stored) and scatter of 4M
    (half present, half new; no growth), through the Python API, best of 3."""
    from doksparse_amd import SparseDOKTensor
    res = {}
    gen = torch.Generator(device=device)
    gen.manual_seed(4040)
    lin = torch.unique(torch.randint(0, 2**40, (nnz,), generator=gen, device=device))
    lin = lin[torch.randperm(lin.numel(), generator=gen, device=device)]
    small = torch.stack([lin >> 20, lin & 0xFFFFF])
    vals = torch.randn(lin.numel(), generator=gen, device=device)
    qs = torch.cat([small[:, : n_q // 2], torch.randint(0, 2**20, (2, n_q // 2), generator=gen, device=device)], dim=1)
    qs = qs[:, torch.randperm(n_q, generator=gen, device=device)].contiguous()
    sv = torch.randn(n_q, generator=gen, device=device)
    for tag, size, shift in (("dok_lin", (2**20, 2**20), 0), ("dok_wide", (2**40, 2**40), 20)):
        coords, q = (small << shift).contiguous(), (qs << shift).contiguous()
        best = {"construct": 1e9, "getitem": 1e9, "setitem": 1e9}
        for _ in range(3):
            ms, dok = timed(lambda: SparseDOKTensor(size, coords, vals, device=device), leg=f"{tag}_construct_10M")
            best["construct"] = min(best["construct"], ms)
            dok.storage().rehash(4 * lin.numel())          # room for the scatter: no growth inside the timed call
            got = dok[q[0], q[1]]
            best["getitem"] = min(best["getitem"], timed(lambda: dok[q[0], q[1]], leg=f"{tag}_getitem_4M")[0])
            def scatter():
                dok[q[0], q[1]] = sv
            best["setitem"] = min(best["setitem"], timed(scatter, leg=f"{tag}_setitem_4M")[0])
            # (a coordinate the random half happens to hold twice keeps either of its two values)
            assert int((dok[q[0], q[1]] != sv).sum().item()) <= 16
            del dok
        assert int((got != 0).sum().item()) >= n_q // 2
        res[f"{tag}_construct_10M_ms"] = round(best["construct"], 4)
        res[f"{tag}_getitem_4M_ms"] = round(best["getitem"], 4)
        res[f"{tag}_setitem_4M_ms"] = round(best["setitem"], 4)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--keys", type=int, default=1 << 26, help="stored keys and queries per batch")
    ap.add_argument("--cpu-keys", type=int, default=1 << 26,
                    help="keys of the CPU baseline (default: the full configuration, a 2.7 GB host table)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--quick", action="store_true", help="skip the set and load-factor-0.9 legs")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the four non-headline configurations, the multi-word layout at 32M keys and "
                         "the DOK indexing kernels at scale (all reported under roofline.other_legs / extra)")
    ap.add_argument("--configs", action="store_true", help="(kept for old command lines: these legs now always run)")
    ap.add_argument("--tagged", action="store_true", help="(kept for old command lines: this leg now always runs)")
    ap.add_argument("--only-tagged", action="store_true",
                    help="run nothing but the --tagged leg and print its figures (for profiling that leg)")
    ap.add_argument("--only-gather", action="store_true",
                    help="run nothing but the random-granule gather (128, 64 and 32 bytes) over the "
                         "load-factor-0.5 table of the default workload, and print its rates")
    ap.add_argument("--only-wide", action="store_true",
                    help="run nothing but the wide-tensor legs of --only-dok")
    ap.add_argument("--only-dok", action="store_true",
                    help="run nothing but the DOK indexing kernels at scale and print their figures (for profiling)")
    ap.add_argument("--markers", action="store_true",
                    help="profiling runs: bracket every measured leg with marker launches (see LegMarks) and "
                         "print the leg numbers at the end")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one read-only pass over the whole table (the live-entry count of "
                         "the read-out path); with the table clear that every run does, this gives "
                         "a profiler a read kernel and a write kernel of known size")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the hashmap path has no multi-GPU leg in this build "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.markers:
        import atexit
        LegMarks.enable(device)
        atexit.register(lambda: print(json.dumps({"leg_ids": LegMarks.ids}), file=sys.stderr, flush=True))
    if args.only_tagged:
        print(json.dumps({"extra": tagged_scale(device)}), flush=True)
        return
    if args.only_gather:
        print(json.dumps({"extra": gather_scale(device, args.keys)}), flush=True)
        return
    if args.only_wide:
        print(json.dumps({"extra": dok_wide_scale(device)}), flush=True)
        return
    if args.only_dok:
        print(json.dumps({"extra": dok_scale(device)}), flush=True)
        return
    n = args.keys
    gen = torch.Generator(device=device)
    gen.manual_seed(1003)
    keys = make_unique_keys(n, gen, device)
    values = torch.randn(n, generator=gen, device=device, dtype=torch.float32)
    queries, n_hit = make_queries(keys, n, gen, device)

    cap05 = 2 * n
    cap09 = int(np.ceil(n / 0.9))
    results = {}

    # ---------------- load factor 0.5: the timed steps -------------------------------------
    hm = build_map(keys, values, cap05, device)
    assert hm.n_elements == n
    out_v = torch.empty(n, 1, device=device, dtype=torch.float32)
    out_f = torch.empty(n, device=device, dtype=torch.bool)
    raw_get, raw_set, raw_clear = raw_calls(hm)

    # correctness gate before any timing: hits return their value, misses are misses.  The value
    # check goes through the *_stats entry point, a separate kernel instantiation, so that a
    # profiler's per-kernel average of the plain get kernel covers identical launches only.
    v, f = hm.get(queries[:, None])
    assert int(f.sum().item()) == n_hit, "unexpected hit count"
    chk = keys[torch.randperm(n, generator=gen, device=device)[: 1 << 20]].contiguous()
    vv = torch.empty(chk.shape[0], 1, device=device, dtype=torch.float32)
    ff = torch.empty(chk.shape[0], device=device, dtype=torch.bool)
    from doksparse_amd import _lib as _dl
    from doksparse_amd.closed_hashmap import _stream_ptr
    _dl.check(_dl.load().dok_map_get_stats(ctypes.byref(hm._desc), chk.data_ptr(), chk.shape[0], vv.data_ptr(),
                                           None, ff.data_ptr(), _stream_ptr(device)), "get_stats")
    vref, _ = hm.get(queries[:, None])          # same launch as the timed one; determinism check
    assert bool(ff.all()) and torch.equal(v, vref)
    idx = torch.searchsorted(torch.sort(keys).values, chk)      # independent of the table: sorted lookup
    assert torch.equal(torch.sort(keys).values[idx], chk)
    order = torch.argsort(keys)
    assert torch.equal(vv[:, 0], values[order[idx]]), "get returned a wrong value"
    chk_expect = vv.clone()
    del v, f, vv, ff, vref, idx, order

    for _ in range(args.warmup):
        hm.get(queries[:, None])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        hm.get(queries[:, None])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    get_mops = n / (ms_per_step * 1e-3) / 1e6

    # kernel-only duration for the roofline
    k_avg, k_min = time_kernel(lambda: raw_get(queries, out_v, out_f), max(args.steps, 5), leg="get_lf05")
    results["get_kernel_ms_lf05"] = round(k_avg, 4)
    results["get_mops_lf05"] = round(n / k_avg / 1e3, 1)
    results["probe_len_lf05"] = round(hm.probe_stats(queries[:, None]), 4)
    results["table_bytes_lf05"] = hm._n_phys * 128
    # practical ceiling: uniformly random 128-byte line gathers over the same bucket array
    chk32 = torch.empty(n, device=device, dtype=torch.int32)
    def line_gather():
        _dl.check(_dl.load().dok_line_gather(ctypes.byref(hm._desc), n, 12345, chk32.data_ptr(),
                                             _stream_ptr(device)), "line_gather")
    line_gather()
    lg_avg, _ = time_kernel(line_gather, 5, leg="line_gather_lf05")
    results["line_gather_glines_s_lf05"] = round(n / lg_avg / 1e6, 2)
    results["line_gather_gbs_lf05"] = round(n * 128 / lg_avg / 1e6, 1)
    del chk32
    if args.calibrate:
        hm._compact(False, False)

    cpu = None
    if not args.no_cpu:
        # the CPU baseline runs on the very arrays the GPU legs use (or, with --cpu-keys below the
        # batch size, on a sample: the first keys and a batch drawn the same way over them)
        m = min(args.cpu_keys, n)
        if m == n:
            hk, hv, hq, hh = keys.cpu().numpy(), values.cpu().numpy(), queries.cpu().numpy(), n_hit
            what = "the benchmark's own keys and query batch"
        else:
            sub_q, hh = make_queries(keys[:m], m, gen, device)
            hk, hv, hq = keys[:m].cpu().numpy(), values[:m].cpu().numpy(), sub_q.cpu().numpy()
            del sub_q
            what = f"a sample (--cpu-keys {m}) of the benchmark's keys with a batch drawn the same way"
        cpu = cpu_baseline(hk, hv, hq, hh, 1003, what)
        del hk, hv, hq

    if not args.quick:
        # set of all n keys into the cleared table: the per-row compare-and-swap kernel, and the
        # bulk path (partition by table range + merge in LDS) that CudaClosedHashmap.set picks
        # for a batch of this size
        s_avg, s_min = time_kernel(lambda: raw_set(keys, values), 5, prep=raw_clear, leg="set_cas_lf05")
        results["set_cas_kernel_ms_lf05"] = round(s_avg, 4)
        results["set_cas_mops_lf05"] = round(n / s_avg / 1e3, 1)
        assert hm.n_elements == n
        bulk = raw_bulk_set(hm, n)
        if bulk is not None:
            raw_clear(); bulk(keys, values)
            assert hm.n_elements == n
            vv = torch.empty(chk.shape[0], 1, device=device, dtype=torch.float32)
            ff = torch.empty(chk.shape[0], device=device, dtype=torch.bool)
            _dl.check(_dl.load().dok_map_get_stats(ctypes.byref(hm._desc), chk.data_ptr(), chk.shape[0],
                                                   vv.data_ptr(), None, ff.data_ptr(), _stream_ptr(device)), "get_stats")
            assert bool(ff.all()) and torch.equal(vv, chk_expect), "bulk insert stored a wrong value"
            del vv, ff
            b_avg, _ = time_kernel(lambda: bulk(keys, values), 5, prep=raw_clear, leg="set_bulk_lf05")
            results["set_bulk_ms_lf05"] = round(b_avg, 4)
            s_avg = min(s_avg, b_avg)
            # the same rows into a table taken as uninitialised memory (what the first set of a
            # new map and a rehash run): no clear before, no read of the table
            del bulk
            bulk = raw_bulk_set(hm, n, build=True)
            bulk(keys, values)
            assert hm.n_elements == n
            bb_avg, _ = time_kernel(lambda: bulk(keys, values), 5, leg="build_lf05")
            results["build_ms_lf05"] = round(bb_avg, 4)
            results["build_mops_lf05"] = round(n / bb_avg / 1e3, 1)
        results["set_ms_lf05"] = round(s_avg, 4)
        results["set_mops_lf05"] = round(n / s_avg / 1e3, 1)
        assert hm.n_elements == n
        del bulk
        # overwrite pass (every key present)
        o_avg, _ = time_kernel(lambda: raw_set(keys, values), 5, leg="overwrite_cas_lf05")
        results["overwrite_mops_lf05"] = round(n / o_avg / 1e3, 1)
        # the same overwrite as `set` runs it when the table is too full to skip the growth check:
        # one pass that overwrites present keys and counts absent ones (none here)
        miss = torch.zeros((), device=device, dtype=torch.long)
        def raw_update():
            _dl.check(_dl.load().dok_map_update_existing(ctypes.byref(hm._desc), keys.data_ptr(), values.data_ptr(), n,
                                                         miss.data_ptr(), _stream_ptr(device)), "update")
        raw_update()
        assert int(miss.item()) == 0
        u_avg, _ = time_kernel(raw_update, 5, leg="update_existing_lf05")
        results["update_existing_ms_lf05"] = round(u_avg, 4)
        results["update_existing_mops_lf05"] = round(n / u_avg / 1e3, 1)
        # remove of a random half of the keys (the keys are in random order); the removed rows
        # are stored again outside the timed region
        half = keys[: n // 2]
        rem_f = torch.empty(n // 2, device=device, dtype=torch.uint8)
        def raw_remove():
            # (the keys are distinct: the variant CudaClosedHashmap.remove runs after its unique)
            _dl.check(_dl.load().dok_map_remove_unique(ctypes.byref(hm._desc), half.data_ptr(), n // 2,
                                                       rem_f.data_ptr(), _stream_ptr(device)), "remove")
        raw_remove()
        assert bool(rem_f.all()) and hm.n_elements == n - n // 2
        r_avg, _ = time_kernel(raw_remove, 5, prep=lambda: raw_set(half, values[: n // 2]), leg="remove_lf05")
        results["remove_ms_lf05"] = round(r_avg, 4)
        results["remove_mops_lf05"] = round((n // 2) / r_avg / 1e3, 1)
        def raw_remove_cas():                  # any batch, equal keys allowed: one compare-and-swap per row
            _dl.check(_dl.load().dok_map_remove(ctypes.byref(hm._desc), half.data_ptr(), n // 2, rem_f.data_ptr(),
                                                _stream_ptr(device)), "remove")
        rc_avg, _ = time_kernel(raw_remove_cas, 3, prep=lambda: raw_set(half, values[: n // 2]), leg="remove_cas_lf05")
        results["remove_cas_mops_lf05"] = round((n // 2) / rc_avg / 1e3, 1)
        # the same removal without per-row flags, partitioned by table range (what `del map[keys]` runs)
        nws = int(_dl.load().dok_bulk_workspace_bytes(ctypes.byref(hm._desc), n // 2))
        if nws > 0:
            rws = torch.empty(nws, device=device, dtype=torch.uint8)
            def raw_remove_bulk():
                _dl.check(_dl.load().dok_map_remove_bulk(ctypes.byref(hm._desc), half.data_ptr(), n // 2, rws.data_ptr(),
                                                         nws, _stream_ptr(device)), "remove_bulk")
            raw_set(half, values[: n // 2]); raw_remove_bulk()
            assert hm.n_elements == n - n // 2
            rb_avg, _ = time_kernel(raw_remove_bulk, 5, prep=lambda: raw_set(half, values[: n // 2]), leg="remove_bulk_lf05")
            results["remove_bulk_ms_lf05"] = round(rb_avg, 4)
            results["remove_bulk_mops_lf05"] = round((n // 2) / rb_avg / 1e3, 1)
            del rws
        del half, rem_f
        del hm
        torch.cuda.empty_cache()

        # ---------------- load factor 0.9 ---------------------------------------------------
        # Which keys end up away from their home bucket depends on the order in which the rows of a
        # build arrive (atomic reservations), and the hottest key of the Zipf batch alone is 5 % of
        # the queries: the table is therefore built four times and the get figures are means over
        # the builds (the spread is reported beside them).
        g9s, p9s = [], []
        for rep in range(4):
            hm9 = build_map(keys, values, cap09, device)
            assert hm9.n_elements == n
            raw_get9, raw_set9, raw_clear9 = raw_calls(hm9)
            if rep == 0:
                v, f = hm9.get(queries[:, None])
                assert int(f.sum().item()) == n_hit
                del v, f
            g9s.append(time_kernel(lambda: raw_get9(queries, out_v, out_f), 5, leg="get_lf09")[0])
            p9s.append(hm9.probe_stats(queries[:, None]))
            if rep < 3:
                del hm9, raw_get9, raw_set9, raw_clear9
        g9 = float(np.mean(g9s))
        results["get_kernel_ms_lf09_builds"] = [round(x, 4) for x in g9s]
        results["probe_len_lf09_builds"] = [round(x, 4) for x in p9s]
        s9, _ = time_kernel(lambda: raw_set9(keys, values), 3, prep=raw_clear9, leg="set_cas_lf09")
        results["set_cas_mops_lf09"] = round(n / s9 / 1e3, 1)
        bulk9 = raw_bulk_set(hm9, n)
        if bulk9 is not None:
            b9, _ = time_kernel(lambda: bulk9(keys, values), 3, prep=raw_clear9, leg="set_bulk_lf09")
            assert hm9.n_elements == n
            results["set_bulk_ms_lf09"] = round(b9, 4)
            s9 = min(s9, b9)
            del bulk9
            bulk9 = raw_bulk_set(hm9, n, build=True)
            bb9, _ = time_kernel(lambda: bulk9(keys, values), 3, leg="build_lf09")
            assert hm9.n_elements == n
            results["build_ms_lf09"] = round(bb9, 4)
        del bulk9
        results["get_kernel_ms_lf09"] = round(g9, 4)
        results["get_mops_lf09"] = round(n / g9 / 1e3, 1)
        results["set_mops_lf09"] = round(n / s9 / 1e3, 1)
        results["probe_len_lf09"] = round(float(np.mean(p9s)), 4)
        results["load_factor_09_physical"] = round(n / (hm9._n_phys * hm9._slots_per_bucket), 4)
        del hm9

    default_workload = n == (1 << 26)
    legs = {}
    if not args.headline_only and not args.quick:
        del keys, values, queries, out_v, out_f
        torch.cuda.empty_cache()
        # the other four configurations at API level (host time included): durations only
        cfg = other_configs(device)
        results.update(cfg)
        for name, ms_key, ops in (("cfg1_set_65536", "cfg1_set_ms", 65536), ("cfg1_get_131072", "cfg1_get_ms", 131072),
                                  ("cfg1_remove_32768", "cfg1_remove_ms", 32768),
                                  ("cfg2_set_1M_f32x3_i64x5", "cfg2_set_ms", 1_000_000),
                                  ("cfg2_upsert_1M", "cfg2_upsert_ms", 1_000_000),
                                  ("cfg2_get_2M", "cfg2_get_ms", 2_000_000), ("cfg2_remove_250K", "cfg2_remove_ms", 250_000),
                                  ("cfg4_construct_50M", "cfg4_construct_50M_ms", cfg["cfg4_entries"]),
                                  ("cfg4_getitem_4096x256", "cfg4_getitem_4096x256_ms", 4096 * 256),
                                  ("cfg4_setitem_10M_with_growth", "cfg4_setitem_10M_ms", 10_000_000),
                                  ("cfg4_setitem_10M_overwrite", "cfg4_setitem_10M_again_ms", 10_000_000),
                                  ("cfg4_readout", "cfg4_readout_ms", cfg["cfg4_entries"]),
                                  ("cfg5_construct_100M", "cfg5_construct_100M_ms", cfg["cfg5_entries"]),
                                  ("cfg5_64_getitems", "cfg5_64_getitems_ms", cfg["cfg5_lookups_per_64_getitems"]),
                                  ("cfg5_remove_20M", "cfg5_remove_20M_ms", cfg["cfg5_entries"] // 5),
                                  ("cfg5_reinsert_20M", "cfg5_reinsert_20M_ms", cfg["cfg5_entries"] // 5)):
            # (API level: the time holds the host's share of the call; the bytes are those of every
            # kernel the call launches)
            legs[name] = leg_entry(name, cfg[ms_key], ops, "api")
        torch.cuda.empty_cache()
        # the multi-word layout and the DOK indexing kernels at scale: kernel level, with profiled bytes
        tg = tagged_scale(device)
        results.update(tg)
        nt = tg["tagged_keys"]
        torch.cuda.empty_cache()
        dk = dok_scale(device)
        results.update(dk)
        for name, leg, ms, ops in (
                ("tagged_set_32M_lf05", "tagged_set_lf05", tg["tagged_set_ms_lf05"], nt),
                ("tagged_build_32M_lf05", "tagged_build_lf05", tg["tagged_build_ms_lf05"], nt),
                ("tagged_overwrite_32M_lf05", "tagged_overwrite_lf05", tg["tagged_overwrite_ms_lf05"], nt),
                ("tagged_get_32M_lf05", "tagged_get_lf05", tg["tagged_get_ms_lf05"], nt),
                ("tagged_remove_8M_lf05", "tagged_remove_lf05", tg["tagged_remove_ms_lf05"], nt // 4),
                ("tagged_set_32M_lf075", "tagged_set_lf075", tg["tagged_set_ms_lf075"], nt),
                ("tagged_build_32M_lf075", "tagged_build_lf075", tg["tagged_build_ms_lf075"], nt),
                ("tagged_get_32M_lf075", "tagged_get_lf075", tg["tagged_get_ms_lf075"], nt),
                ("dok_getitem_2p26", "dok_getitem_2p26", dk["dok_getitem_2p26_ms"], 1 << 26),
                ("dok_setitem_10M", "dok_setitem_10M", dk["dok_setitem_10M_ms"], 10_000_000),
                ("dok_setitem_10M_overwrite", "dok_setitem_10M_overwrite", dk["dok_setitem_10M_overwrite_ms"], 10_000_000),
                ("dok_readout_55M", "dok_readout", dk["dok_readout_ms"], dk["dok_entries"]),
                ("dok_lin_2p20x2p20_getitem_4M", "dok_lin_getitem_4M", dk.get("dok_lin_getitem_4M_ms"), 1 << 22),
                ("dok_lin_2p20x2p20_setitem_4M", "dok_lin_setitem_4M", dk.get("dok_lin_setitem_4M_ms"), 1 << 22),
                ("dok_lin_2p20x2p20_construct_10M", "dok_lin_construct_10M", dk.get("dok_lin_construct_10M_ms"), 10_000_000),
                ("dok_wide_2p40x2p40_getitem_4M", "dok_wide_getitem_4M", dk.get("dok_wide_getitem_4M_ms"), 1 << 22),
                ("dok_wide_2p40x2p40_setitem_4M", "dok_wide_setitem_4M", dk.get("dok_wide_setitem_4M_ms"), 1 << 22),
                ("dok_wide_2p40x2p40_construct_10M", "dok_wide_construct_10M", dk.get("dok_wide_construct_10M_ms"), 10_000_000)):
            if ms is None:
                continue
            # (the two construct / getitem / setitem triples of the wide-tensor comparison are API level)
            legs[name] = leg_entry(leg, ms, ops, "api" if leg.startswith(("dok_lin_", "dok_wide_")) else "kernel")

    line_model_gbs = n * B_GET / (k_avg * 1e-3) / 1e9
    m_get = measured("get_lf05", k_avg) if default_workload else None
    # the other legs the metric names, with measured HBM bytes (never a per-op model)
    if default_workload:
        for name, entry, ms_key, ops in (("get_lf09", "get_lf09", "get_kernel_ms_lf09", n),
                                         ("set_lf05", "set_bulk_lf05", "set_bulk_ms_lf05", n),
                                         ("build_lf05", "build_lf05", "build_ms_lf05", n),
                                         ("set_lf09", "set_bulk_lf09", "set_bulk_ms_lf09", n),
                                         ("build_lf09", "build_lf09", "build_ms_lf09", n),
                                         ("set_per_row_lf05", "set_cas_lf05", "set_cas_kernel_ms_lf05", n),
                                         ("update_existing_lf05", "update_existing_lf05", "update_existing_ms_lf05", n),
                                         ("remove_lf05", "remove_lf05", "remove_ms_lf05", n // 2),
                                         ("remove_bulk_lf05", "remove_bulk_lf05", "remove_bulk_ms_lf05", n // 2)):
            ms = results.get(ms_key)
            if ms is not None:
                legs[name] = leg_entry(entry, ms, ops, "kernel")
    line = {
        "metric": "hashmap get/set Mops/s at 64M keys LF 0.5/0.9; achieved HBM GB/s % of peak",
        "value": round(get_mops, 1),
        "unit": "Mops/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int64",
        "data": "synthetic",
        "config": {
            "workload": f"get of {n} queries (50% Zipf(1.1) hits, 50% uniform misses) against {n} "
                        f"unique int64 keys -> float32 values, capacity {cap05} (load factor 0.5)",
            "keys": n, "capacity": cap05, "key_bytes": 8, "value_bytes": 4,
        },
        "roofline": {
            "bound": "hbm",
            # achieved / frac: the bytes that crossed the HBM interface per launch (rocprofv3
            # FETCH_SIZE + WRITE_SIZE, `traffic`) over the kernel's live duration; null when no
            # profile of the current kernel sources exists
            "achieved": m_get and m_get["gbs"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": m_get and m_get["frac"],
            "traffic": m_get and m_get["traffic"],
            "kernel": "p8_get_kernel<4, false, 0>",
            "kernel_ms": round(k_avg, 4),
            # the line-granular model: one 128-byte bucket line per query plus the batch row and the
            # outputs, whether or not the line came from HBM (the Zipf half of the batch is largely
            # cache-resident, so this exceeds what the memory interface carried)
            "model_bytes_per_op": B_GET,
            "line_model_gbs": round(line_model_gbs, 1),
            "frac_line_model": round(line_model_gbs / HBM_PEAK_GBS, 4),
            # what this GPU reaches on uniformly random 128-byte lines of the same table
            "random_line_ceiling_gbs": results.get("line_gather_gbs_lf05"),
            "profiled_csrc_sha16": PROFILED["csrc_sha16"],
            "csrc_sha16": csrc_sha16(),
            "other_legs": legs,
        },
        "extra": results,
    }
    if cpu is not None:
        line["cpu_baseline"] = cpu
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
