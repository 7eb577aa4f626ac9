"""CPU-side checks of the product: helper functions, the C ABI surface, selector handling.
No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from doksparse_amd import CudaClosedHashmap, SparseDOKTensor, _lib
from doksparse_amd.util import (dtype2ctype, get_tensor_accessor_argument_array, next_power_of_2,
                                shape_to_stride, str2dtype)
from oracle.ref_dok import RefSparseDOKTensor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_util_helpers():
    assert [next_power_of_2(n) for n in (0, 1, 2, 3, 4, 5, 1023, 1024, 1025, 50_000_000)] == \
        [1, 1, 2, 4, 4, 8, 1024, 1024, 2048, 2**26]
    for shape in [(7,), (3, 4), (2, 3, 5), (4, 1, 6, 2)]:
        assert shape_to_stride(shape) == torch.empty(shape).stride()
        assert np.unravel_index(17 % int(np.prod(shape)), shape) == tuple(
            (17 % int(np.prod(shape))) // s % d for s, d in zip(shape_to_stride(shape), shape))
    assert shape_to_stride(()) == ()
    assert str2dtype("long") is torch.int64 and str2dtype("half") is torch.float16
    assert str2dtype(torch.float32) is torch.float32
    with pytest.raises(ValueError):
        str2dtype("nope")
    assert dtype2ctype(torch.int64) == "int64_t" and dtype2ctype("float") == "float"
    a = torch.zeros(3, 4, dtype=torch.long)
    b = a.T.contiguous().T
    arr = get_tensor_accessor_argument_array(a, b)
    assert arr.shape == (2, 5)
    assert arr[0].tolist() == [a.data_ptr(), 3, 4, 4, 1] and arr[1].tolist() == [b.data_ptr(), 3, 4, 1, 3]


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "dokhip.h")).read()
    declared = set(re.findall(r"\b(dok_[a-z0-9_]+)\s*\(", header))
    declared -= {"dok_table_t", "dok_view_t", "dok_index_t"}
    assert declared == set(_lib.SIGNATURES), (declared ^ set(_lib.SIGNATURES))
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name


def test_struct_sizes_match_the_header():
    # dok_table_t: 2 pointers + 2 x 8 + 4 x 4 + 14 x 8 bytes; dok_view_t: pointer + 8 + 14 x 8
    assert _lib.DOK_MAX_DIMS == 14
    assert ctypes.sizeof(_lib.DokTable) == 8 + 8 + 8 + 8 + 16 + 14 * 8
    assert ctypes.sizeof(_lib.DokView) == 8 + 8 + 14 * 8
    assert ctypes.sizeof(_lib.DokIndex) == 8 + 14 * 8 + 14 * (8 + 8 + 14 * 8)


def test_layout_selection():
    lib = _lib.load()
    s = ctypes.c_int32()
    expect = {(8, 4): (1, 10), (8, 8): (1, 7), (8, 2): (1, 12), (8, 1): (1, 13), (4, 4): (1, 10),
              (12, 40): (2, 2), (16, 4): (2, 4), (32, 2): (2, 2), (3, 3): (2, 5)}
    for (kb, vb), (layout, slots) in expect.items():
        assert lib.dok_layout_of(kb, vb, ctypes.byref(s)) == layout and s.value == slots
    assert lib.dok_layout_of(64, 64, None) == _lib.DOK_EUNSUPPORTED
    assert lib.dok_layout_of(0, 4, None) == _lib.DOK_EUNSUPPORTED
    assert lib.dok_phys_buckets_for(2**27, 8, 4) == (2**27 + 9) // 10
    assert lib.dok_phys_buckets_for(0, 8, 4) == 1


def test_bad_descriptors_are_rejected_without_a_launch():
    lib = _lib.load()
    t = _lib.DokTable()
    assert lib.dok_table_clear(ctypes.byref(t), None) == _lib.DOK_EINVAL      # null pointers
    t.buckets, t.header, t.n_phys_buckets, t.key_bytes, t.value_bytes = 4096, 8192, 1, 8, 4
    assert lib.dok_map_get(ctypes.byref(t), None, -1, None, None, None, None) == _lib.DOK_EINVAL
    assert lib.dok_map_get(ctypes.byref(t), None, 0, None, None, None, None) == _lib.DOK_OK  # empty batch
    assert lib.dok_map_get(ctypes.byref(t), None, 5, None, None, None, None) == _lib.DOK_EINVAL
    t.buckets = 4100                                                          # not 128-byte aligned
    assert lib.dok_map_set(ctypes.byref(t), 8, 8, 1, None, None) == _lib.DOK_EINVAL
    t.buckets, t.key_bytes, t.value_bytes = 4096, 200, 4
    assert lib.dok_map_set(ctypes.byref(t), 8, 8, 1, None, None) == _lib.DOK_EUNSUPPORTED
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.DOK_EUNSUPPORTED, "x")
    with pytest.raises(AssertionError):
        _lib.check(_lib.DOK_EINVAL, "x")


def test_static_compact_size_check_needs_no_gpu():
    lib = _lib.load()
    assert lib.dok_static_scratch_bytes() == (8 << 20) + 256
    t = _lib.DokTable()
    t.buckets, t.header, t.key_bytes, t.value_bytes = 4096, 8192, 8, 4
    t.n_phys_buckets = 1 << 28                      # the documented limit itself is served
    assert lib.dok_compact_scratch_bytes(ctypes.byref(t)) <= lib.dok_static_scratch_bytes()
    t.n_phys_buckets = (1 << 28) + 256 * 32         # more chunk counters than the scratch holds
    assert lib.dok_compact_scratch_bytes(ctypes.byref(t)) > lib.dok_static_scratch_bytes()
    assert lib.dok_map_compact_static(ctypes.byref(t), None, None, 0, 8, None) == _lib.DOK_ETOOLARGE
    with pytest.raises(ValueError):
        _lib.check(_lib.DOK_ETOOLARGE, "x")


def test_hashmap_before_any_set():
    hm = CudaClosedHashmap(n_buckets=64, device="cpu")
    assert hm.n_buckets == 64 and hm.n_elements == 0 and len(hm) == 0
    assert hm._keys is None and hm._values is None and hm.keys() is None
    assert hm._empty_marker == -1 and hm._removed_marker == -3
    assert (hm._uuid == -1).all() and hm._uuid.shape == (64,)
    with pytest.raises(RuntimeError, match="store something first"):
        hm.get(torch.zeros(1, 1, dtype=torch.long))
    with pytest.raises(RuntimeError, match="store something first"):
        hm.remove(torch.zeros(1, 1, dtype=torch.long))


def test_compat_hash_methods_follow_the_reference_formulas():
    hm = CudaClosedHashmap(n_buckets=97, device="cpu", key_size=2,
                           prime1=torch.tensor([101, 103]), prime2=torch.tensor([1009, 1013]),
                           alpha1=torch.tensor([3, 5]), alpha2=torch.tensor([7, 11]),
                           beta1=torch.tensor([1, 2]), beta2=torch.tensor([4, 6]))
    keys = torch.tensor([[10, 20], [0, 1], [-3, 8]])
    h = [abs(((3 * a + 1) % 101) * ((5 * b + 2) % 103)) % 97 for a, b in keys.tolist()]
    u = [abs(((7 * a + 4) % 1009) * ((11 * b + 6) % 1013)) for a, b in keys.tolist()]
    assert hm.get_hash(keys).tolist() == h and hm.get_uuid(keys).tolist() == u
    # floats are hashed by bit pattern with minus zero mapped to plus zero
    fk = torch.tensor([[0.0, -0.0], [1.5, 2.0]])
    bits = fk.view(torch.int32).long()
    bits[bits == -2**31] = 0
    exp = (((3 * bits[:, 0] + 1) % 101) * ((5 * bits[:, 1] + 2) % 103)).abs() % 97
    assert torch.equal(hm.get_hash(fk), exp)
    assert 0 < float(hm.test_uniformity(torch.arange(2000).reshape(1000, 2))) <= 1.0


SELECTOR_CASES = [
    lambda r, c, m: (r, c),
    lambda r, c, m: (r[:, None], c[None, :]),
    lambda r, c, m: (r,),
    lambda r, c, m: r,
    lambda r, c, m: (slice(None), c),
    lambda r, c, m: (slice(2, 9), slice(None, 5)),
    lambda r, c, m: (slice(5, 3), c),
    lambda r, c, m: (r.tolist(), slice(1, 4)),
    lambda r, c, m: (r.to(torch.int32), c.to(torch.int16)),
    lambda r, c, m: (3, c),
    lambda r, c, m: (3, slice(None)),
    lambda r, c, m: (slice(None), m),
    lambda r, c, m: (r.numpy(), c.numpy()),
    lambda r, c, m: (slice(None), slice(None)),
    lambda r, c, m: slice(1, 3),
]


@pytest.mark.parametrize("case", range(len(SELECTOR_CASES)))
def test_selector_handling_matches_the_oracle(case):
    g = torch.Generator().manual_seed(case)
    r = torch.randint(0, 13, (6,), generator=g)
    c = torch.randint(0, 17, (6,), generator=g)
    m = torch.rand(17, generator=g) < 0.5
    sel = SELECTOR_CASES[case](r, c, m)
    mine, mine_sc = SparseDOKTensor(size=(13, 17), device="cpu")._handle_selectors(sel)
    ref, ref_sc = RefSparseDOKTensor((13, 17))._handle_selectors(sel)
    assert mine_sc == ref_sc
    assert len(mine) == len(ref) == 2
    for a, b in zip(mine, ref):
        assert a.shape == b.shape and torch.equal(a, b)


def test_selector_handling_4d_axis_rule():
    dok = SparseDOKTensor(size=(6, 7, 5, 4), device="cpu")
    ref = RefSparseDOKTensor((6, 7, 5, 4))
    i, k = torch.tensor([0, 5, 2]), torch.tensor([3, 0, 1])
    mask = torch.tensor([True, False, True, True])
    for sel in [(slice(None), i, slice(None), k), (i, slice(None), k), (4, slice(0, 3), i[:2], k[:2]),
                (2, slice(0, 5), i[:, None], mask), (slice(None), slice(None), slice(None), mask)]:
        mine, msc = dok._handle_selectors(sel)
        theirs, rsc = ref._handle_selectors(sel)
        assert msc == rsc
        for a, b in zip(mine, theirs):
            assert a.shape == b.shape and torch.equal(a, b)


def test_selector_errors():
    dok = SparseDOKTensor(size=(5, 6), device="cpu")
    with pytest.raises(ValueError):
        dok._handle_selectors((slice(0, 4, 2),))            # the reference would silently ignore the step
    with pytest.raises(ValueError):
        dok._handle_selectors((1.5,))
    with pytest.raises(IndexError):
        dok._handle_selectors((0, 0, 0))
    # negative slice bounds are taken from the end
    sel, _ = dok._handle_selectors((slice(-2, None), slice(None, -4)))
    assert sel[0].shape == (2, 2) and sel[0][:, 0].tolist() == [3, 4] and sel[1][0].tolist() == [0, 1]


def test_empty_dok_tensor_on_cpu_reads_zero():
    dok = SparseDOKTensor(size=(5, 6), device="cpu", dtype="float")
    assert dok.shape == (5, 6) and dok.ndim == 2 and dok.dtype == torch.float32 and dok.is_sparse
    assert dok._nnz() == 0 and dok.sparsity == 1.0
    assert torch.equal(dok[1:3, :], torch.zeros(2, 6))
    assert torch.equal(dok.to_dense(), torch.zeros(5, 6))
    assert dok.indices().shape == (2, 0) and dok.values().shape == (0,)
    assert dok[:, 2, ].shape == (5,)


def _coords_from_plan(ix, out_shape, ndim):
    """Evaluate a dok_index_t the way the kernels do: coordinate = base + (data[off] | off)."""
    grids = np.indices(out_shape).reshape(len(out_shape), -1) if len(out_shape) else np.zeros((0, 1), dtype=np.int64)
    n = grids.shape[1] if len(out_shape) else 1
    out = []
    for d in range(ndim):
        v = ix.sel[d]
        off = np.zeros(n, dtype=np.int64)
        for j in range(len(out_shape)):
            off += grids[j] * v.strides[j]
        if v.data:
            buf = (ctypes.c_int64 * (int(off.max()) + 1 if n else 1)).from_address(v.data)
            vals = np.frombuffer(buf, dtype=np.int64)[off]
        else:
            vals = off
        out.append(vals + v.base)
    return out


@pytest.mark.parametrize("case", range(len(SELECTOR_CASES)))
def test_affine_plan_equals_materialised_selectors(case):
    g = torch.Generator().manual_seed(case)
    r = torch.randint(0, 13, (6,), generator=g)
    c = torch.randint(0, 17, (6,), generator=g)
    m = torch.rand(17, generator=g) < 0.5
    sel = SELECTOR_CASES[case](r, c, m)
    dok = SparseDOKTensor(size=(13, 17), device="cpu")
    mats, sc1 = dok._handle_selectors(sel)
    plan, keep = dok._plan(sel)
    ix, out_shape, sc2 = plan.ix, plan.out_shape, plan.scalar_positions
    assert sc1 == sc2 and tuple(mats[0].shape) == out_shape
    if int(np.prod(out_shape)) == 0:
        return
    for got, exp in zip(_coords_from_plan(ix, out_shape, 2), mats):
        assert np.array_equal(got, exp.reshape(-1).numpy())


def test_affine_plan_4d_and_views():
    dok = SparseDOKTensor(size=(6, 7, 5, 4), device="cpu")
    i, k = torch.tensor([0, 5, 2]), torch.tensor([3, 0, 1])
    mask = torch.tensor([True, False, True, True])
    for sel in [(slice(None), i, slice(None), k), (i, slice(None), k), (4, slice(0, 3), i[:2], k[:2]),
                (2, slice(1, 5), i[:, None], mask), (3,), (3, 2, 1, 0), (slice(2, 2),)]:
        mats, sc1 = dok._handle_selectors(sel)
        plan, keep = dok._plan(sel)
        ix, out_shape, sc2 = plan.ix, plan.out_shape, plan.scalar_positions
        assert sc1 == sc2 and tuple(mats[0].shape) == out_shape
        if int(np.prod(out_shape)) == 0:
            continue
        for got, exp in zip(_coords_from_plan(ix, out_shape, 4), mats):
            assert np.array_equal(got, exp.reshape(-1).numpy())
    # a permuted view fills the descriptor in the storage's dimension order
    v = dok.permute(2, 0, 3, 1)
    plan, keep = v._plan((1, slice(None), 2, slice(0, 3)))
    ix, out_shape = plan.ix, plan.out_shape
    assert out_shape == (6, 3)
    assert ix.sel[2].base == 1 and ix.sel[3].base == 2          # view dims 0, 2 -> storage dims 2, 3
    assert list(ix.sel[0].strides)[:2] == [1, 0] and list(ix.sel[1].strides)[:2] == [0, 1]


def test_plans_are_reused_by_structure_and_refreshed_by_value():
    """An expression of a structure seen before takes the cached descriptor with only its integer
    bases and data pointers refreshed: the coordinates it yields must be those of a fresh plan, for
    other integers, other index tensors of the same shape, and a mask that was changed in place."""
    dok = SparseDOKTensor(size=(6, 7, 5, 4), device="cpu")
    idx_a, idx_b = torch.tensor([[0], [3], [4]]), torch.tensor([[2], [2], [1]])
    mask = torch.tensor([True, False, True, True])
    first, _ = dok._plan((2, slice(1, 5), idx_a, mask))
    for i, idx in ((2, idx_a), (5, idx_b), (0, idx_a.clone())):
        sel = (i, slice(1, 5), idx, mask)
        plan, keep = dok._plan(sel)
        assert plan is first                                   # same structure: the cached plan
        mats, sc = dok._handle_selectors(sel)
        assert sc == plan.scalar_positions and tuple(mats[0].shape) == plan.out_shape
        for got, exp in zip(_coords_from_plan(plan.ix, plan.out_shape, 4), mats):
            assert np.array_equal(got, exp.reshape(-1).numpy())
    assert dok[2, 1:5, idx_a, mask].shape == first.final_shape
    # other slice bounds, another index shape: other plans
    assert dok._plan((2, slice(0, 5), idx_a, mask))[0] is not first
    assert dok._plan((2, slice(1, 5), idx_a[:2], mask))[0] is not first
    # a mask changed in place selects other columns: its version is part of the structure
    mask[1] = True
    plan2, keep = dok._plan((2, slice(1, 5), idx_a, mask))
    assert plan2 is not first and plan2.out_shape[-1] == 4 or plan2.out_shape != first.out_shape
    mats, _ = dok._handle_selectors((2, slice(1, 5), idx_a, mask))
    for got, exp in zip(_coords_from_plan(plan2.ix, plan2.out_shape, 4), mats):
        assert np.array_equal(got, exp.reshape(-1).numpy())
    # selectors that are converted on the way (lists, int32 tensors) are planned afresh every time
    p1, _ = dok._plan(([1, 2], 0))
    p2, _ = dok._plan(([1, 2], 0))
    assert p1 is not p2
    # a permuted view keeps plans of its own
    v = dok.permute(3, 2, 1, 0)
    assert v._plans == {} and len(dok._plans) >= 3
    dok.permute_(1, 0, 2, 3)
    assert dok._plans == {}


def test_bulk_path_decision():
    """The host rule that sends a batch through the bulk insert: large batches with enough rows
    per bucket, fewer rows per bucket when the table ends up nearly full."""
    from doksparse_amd.closed_hashmap import bulk_pays
    M = 1 << 20
    S = 10                                        # slots per bucket of int64 -> float32
    # the headline build: 64M rows into 2^27 slots
    assert bulk_pays(64 * M, 128 * M // S, S, 0)
    # small batches never; from a million rows on with at least 2 rows per bucket
    assert not bulk_pays(M // 2, M // 2 // S, S, 0)
    assert bulk_pays(4 * M, 4 * M // S, S, 0) and bulk_pays(M, M // 2, S, 0) and not bulk_pays(M, M, S, 0)
    # a large batch that is thin against the table (1.25 rows per bucket, table stays empty)
    assert not bulk_pays(16 * M, int(16 * M / 1.25), S, 0)
    # the same density pays once the table ends up more than 70 % full ...
    nb = 10 * M
    assert not bulk_pays(16 * M, nb, S, 0)                    # 1.6 rows per bucket, ends 16 % full
    assert bulk_pays(16 * M, nb, S, int(0.6 * nb * S))        # ends 76 % full
    # ... but not below 1.5 rows per bucket
    assert not bulk_pays(12 * M, nb, S, int(0.8 * nb * S))


def test_row_width_rule_and_unique_rows_inverse():
    """Which rows fit a 128-byte bucket (tag word + key words + value words), and the bit-pattern
    unique with its inverse that the out-of-line value path groups a batch by."""
    import torch
    from doksparse_amd import closed_hashmap as ch
    k1, k3, k15 = torch.zeros(2, 1, dtype=torch.long), torch.zeros(2, 3), torch.zeros(2, 15, dtype=torch.long)
    assert ch._row_fits(k1, torch.zeros(2, 1))                                  # packed layout
    assert ch._row_fits(k3, torch.zeros(2, 5, dtype=torch.long))                # 8 * (1 + 2 + 5) = 64
    assert ch._row_fits(k1, torch.zeros(2, 14, dtype=torch.long))               # 8 * (1 + 1 + 14) = 128
    assert not ch._row_fits(k1, torch.zeros(2, 15, dtype=torch.long))
    assert not ch._row_fits(k3, torch.zeros(2, 40))
    assert not ch._row_fits(k15, torch.zeros(2, 1))                             # the key alone is too wide
    nan = float("nan")
    keys = torch.tensor([[0.0, 1.0], [-0.0, 1.0], [nan, 2.0], [0.0, 1.0], [nan, 2.0], [-3.0, 0.5]])
    uniq, inv = ch.unique_rows_inverse(keys)
    assert uniq.shape == (4, 2) and inv.shape == (6,)
    assert torch.equal(uniq.view(torch.int32), ch.unique_rows(keys).view(torch.int32))
    assert torch.equal(uniq[inv].view(torch.int32), keys.view(torch.int32))     # -0.0 and +0.0 apart, equal NaNs together
    assert inv[0] == inv[3] and inv[2] == inv[4] and inv[0] != inv[1]
