"""GPU parity of the bulk insert (partition by table range + merge in LDS) against the CPU oracle.

The bulk path is normally chosen only for batches of a million rows and more; the tests lower
the thresholds so that every `set` below goes through it, at sizes the oracle finishes in
seconds, and compare the resulting map - not the slot placement - with the oracle's."""
import ctypes

import numpy as np
import pytest
import torch

from oracle.ref_hashmap import RefClosedHashmap
from test_gpu_hashmap import _assert_same_map, _check_get, _to, _unique_i64

pytestmark = pytest.mark.gpu


@pytest.fixture
def bulk_always(monkeypatch):
    from doksparse_amd import closed_hashmap as ch
    monkeypatch.setattr(ch, "BULK_MIN_ROWS", 0)
    monkeypatch.setattr(ch, "BULK_MIN_ROWS_PER_BUCKET", 0.0)
    monkeypatch.setattr(ch, "BULK_REMOVE_MIN_ROWS_PER_BUCKET", 0.0)
    return ch


def _bulk_never(monkeypatch):
    from doksparse_amd import closed_hashmap as ch
    monkeypatch.setattr(ch, "BULK_MIN_ROWS", 1 << 62)


@pytest.mark.parametrize("key_dtype,value_dtype", [
    (np.int64, np.float32), (np.int64, np.int64), (np.int64, np.float16), (np.int64, np.int8),
    (np.int32, np.int32), (np.int16, np.float64),
])
@pytest.mark.parametrize("n,capacity", [(5000, 16384), (20000, 22300), (300, 330), (60000, 2_000_000), (7, 8)])
def test_bulk_upsert_matches_oracle(cuda, monkeypatch, key_dtype, value_dtype, n, capacity):
    """Pre-populated table with tombstones, then one bulk batch mixing overwrites and new keys;
    load factors up to 0.9, tables smaller and larger than one merge range."""
    from doksparse_amd import CudaClosedHashmap, closed_hashmap as ch
    rng = np.random.default_rng(n + capacity)
    hi = min(2**62, int(np.iinfo(key_dtype).max))
    if hi < 2**20:
        n = min(n, hi // 8)
        keys = rng.permutation(hi)[: 2 * n].astype(key_dtype)
    else:
        keys = _unique_i64(rng, 2 * n, hi=hi).astype(key_dtype)
    vmax = 100 if np.dtype(value_dtype).itemsize == 1 else 30000
    hm = CudaClosedHashmap(n_buckets=capacity, device=cuda, rehash_threshold=1.0)
    ref = RefClosedHashmap(n_buckets=capacity, rehash_threshold=1.0, rng=np.random.default_rng(1))

    _bulk_never(monkeypatch)
    first = keys[: n // 3, None]
    v1 = rng.integers(-vmax, vmax, size=(first.shape[0], 1)).astype(value_dtype)
    hm.set(*_to(cuda, first, v1)); ref.set(first, v1)
    gone = keys[: n // 6, None]
    if gone.shape[0]:
        hm.remove(torch.from_numpy(gone).to(cuda)); ref.remove(gone)

    monkeypatch.setattr(ch, "BULK_MIN_ROWS", 0)
    monkeypatch.setattr(ch, "BULK_MIN_ROWS_PER_BUCKET", 0.0)
    batch = keys[n // 8: n, None]
    batch = batch[rng.permutation(batch.shape[0])]
    v2 = rng.integers(-vmax, vmax, size=(batch.shape[0], 1)).astype(value_dtype)
    hm.set(*_to(cuda, batch, v2)); ref.set(batch, v2)
    assert hm.n_elements == ref.n_elements
    _assert_same_map(hm, ref)
    _check_get(hm, ref, keys[:, None], cuda, fallback=3)
    # and a second bulk batch on top: all overwrites
    v3 = rng.integers(-vmax, vmax, size=(batch.shape[0], 1)).astype(value_dtype)
    hm.set(*_to(cuda, batch, v3)); ref.set(batch, v3)
    assert hm.n_elements == ref.n_elements
    _assert_same_map(hm, ref)


def test_bulk_nearly_full_table_larger_than_one_pass_of_workgroups(cuda, bulk_always):
    """2.7M keys into 3M slots (load factor 0.9, ~1170 merge ranges): workgroups merge several
    consecutive ranges each, probe chains cross range boundaries, and the rows that do are handed
    from one range to the next.  Then a second batch of the same size: overwrites plus the keys
    that fill the table to 97 %.  Keys are unique inside each batch, so the expected map is known
    without the oracle (whose slot-by-slot probing takes minutes at this load): the last value
    written to each key."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(31)
    n, extra, capacity = 2_700_000, 210_000, 3_000_000
    keys = _unique_i64(rng, n + extra)
    vals = rng.standard_normal((keys.shape[0], 1)).astype(np.float32)
    hm = CudaClosedHashmap(n_buckets=capacity, device=cuda, rehash_threshold=1.0)
    hm.set(*_to(cuda, keys[:n, None], vals[:n]))
    assert hm.n_elements == n
    got, found = hm.get(torch.from_numpy(keys[:, None]).to(cuda))
    found = found.cpu().numpy()
    assert found[:n].all() and not found[n:].any()
    assert np.array_equal(got.cpu().numpy()[:n], vals[:n])

    again = np.concatenate([keys[n:], keys[: n - extra]])
    v2 = rng.standard_normal((again.shape[0], 1)).astype(np.float32)
    hm.set(*_to(cuda, again[:, None], v2))
    assert hm.n_elements == n + extra
    expect = vals.copy()
    expect[n:] = v2[:extra]
    expect[: n - extra] = v2[extra:]
    absent = _unique_i64(rng, 100_000) | (1 << 62)
    got, found = hm.get(torch.from_numpy(np.concatenate([keys, absent])[:, None]).to(cuda), fallback_value=-1.0)
    found, got = found.cpu().numpy(), got.cpu().numpy()
    assert found[: keys.shape[0]].all() and not found[keys.shape[0]:].any()
    assert np.array_equal(got[: keys.shape[0]], expect) and (got[keys.shape[0]:] == -1.0).all()
    k_out, v_out = hm.items()
    order = np.argsort(k_out.cpu().numpy().reshape(-1))
    ref_order = np.argsort(keys)
    assert np.array_equal(k_out.cpu().numpy().reshape(-1)[order], keys[ref_order])
    assert np.array_equal(v_out.cpu().numpy()[order], expect[ref_order])


def test_bulk_equal_keys_inside_one_batch(cuda, bulk_always):
    """Every key 32 times in one bulk batch: one slot per key, holding one of its values."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(11)
    base = _unique_i64(rng, 3000)
    keys = np.repeat(base, 32)
    perm = rng.permutation(keys.shape[0])
    keys = keys[perm]
    ids = np.repeat(np.arange(base.shape[0]), 32)[perm]
    copy = rng.integers(0, 2**30, size=keys.shape[0])
    vals = (ids * 2**32 + copy).astype(np.int64)
    for capacity in (3400, 8192, 200_000):
        hm = CudaClosedHashmap(n_buckets=capacity, device=cuda, rehash_threshold=1.0)
        hm.set(*_to(cuda, keys[:, None], vals[:, None]))
        assert hm.n_elements == base.shape[0]
        gk, _ = hm.items()
        assert gk.shape[0] == base.shape[0] and np.unique(gk.cpu().numpy()).shape[0] == base.shape[0]
        out, found = hm.get(torch.from_numpy(base[:, None]).to(cuda))
        assert bool(found.all())
        out = out.cpu().numpy().reshape(-1)
        written = {}
        for i_, c_ in zip(ids, copy):
            written.setdefault(int(i_), set()).add(int(c_))
        for i_ in range(base.shape[0]):
            assert out[i_] >> 32 == i_ and int(out[i_] & (2**32 - 1)) in written[i_]


def test_bulk_reserved_patterns_and_full_table(cuda, bulk_always):
    from doksparse_amd import CudaClosedHashmap
    X = np.uint64(0x9E3779B97F4A7C15)
    special = np.array([X, X ^ np.uint64(1), 0, 1, np.uint64(2**64 - 1), np.uint64(2**63)],
                       dtype=np.uint64).view(np.int64)[:, None]
    vals = np.arange(1, special.shape[0] + 1, dtype=np.float32)[:, None]
    hm = CudaClosedHashmap(n_buckets=64, device=cuda)
    ref = RefClosedHashmap(n_buckets=64)
    hm.set(*_to(cuda, special, vals)); ref.set(special, vals)
    assert hm.n_elements == ref.n_elements == special.shape[0]
    _check_get(hm, ref, special, cuda)
    _assert_same_map(hm, ref)

    # more distinct keys than physical slots: the surplus is reported, nothing is lost silently
    hm = CudaClosedHashmap(n_buckets=100, device=cuda, rehash_threshold=1e9)
    keys = _unique_i64(np.random.default_rng(2), 400)[:, None]
    v = np.arange(400, dtype=np.float32)[:, None]
    slots = 10 * 10                                  # 100 slots asked for = 10 buckets of 10
    with pytest.raises(RuntimeError, match=f"full: {400 - slots} rows"):
        hm.set(*_to(cuda, keys, v))
    assert slots == hm._n_phys * hm._slots_per_bucket
    h = hm._header.cpu()
    assert int(h[0]) == slots and int(h[1]) == 0     # reported once, then cleared
    out, found = hm.get(torch.from_numpy(keys).to(cuda))
    assert int(found.sum().item()) == slots
    assert torch.equal(out[found].cpu(), torch.from_numpy(v)[found.cpu()])


def test_bulk_coordinate_keys_and_coo_constructor(cuda, bulk_always):
    """Coordinate-keyed maps: row-major key rows and the [ndim, n] COO layout both go through the
    bulk path; rows outside the size are skipped and counted."""
    from doksparse_amd import CudaClosedHashmap, SparseDOKTensor
    rng = np.random.default_rng(21)
    size = (300, 77, 5)
    lin = rng.permutation(int(np.prod(size)))[:40000]
    coords = np.stack(np.unravel_index(lin, size))
    vals = rng.standard_normal(lin.shape[0]).astype(np.float32)
    dok = SparseDOKTensor(size, torch.from_numpy(coords).to(cuda), torch.from_numpy(vals).to(cuda), device=cuda)
    dense = torch.zeros(size)
    dense[tuple(torch.from_numpy(coords))] = torch.from_numpy(vals)
    assert dok._nnz() == lin.shape[0]
    assert torch.equal(dok.to_dense().cpu(), dense)
    rows = torch.arange(0, 300, 7, device=cuda)
    assert torch.equal(dok[rows[:, None], 3:60, 2].cpu(), dense[rows.cpu()[:, None], 3:60, 2])

    hm = CudaClosedHashmap(n_buckets=50000, device=cuda, coord_dims=size, rehash_threshold=1.0)
    bad = coords.T.copy()
    bad[::100, 1] = 77                                   # out of range in dimension 1
    hm.set(torch.from_numpy(bad).to(cuda), torch.from_numpy(vals[:, None]).to(cuda))
    h = hm._header.cpu()
    n_bad = bad[::100].shape[0]
    assert int(h[3]) == n_bad and int(h[0]) == lin.shape[0] - n_bad


def test_bulk_entry_point_rejects_bad_arguments(cuda):
    from doksparse_amd import CudaClosedHashmap, _lib
    lib = _lib.load()
    hm = CudaClosedHashmap(n_buckets=4096, device=cuda)
    k = torch.arange(100, device=cuda)[:, None]
    v = torch.ones(100, 1, device=cuda)
    hm.set(k, v)
    desc = ctypes.byref(hm._desc)
    need = int(lib.dok_bulk_workspace_bytes(desc, 100))
    assert need > 0
    ws = torch.empty(need, device=cuda, dtype=torch.uint8)
    assert lib.dok_map_set_bulk(desc, k.data_ptr(), v.data_ptr(), 100, ws.data_ptr(), need - 1, None) == _lib.DOK_EINVAL
    assert lib.dok_map_set_bulk(desc, k.data_ptr(), v.data_ptr(), 100, ws.data_ptr() + 8, need, None) == _lib.DOK_EINVAL
    assert lib.dok_map_set_bulk(desc, None, v.data_ptr(), 100, ws.data_ptr(), need, None) == _lib.DOK_EINVAL
    assert lib.dok_map_set_bulk(desc, k.data_ptr(), v.data_ptr(), 0, ws.data_ptr(), need, None) == _lib.DOK_OK
    assert lib.dok_coo_set_bulk(desc, k.data_ptr(), v.data_ptr(), 100, ws.data_ptr(), need, None) == _lib.DOK_EINVAL
    # the multi-word layout's bulk form needs the list of deferred rows: 8 bytes per row + 256
    hm2 = CudaClosedHashmap(n_buckets=256, device=cuda)
    k2, v2 = torch.rand(10, 3, device=cuda), torch.zeros(10, 5, device=cuda, dtype=torch.long)
    hm2.set(k2, v2)
    assert int(lib.dok_bulk_workspace_bytes(ctypes.byref(hm2._desc), 10)) == 8 * 10 + 256
    assert lib.dok_map_set_bulk(ctypes.byref(hm2._desc), k2.data_ptr(), v2.data_ptr(), 10, ws.data_ptr(), 8 * 10 + 248, None) \
        == _lib.DOK_EINVAL
    assert lib.dok_coo_set_bulk(ctypes.byref(hm2._desc), k2.data_ptr(), v2.data_ptr(), 10, ws.data_ptr(), need, None) \
        == _lib.DOK_EINVAL                                   # not a coordinate table
    torch.cuda.synchronize()
    assert hm.n_elements == 100


def test_bulk_call_replays_inside_a_hip_graph(cuda):
    """dok_map_set_bulk on fixed buffers (keys, values, workspace) captured into a HIP graph and
    replayed on changing contents, with eager work between the replays; every replay is checked
    against the oracle."""
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    rng = np.random.default_rng(99)
    n = 30000
    allk = _unique_i64(rng, 4 * n)
    hm = CudaClosedHashmap(n_buckets=5 * n, device=cuda, rehash_threshold=1.0)
    ref = RefClosedHashmap(n_buckets=5 * n, rng=np.random.default_rng(3), rehash_threshold=1.0)
    k0, v0 = allk[:n, None], rng.standard_normal((n, 1)).astype(np.float32)
    hm.set(*_to(cuda, k0, v0)); ref.set(k0, v0)

    sk = torch.from_numpy(k0).to(cuda)                      # static inputs of the graph
    sv = torch.from_numpy(v0).to(cuda)
    desc = ctypes.byref(hm._desc)
    need = int(lib.dok_bulk_workspace_bytes(desc, n))
    ws = torch.empty(need, device=cuda, dtype=torch.uint8)

    def bulk():
        _lib.check(lib.dok_map_set_bulk(desc, sk.data_ptr(), sv.data_ptr(), n, ws.data_ptr(), need,
                                        _stream_ptr(cuda)), "set_bulk")
    bulk()                                                   # eager warm-up (module load, occupancy query)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        bulk()
    torch.cuda.synchronize()
    for r in range(1, 4):
        newk = np.concatenate([allk[r * n:r * n + n // 2], allk[(r - 1) * n:(r - 1) * n + n // 2]])[:, None]
        newv = rng.standard_normal((n, 1)).astype(np.float32)
        sk.copy_(torch.from_numpy(newk)); sv.copy_(torch.from_numpy(newv))
        graph.replay()
        torch.cuda.synchronize()
        ref.set(newk, newv)
        assert hm.n_elements == ref.n_elements
        _check_get(hm, ref, allk[:, None], cuda)             # eager work between replays
        _assert_same_map(hm, ref)


@pytest.mark.parametrize("value_dtype", [np.float32, np.int64, np.float16, np.int8])
def test_bulk_rehash_keeps_the_map(cuda, bulk_always, value_dtype):
    """rehash through the bulk path (the old table is the batch): live entries move, tombstones
    and empty slots do not, the two reserved key patterns survive; growing and shrinking."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(17)
    X = np.uint64(0x9E3779B97F4A7C15)
    special = np.array([X, X ^ np.uint64(1)], dtype=np.uint64).view(np.int64)
    keys = np.concatenate([_unique_i64(rng, 60000), special])[:, None]
    vals = rng.integers(-100, 100, size=(keys.shape[0], 1)).astype(value_dtype)
    hm = CudaClosedHashmap(n_buckets=70000, device=cuda, rehash_threshold=1.0)
    ref = RefClosedHashmap(n_buckets=70000, rehash_threshold=1.0, rng=np.random.default_rng(1))
    hm.set(*_to(cuda, keys, vals)); ref.set(keys, vals)
    gone = keys[::3]
    hm.remove(torch.from_numpy(gone).to(cuda)); ref.remove(gone)
    for new_size in (300_000, 45_000, 1_000_000):
        hm.rehash(new_size); ref.rehash(new_size)
        assert hm.n_buckets == ref.n_buckets == new_size
        assert hm.n_elements == ref.n_elements
        _assert_same_map(hm, ref)
        _check_get(hm, ref, keys, cuda, fallback=5)
    # the rehashed table is an ordinary table: per-row set, remove and get keep working on it
    more = (_unique_i64(rng, 5000) | (1 << 62))[:, None]
    mv = rng.integers(-100, 100, size=(5000, 1)).astype(value_dtype)
    hm.set(*_to(cuda, more, mv)); ref.set(more, mv)
    hm.remove(torch.from_numpy(keys[1::3]).to(cuda)); ref.remove(keys[1::3])
    assert hm.n_elements == ref.n_elements
    _assert_same_map(hm, ref)


def test_bulk_rehash_of_a_coordinate_keyed_tensor(cuda, bulk_always):
    from doksparse_amd import SparseDOKTensor
    g = torch.Generator().manual_seed(4)
    size = (500, 300)
    lin = torch.randperm(size[0] * size[1], generator=g)[:30000]
    coords = torch.stack([lin // size[1], lin % size[1]])
    vals = torch.randn(30000, generator=g)
    dok = SparseDOKTensor(size, coords.to(cuda), vals.to(cuda), device=cuda)
    dense = torch.zeros(size)
    dense[coords[0], coords[1]] = vals
    dok.storage().rehash(200_000)
    assert dok._nnz() == 30000
    assert torch.equal(dok.to_dense().cpu(), dense)
    more = torch.randperm(size[0] * size[1], generator=g)[:40000]
    mv = torch.randn(40000, generator=g)
    dok[(more // size[1]).to(cuda), (more % size[1]).to(cuda)] = mv.to(cuda)       # grows again
    dense[more // size[1], more % size[1]] = mv
    assert torch.equal(dok.to_dense().cpu(), dense)


def test_bulk_and_per_row_insert_agree_on_random_configurations(cuda, monkeypatch):
    """Twenty-four random configurations (size, load factor up to 0.97, share of repeated keys, value
    width): three batches each with removals in between, once through the per-row kernel and once
    through the bulk path.  Values are a function of key and batch number, so the resulting map
    is unique and must be the same (which the oracle pins for the per-row path elsewhere)."""
    from doksparse_amd import CudaClosedHashmap, closed_hashmap as ch
    rng = np.random.default_rng(2024)

    def val_of(keys, rnd, dt):
        x = (keys * 2654435761 + rnd * 97) >> 7
        if dt.is_floating_point:
            return ((x % 2001) - 1000).to(dt)
        if dt == torch.int8:
            return ((x % 201) - 100).to(dt)
        return x.to(dt)

    for case in range(24):
        n = int(10 ** rng.uniform(3, 6.2))
        lf = float(rng.uniform(0.2, 0.97))
        dt = [torch.float32, torch.int64, torch.float16, torch.int8][case % 4]
        universe = int(n * rng.uniform(0.6, 1.5)) + 10
        cap = int(universe / lf) + 16
        g = torch.Generator(device=cuda); g.manual_seed(case)
        keyspace = torch.randint(-2**62, 2**62, (universe,), generator=g, device=cuda)
        maps = []
        for bulk in (False, True):
            monkeypatch.setattr(ch, "BULK_MIN_ROWS", 0 if bulk else 1 << 62)
            monkeypatch.setattr(ch, "BULK_MIN_ROWS_PER_BUCKET", 0.0)
            hm = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=1e9, seed=77 + case)
            gg = torch.Generator(device=cuda); gg.manual_seed(1000 + case)
            for rnd in range(3):
                k = keyspace[torch.randint(0, universe, (n,), generator=gg, device=cuda)]
                hm.set(k[:, None], val_of(k, rnd, dt)[:, None])
                if rnd == 0:
                    gone = keyspace[torch.randint(0, universe, (n // 5,), generator=gg, device=cuda)]
                    hm._remove_rows(gone[:, None].contiguous())
            h = hm._header.cpu()
            keys, vals = hm.items()
            order = torch.argsort(keys.reshape(-1))
            maps.append((keys.reshape(-1)[order], vals.reshape(-1)[order], int(h[0]), int(h[1])))
        a, b = maps
        assert a[2] == b[2] == a[0].shape[0] and a[3] == b[3] == 0, (case, a[2:], b[2:])
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]), f"case {case}: maps differ"


def _garbage(hm):
    """Overwrite the table's bucket memory and header with a pattern no kernel writes."""
    hm._table.fill_(0xA5)
    hm._header.fill_(-0x0123456789ABCDEF)


@pytest.mark.parametrize("value_dtype", [np.float32, np.int64, np.float16, np.int8])
@pytest.mark.parametrize("n,capacity", [(5000, 16384), (20000, 22300), (300, 400), (3000, 2_000_000), (7, 8)])
def test_build_into_uninitialised_table_matches_oracle(cuda, value_dtype, n, capacity):
    """dok_map_build_bulk = clear + bulk insert in one pass: table memory and header are filled
    with garbage first, ranges with and without rows (the sparse 2M-slot table), equal keys in the
    batch, the reserved key patterns.  Afterwards the table must behave like any other: lookups,
    read-out, count, a removal and a per-row insert on top."""
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    rng = np.random.default_rng(n + capacity + np.dtype(value_dtype).itemsize)
    XOR = np.uint64(0x9E3779B97F4A7C15).astype(np.int64)
    keys = _unique_i64(rng, 2 * n, hi=2**62)
    keys[0], keys[1] = XOR, XOR ^ np.int64(1)                   # the two reserved stored patterns
    vmax = 100 if np.dtype(value_dtype).itemsize == 1 else 30000
    hm = CudaClosedHashmap(n_buckets=capacity, device=cuda, rehash_threshold=1.0)
    ref = RefClosedHashmap(n_buckets=capacity, rehash_threshold=1.0, rng=np.random.default_rng(1))
    # allocate through a tiny first set, then throw the contents away
    seed_v = np.zeros((1, 1), dtype=value_dtype)
    hm.set(*_to(cuda, keys[-1:, None], seed_v))
    _garbage(hm)
    batch = np.concatenate([keys[:n], keys[: n // 10]])[:, None]      # a tenth of the keys twice
    vals = rng.integers(-vmax, vmax, size=(batch.shape[0], 1)).astype(value_dtype)
    tk, tv = _to(cuda, batch, vals)
    desc = ctypes.byref(hm._desc)
    nbytes = int(lib.dok_bulk_workspace_bytes(desc, batch.shape[0]))
    assert nbytes > 0
    ws = torch.empty(nbytes, device=cuda, dtype=torch.uint8)
    _lib.check(lib.dok_map_build_bulk(desc, tk.data_ptr(), tv.data_ptr(), batch.shape[0], ws.data_ptr(), nbytes,
                                      _stream_ptr(cuda)), "build")
    # the oracle: unique keys first, then the repeated ones (either value of an equal key is allowed)
    ref.set(batch[:n], vals[:n])
    assert hm.n_elements == ref.n_elements == n
    got_v, got_f = hm.get(tk)
    assert bool(got_f.all())
    got = got_v.cpu().numpy()
    first = {int(k): v for k, v in zip(batch[:n, 0], vals[:n, 0])}
    second = {int(k): v for k, v in zip(batch[n:, 0], vals[n:, 0])}
    for k, g in zip(batch[:, 0], got[:, 0]):
        assert g == first[int(k)] or (int(k) in second and g == second[int(k)])
    ks, vs = hm.items()
    assert sorted(ks.cpu().numpy().reshape(-1).tolist()) == sorted(batch[:n, 0].tolist())
    _, miss = hm.get(torch.from_numpy(keys[n:, None]).to(cuda))
    assert not bool(miss.any())
    # ordinary operations on the built table
    ref2 = RefClosedHashmap(n_buckets=capacity, rehash_threshold=1.0, rng=np.random.default_rng(2))
    ref2.set(ks.cpu().numpy().reshape(-1, 1), vs.cpu().numpy().reshape(-1, 1))
    gone = keys[: n // 2, None]
    hm.remove(torch.from_numpy(gone).to(cuda)); ref2.remove(gone)
    more = keys[n: n + n // 4, None]
    mv = rng.integers(-vmax, vmax, size=(more.shape[0], 1)).astype(value_dtype)
    if more.shape[0]:
        hm.set(*_to(cuda, more, mv)); ref2.set(more, mv)
    assert hm.n_elements == ref2.n_elements
    _assert_same_map(hm, ref2)
    _check_get(hm, ref2, keys[:, None], cuda, fallback=5)


def test_first_set_of_a_new_map_builds_without_clear(cuda, bulk_always):
    """CudaClosedHashmap.set on a new map: the table is allocated uninitialised and built in one
    pass when the batch takes the bulk path, cleared first otherwise; either way it is complete
    when set returns, also for an empty first batch."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(11)
    keys = _unique_i64(rng, 40000, hi=2**62)
    vals = rng.integers(-1000, 1000, size=(40000, 1)).astype(np.int32)
    hm = CudaClosedHashmap(n_buckets=60000, device=cuda)
    hm.set(*_to(cuda, keys[:30000, None], vals[:30000]))
    assert not hm._pending_clear and hm.n_elements == 30000
    ref = RefClosedHashmap(n_buckets=60000, rng=np.random.default_rng(1))
    ref.set(keys[:30000, None], vals[:30000])
    _assert_same_map(hm, ref)
    _check_get(hm, ref, keys[:, None], cuda, fallback=-1)
    # empty first batch: the table must still come out cleared
    hm2 = CudaClosedHashmap(n_buckets=1000, device=cuda)
    hm2.set(torch.empty(0, 1, dtype=torch.long, device=cuda), torch.empty(0, 1, dtype=torch.int32, device=cuda))
    assert not hm2._pending_clear and hm2.n_elements == 0
    assert hm2.items()[0].shape[0] == 0
    _, f = hm2.get(torch.from_numpy(keys[:100, None]).to(cuda))
    assert not bool(f.any())
    # first batch above the growth threshold: the count is read before the insert
    hm3 = CudaClosedHashmap(n_buckets=1000, device=cuda)
    hm3.set(*_to(cuda, keys[:5000, None], vals[:5000]))
    assert hm3.n_elements == 5000 and hm3.n_buckets >= 5000
    ref3 = RefClosedHashmap(n_buckets=1000, rng=np.random.default_rng(1))
    ref3.set(keys[:5000, None], vals[:5000])
    assert hm3.n_buckets == ref3.n_buckets
    _assert_same_map(hm3, ref3)


def test_bulk_rehash_overwrites_an_uninitialised_destination(cuda):
    """dok_map_rehash_bulk needs no cleared destination: garbage in, the source's entries out."""
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    rng = np.random.default_rng(21)
    n = 50000
    keys = _unique_i64(rng, n + 1000, hi=2**62)
    vals = rng.standard_normal((n, 1)).astype(np.float32)
    src = CudaClosedHashmap(n_buckets=70000, device=cuda, rehash_threshold=1.0)
    src.set(*_to(cuda, keys[:n, None], vals))
    src.remove(torch.from_numpy(keys[:5000, None]).to(cuda))
    dst = CudaClosedHashmap(n_buckets=400000, device=cuda, rehash_threshold=1.0, seed=99)
    dst.set(*_to(cuda, keys[n:, None], vals[:1000]))          # allocates; these entries must vanish
    _garbage(dst)
    a, b = ctypes.byref(src._desc), ctypes.byref(dst._desc)
    nbytes = int(lib.dok_rehash_bulk_workspace_bytes(a, b))
    assert nbytes > 0
    ws = torch.empty(nbytes, device=cuda, dtype=torch.uint8)
    _lib.check(lib.dok_map_rehash_bulk(a, b, ws.data_ptr(), nbytes, _stream_ptr(cuda)), "rehash")
    assert dst.n_elements == n - 5000
    v, f = dst.get(torch.from_numpy(keys[:, None]).to(cuda))
    f = f.cpu().numpy()
    assert not f[:5000].any() and f[5000:n].all() and not f[n:].any()
    assert np.array_equal(v.cpu().numpy()[5000:n], vals[5000:])
    ks, _ = dst.items()
    assert sorted(ks.cpu().numpy().reshape(-1).tolist()) == sorted(keys[5000:n].tolist())


def test_bulk_upsert_into_a_populated_table_with_tombstones(cuda, bulk_always):
    """1.5M keys at load factor 0.88, a fifth removed (tombstones), then one bulk batch of
    overwrites (also of keys that sit in the range after their home's - their rows follow the
    home bucket's displacement marks across the range boundary), re-inserts of removed keys and
    new keys.  Keys are unique inside each batch, so the expected map is known in closed form."""
    from doksparse_amd import CudaClosedHashmap
    from test_gpu_fullsize import SortedMap
    gen = torch.Generator(device=cuda); gen.manual_seed(77)
    n = 1_500_000
    draw = torch.unique(torch.randint(0, 2**62, (2 * n + 50_000,), generator=gen, device=cuda))
    draw = draw[torch.randperm(draw.numel(), generator=gen, device=cuda)]
    keys, extra = draw[:n].contiguous(), draw[n: n + n // 4].contiguous()
    vals = torch.randint(-2**31, 2**31 - 1, (n,), generator=gen, device=cuda, dtype=torch.int64).to(torch.int32)
    hm = CudaClosedHashmap(n_buckets=int(n / 0.88), device=cuda, rehash_threshold=1.0)
    hm.set(keys[:, None], vals[:, None])
    assert hm.n_elements == n
    gone = keys[: n // 5]
    assert bool(hm._remove_rows(gone[:, None].contiguous()).all())
    # the batch: half of the surviving keys, half of the removed ones, and new keys
    batch = torch.cat([keys[n // 5:][: 2 * n // 5], gone[: n // 10], extra[: n // 8]])
    batch = batch[torch.randperm(batch.numel(), generator=gen, device=cuda)].contiguous()
    bvals = torch.randint(-2**31, 2**31 - 1, (batch.numel(),), generator=gen, device=cuda, dtype=torch.int64).to(torch.int32)
    hm.set(batch[:, None], bvals[:, None])
    untouched = keys[n // 5:][2 * n // 5:]
    model = SortedMap(torch.cat([untouched, batch]),
                      torch.cat([vals[n // 5:][2 * n // 5:], bvals]))
    assert hm.n_elements == model.keys.numel()
    probe = torch.cat([keys, extra])
    got_v, got_f = hm.get(probe[:, None])
    exp_v, exp_f = model.get(probe)
    assert torch.equal(got_f, exp_f) and torch.equal(got_v[:, 0], exp_v)
    ks, vs = hm.items()
    order = torch.argsort(ks[:, 0])
    assert torch.equal(ks[order, 0], model.keys) and torch.equal(vs[order, 0], model.values)


@pytest.mark.parametrize("distinct", [1, 300, 20000])
def test_build_with_many_equal_keys(cuda, bulk_always, distinct):
    """First set of a new map (fresh-table merge) with every key repeated many times: each key is
    stored once and holds the value of one of its rows."""
    from doksparse_amd import CudaClosedHashmap
    gen = torch.Generator(device=cuda); gen.manual_seed(distinct)
    n = 400_000
    base = torch.unique(torch.randint(0, 2**62, (distinct + 16,), generator=gen, device=cuda))[:distinct]
    keys = base[torch.randint(0, distinct, (n,), generator=gen, device=cuda)].contiguous()
    vals = torch.arange(n, device=cuda, dtype=torch.int32)
    hm = CudaClosedHashmap(n_buckets=max(2 * distinct, 64), device=cuda, rehash_threshold=1.0)
    hm.set(keys[:, None], vals[:, None])
    assert hm.n_elements == int(torch.unique(keys).numel())
    v, f = hm.get(keys[:, None])
    assert bool(f.all())
    assert bool((keys[v[:, 0].long()] == keys).all())      # the value is the index of a row with this key
    ks, _ = hm.items()
    assert torch.equal(torch.sort(ks[:, 0]).values, torch.unique(keys))
    # the same rows again, now as an upsert into the populated table (every row of a key beyond
    # what its range's region of the partition holds takes the spill list)
    hm.set(keys[:, None], (vals + n)[:, None])
    assert hm.n_elements == int(torch.unique(keys).numel())
    v, f = hm.get(keys[:, None])
    assert bool(f.all()) and bool((v[:, 0] >= n).all())
    assert bool((keys[(v[:, 0] - n).long()] == keys).all())


@pytest.mark.parametrize("size", [(900_000,), (5000, 3000), (300, 77, 50), (40, 30, 20, 16), (12, 9, 8, 7, 11),
                                  (9, 8, 7, 6, 5, 4), (5, 4, 7, 3, 6, 5, 4), (3, 5, 4, 3, 6, 2, 5, 4)])
def test_bulk_and_per_row_agree_on_coordinate_batches(cuda, monkeypatch, size):
    """Coordinate keys in both layouts ([n, ndim] rows and [ndim, n] COO columns; three and more
    dimensions are linearised by the bulk path's first count), repeated coordinates, coordinates
    outside the size, a removal in between and a second batch: the per-row kernels and the bulk
    path must leave the same map and the same counters."""
    from doksparse_amd import CudaClosedHashmap, closed_hashmap as ch
    gen = torch.Generator(device=cuda); gen.manual_seed(len(size))
    vol = int(np.prod(size))
    n = min(200_000, vol // 3)

    def batch(rnd):
        c = torch.stack([torch.randint(0, s, (n,), generator=gen, device=cuda) for s in size])      # [ndim, n]
        c[0, ::97] = size[0] + rnd                                       # rows outside the size
        lin = torch.zeros(n, dtype=torch.long, device=cuda)
        for d, s in enumerate(size):
            lin = lin * s + c[d]
        return c, ((lin * 31 + rnd) % 1000).to(torch.float32)           # equal coordinates carry equal values

    b1, b2 = batch(0), batch(1)
    gone = b1[0][:, 5:n // 4:3].T.contiguous()
    gone = gone[(gone[:, 0] < size[0])]
    results = []
    for bulk in (False, True):
        monkeypatch.setattr(ch, "BULK_MIN_ROWS", 0 if bulk else 1 << 62)
        monkeypatch.setattr(ch, "BULK_MIN_ROWS_PER_BUCKET", 0.0)
        per_layout = []
        for coo in (False, True):
            hm = CudaClosedHashmap(n_buckets=int(1.3 * 2 * n), device=cuda, coord_dims=size, rehash_threshold=1.0,
                                   seed=4242)
            for c, v in (b1, b2):
                if coo:
                    hm.set_coo(c.contiguous(), v[:, None].contiguous())
                else:
                    hm.set(c.T.contiguous(), v[:, None].contiguous())
                if c is b1[0]:
                    hm._remove_rows(gone)
            idx, vals = hm.items_coo()
            lin = torch.zeros(idx.shape[1], dtype=torch.long, device=cuda)
            for d, s in enumerate(size):
                lin = lin * s + idx[d]
            order = torch.argsort(lin)
            h = hm._header.cpu()
            per_layout.append((lin[order], vals.reshape(-1)[order], int(h[0]), int(h[1]), int(h[3])))
        results.append(per_layout)
    ref = results[0][0]
    assert ref[2] == ref[0].shape[0] and ref[3] == 0 and ref[4] == 2 * len(range(0, n, 97))
    for per_layout in results:
        for got in per_layout:
            assert got[2:] == ref[2:]
            assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])


# ---- the multi-word layout's bulk form: one compare-and-swap per new row, deferred rows in a second launch

@pytest.fixture
def tagged_fast_always(monkeypatch):
    from doksparse_amd import closed_hashmap as ch
    monkeypatch.setattr(ch, "TAGGED_FAST_MIN_ROWS", 0)
    return ch


def test_multiword_fast_and_per_row_insert_agree_on_random_configurations(cuda, monkeypatch):
    """Random configurations of the multi-word layout (key / value widths of one to four slots per
    bucket, load factors up to 0.95, batches with many repeated keys, keys with zero words, removals in
    between so that tombstones are re-used): three batches each, once through the per-row protocol
    and once through the fast form - the first batch of a map as a build into the new table, later
    ones as upserts where the values are one word wide.  Values are a function of key and batch, so
    the resulting map is unique and must be the same."""
    from doksparse_amd import CudaClosedHashmap, closed_hashmap as ch, _lib
    rng = np.random.default_rng(77)
    geoms = [(2, torch.int64, 1, torch.float32), (3, torch.float32, 5, torch.int64), (13, torch.int64, 1, torch.float16),
             (4, torch.int64, 1, torch.int64), (2, torch.int64, 1, torch.int8), (5, torch.int32, 2, torch.int64)]

    def val_of(keys, rnd, vw, dt):
        x = (keys.to(torch.int64).sum(dim=1) * 2654435761 + rnd * 97) >> 5
        cols = torch.stack([(x + 13 * c) % 251 - 125 for c in range(vw)], dim=1)
        return cols.to(dt)

    for case in range(18):
        kw, kdt, vw, vdt = geoms[case % len(geoms)]
        n = int(10 ** rng.uniform(2.5, 5.3))
        lf = float(rng.uniform(0.2, 0.95))
        universe = int(n * rng.uniform(0.3, 1.5)) + 10
        cap = int(universe / lf) + 16
        g = torch.Generator(device=cuda); g.manual_seed(case)
        if kdt.is_floating_point:
            keyspace = torch.randint(-2**20, 2**20, (universe, kw), generator=g, device=cuda).to(kdt)
        else:
            keyspace = torch.randint(-2**30, 2**30, (universe, kw), generator=g, device=cuda).to(kdt)
        keyspace[0] = 0                                  # the all-zero key ...
        keyspace[1: min(200, universe // 4), case % kw] = 0   # ... and keys with one zero word (the fast form defers both kinds)
        keyspace = torch.unique(keyspace, dim=0)
        universe = keyspace.shape[0]
        maps = []
        for fast in (False, True):
            monkeypatch.setattr(ch, "TAGGED_FAST_MIN_ROWS", 0 if fast else 1 << 62)
            hm = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=1e9, seed=501 + case)
            gg = torch.Generator(device=cuda); gg.manual_seed(2000 + case)
            for rnd in range(3):
                pick = torch.randint(0, universe, (n,), generator=gg, device=cuda)
                pick[:3] = 0                             # the zero key, three times in every batch
                k = keyspace[pick]
                hm.set(k, val_of(k, rnd, vw, vdt))
                assert hm._layout == _lib.DOK_LAYOUT_TAGGED
                if rnd < 2:
                    gone = keyspace[torch.randint(0, universe, (n // 4,), generator=gg, device=cuda)]
                    hm._remove_rows(gone.contiguous())
            h = hm._header.cpu()
            keys, vals = hm.items()
            kb = keys.contiguous().view(torch.uint8).reshape(keys.shape[0], -1).cpu().numpy()
            order = np.lexsort(kb.T[::-1])
            maps.append((kb[order], vals.cpu().numpy()[order], int(h[0]), int(h[1])))
        a, b = maps
        assert a[2] == b[2] == a[0].shape[0] and a[3] == b[3] == 0, (case, a[2:], b[2:])
        assert np.array_equal(a[0], b[0]), f"case {case}: key sets differ"
        assert np.array_equal(a[1].view(np.uint8), b[1].view(np.uint8)), f"case {case}: values differ"
        assert len({r.tobytes() for r in a[0]}) == a[0].shape[0], f"case {case}: a key is stored twice"


def test_multiword_fast_insert_with_nothing_but_equal_keys(cuda, tagged_fast_always):
    """A batch of 200,000 rows that holds 5 distinct keys (every row but five is deferred), as the
    first batch of a map and as an upsert: one slot per key, an untorn value of one of its rows."""
    from doksparse_amd import CudaClosedHashmap
    g = torch.Generator(device=cuda).manual_seed(9)
    base = torch.randint(-2**40, 2**40, (5, 2), generator=g, device=cuda)
    pick = torch.randint(0, 5, (200_000,), generator=g, device=cuda)
    rowv = torch.arange(200_000, device=cuda, dtype=torch.float32)[:, None]
    for first in (True, False):
        hm = CudaClosedHashmap(n_buckets=4096, device=cuda)
        if not first:
            hm.set(torch.randint(2**41, 2**42, (1000, 2), generator=g, device=cuda), torch.zeros(1000, 1, device=cuda))
        hm.set(base[pick], rowv)
        assert hm.n_elements == 5 + (0 if first else 1000)
        v, f = hm.get(base)
        assert bool(f.all())
        for j in range(5):
            r = int(v[j, 0].item())
            assert int(pick[r].item()) == j             # the stored value is the row number of a row of that key


def test_multiword_bulk_entry_points_through_the_c_abi(cuda):
    """dok_bulk_workspace_bytes / dok_map_set_bulk / dok_map_build_bulk on a multi-word table, called
    through ctypes: the build takes the table as uninitialised memory, bad workspaces are refused."""
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    rng = np.random.default_rng(3)
    n = 50_000
    keys = np.unique(rng.random((n, 3), dtype=np.float32), axis=0)
    n = keys.shape[0]
    vals = rng.integers(0, 2**62, size=(n, 5), dtype=np.int64)
    hm = CudaClosedHashmap(n_buckets=2 * n, device=cuda, rehash_threshold=1e9)
    k, v = _to(cuda, keys, vals)
    hm.set(k[:4], v[:4])
    desc, st = ctypes.byref(hm._desc), _stream_ptr(cuda)
    need = int(lib.dok_bulk_workspace_bytes(desc, n))
    assert need == 8 * n + 256
    ws = torch.empty(need, device=cuda, dtype=torch.uint8)
    hm._table.fill_(0xA5)                                # garbage: the build must not read it
    hm._header.fill_(-77)
    assert lib.dok_map_build_bulk(desc, k.data_ptr(), v.data_ptr(), n, ws.data_ptr(), need, st) == 0
    ref = RefClosedHashmap(n_buckets=2 * n, rng=np.random.default_rng(8))
    ref.set(keys, vals)
    assert hm.n_elements == ref.n_elements == n
    _assert_same_map(hm, ref)
    # upsert with 40-byte values: no fast form for them, the per-row protocol runs instead - same result
    vals2 = vals + 1
    assert lib.dok_map_set_bulk(desc, k.data_ptr(), torch.from_numpy(vals2).to(cuda).data_ptr(), n, ws.data_ptr(), need, st) == 0
    ref.set(keys, vals2)
    _assert_same_map(hm, ref)
    assert lib.dok_map_set_bulk(desc, k.data_ptr(), v.data_ptr(), n, ws.data_ptr(), need - 8, st) == _lib.DOK_EINVAL
    assert lib.dok_map_set_bulk(desc, k.data_ptr(), v.data_ptr(), n, ws.data_ptr() + 8, need, st) == _lib.DOK_EINVAL
    assert lib.dok_map_set_bulk(desc, k.data_ptr(), v.data_ptr(), n, None, need, st) == _lib.DOK_EINVAL
    _assert_same_map(hm, ref)


# ---- bulk removal: keys partitioned by table range, lookups in table order, no per-row flags

@pytest.mark.parametrize("key_dtype,value_dtype", [(np.int64, np.float32), (np.int64, np.int64), (np.int32, np.float16),
                                                   (np.int16, np.int8)])
def test_bulk_removal_matches_oracle(cuda, bulk_always, key_dtype, value_dtype):
    """`del map[keys]` through dok_map_remove_bulk (thresholds lowered): batches with absent keys,
    keys given several times, the two key patterns that live in the table header, on tables of a few
    ranges and of many; entry count and remaining map against the oracle after every batch."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(5)
    lim = min(2**62, int(np.iinfo(key_dtype).max))
    for n, cap in ((40000, 65536), (3000, 3300), (200000, 1 << 20), (40, 64)):
        n = min(n, lim // 2)
        pool = np.unique(rng.integers(-lim, lim, size=3 * n, dtype=np.int64).astype(key_dtype))
        rng.shuffle(pool)
        keys = pool[:n].copy()
        special = np.array([0x9E3779B97F4A7C15, 0x9E3779B97F4A7C14], dtype=np.uint64).view(np.int64)
        if key_dtype == np.int64:
            keys[:2] = special                               # stored words 0 and 1: the header's side slots
            keys = np.unique(keys)
            n = keys.shape[0]
        vals = rng.integers(-100, 100, size=(n, 1)).astype(value_dtype)
        hm = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=1e9)
        ref = RefClosedHashmap(n_buckets=cap, rehash_threshold=1e9, rng=np.random.default_rng(9))
        hm.set(*_to(cuda, keys[:, None], vals))
        ref.set(keys[:, None], vals)
        for frac in (0.3, 0.5):
            m = int(n * frac)
            gone = np.concatenate([keys[rng.permutation(n)[:m]], pool[n:n + m // 3], keys[:m // 4]])   # present, absent, repeats
            if key_dtype == np.int64:
                gone = np.concatenate([gone, special[:1], special[:1]])
            rng.shuffle(gone)
            del hm[torch.from_numpy(gone[:, None]).to(cuda)]
            ref.remove(gone[:, None])
            assert hm.n_elements == ref.n_elements
            _assert_same_map(hm, ref)
            _check_get(hm, ref, np.concatenate([keys, pool[n:2 * n]])[:, None], cuda, fallback=-1)
        # what was removed can be stored again (tombstones re-used), and removed again
        hm.set(*_to(cuda, keys[:, None], vals))
        ref.set(keys[:, None], vals)
        assert hm.n_elements == ref.n_elements == n
        del hm[torch.from_numpy(keys[:, None]).to(cuda)]
        assert hm.n_elements == 0 and hm.items()[0].shape[0] == 0


def test_bulk_removal_of_coordinate_rows_and_rejections(cuda, bulk_always):
    """The same on a coordinate-keyed tensor (key rows are linearised on the way; rows outside the
    size are ignored), and the entry point's argument checks."""
    from doksparse_amd import SparseDOKTensor, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    g = torch.Generator().manual_seed(3)
    size = (300, 40, 25)
    flat = torch.randperm(300 * 40 * 25, generator=g)[:60000]
    idx = torch.stack(torch.unravel_index(flat, size))
    vals = torch.randn(60000, generator=g)
    dok = SparseDOKTensor(size, idx.to(cuda), vals.to(cuda), device=cuda)
    hm = dok.storage()
    gone = torch.cat([idx[:, :25000].T, torch.tensor([[300, 0, 0], [-1, 5, 5], [5, 40, 1]]), idx[:, :100].T]).contiguous().to(cuda)
    del hm[gone]
    assert dok._nnz() == 35000
    dense = torch.zeros(size)
    dense[tuple(idx[:, 25000:])] = vals[25000:]
    assert torch.equal(dok.to_dense().cpu(), dense)
    desc = ctypes.byref(hm._desc)
    need = int(lib.dok_bulk_workspace_bytes(desc, gone.shape[0]))
    ws = torch.empty(need, device=cuda, dtype=torch.uint8)
    assert lib.dok_map_remove_bulk(desc, gone.data_ptr(), gone.shape[0], ws.data_ptr(), need - 1, None) == _lib.DOK_EINVAL
    assert lib.dok_map_remove_bulk(desc, None, gone.shape[0], ws.data_ptr(), need, None) == _lib.DOK_EINVAL
    assert lib.dok_map_remove_bulk(desc, gone.data_ptr(), 0, ws.data_ptr(), need, None) == _lib.DOK_OK
    from doksparse_amd import CudaClosedHashmap
    hm2 = CudaClosedHashmap(n_buckets=256, device=cuda)
    hm2.set(torch.rand(10, 3, device=cuda), torch.zeros(10, 5, device=cuda, dtype=torch.long))
    assert lib.dok_map_remove_bulk(ctypes.byref(hm2._desc), gone.data_ptr(), 10, ws.data_ptr(), need, None) == _lib.DOK_EUNSUPPORTED
    torch.cuda.synchronize()
    assert dok._nnz() == 35000
