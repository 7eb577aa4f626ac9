"""GPU parity: the HIP hashmap (through the C ABI) against the CPU oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle.ref_hashmap import RefClosedHashmap

pytestmark = pytest.mark.gpu


def _sorted_items(keys, values):
    """Order-independent view of a key->value map: rows sorted by key bytes."""
    n = keys.shape[0]
    k = np.ascontiguousarray(keys).reshape(n, int(np.prod(keys.shape[1:])))
    v = np.ascontiguousarray(values).reshape(n, int(np.prod(values.shape[1:])))
    kb = k.view(np.uint8).reshape(n, k.shape[1] * k.itemsize)
    order = np.lexsort(kb.T[::-1])
    return k[order], v[order]


def _assert_same_map(hm, ref):
    keys, values = hm.items()
    rk, rv = ref.keys(), ref.values()
    assert hm.n_elements == ref.n_elements == keys.shape[0] == rk.shape[0]
    a = _sorted_items(keys.cpu().numpy(), values.cpu().numpy())
    b = _sorted_items(rk, rv)
    assert np.array_equal(a[0].view(np.uint8), b[0].view(np.uint8)), "key sets differ"
    assert np.array_equal(a[1].view(np.uint8), b[1].view(np.uint8)), "values differ"


def _unique_i64(rng, n, hi=2**62):
    k = np.unique(rng.integers(0, hi, size=int(n * 1.01) + 16, dtype=np.int64))
    rng.shuffle(k)
    assert k.shape[0] >= n
    return k[:n]


def test_cfg1_int64_scalar_keys(cuda):
    """65,536 unique int64 keys -> int64 values, capacity 131,072: set all, get those plus
    65,536 absent keys, remove a random half, get again."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(1001)
    n = 65536
    allk = _unique_i64(rng, 2 * n)
    present, absent = allk[:n], allk[n:]
    vals = rng.integers(-2**62, 2**62, size=(n, 1), dtype=np.int64)

    hm = CudaClosedHashmap(n_buckets=131072, device=cuda)
    ref = RefClosedHashmap(n_buckets=131072, rng=np.random.default_rng(7))
    hm.set(torch.from_numpy(present[:, None]).to(cuda), torch.from_numpy(vals).to(cuda))
    ref.set(present[:, None], vals)
    assert hm.n_elements == ref.n_elements == n
    assert hm.n_buckets == ref.n_buckets == 131072
    _assert_same_map(hm, ref)

    q = np.concatenate([present, absent])
    q = q[rng.permutation(q.shape[0])][:, None]
    v, f = hm.get(torch.from_numpy(q).to(cuda))
    rv, rf = ref.get(q)
    assert np.array_equal(f.cpu().numpy(), rf)
    assert np.array_equal(v.cpu().numpy(), rv)
    assert f.sum().item() == n

    # a fallback row is returned for misses
    v2, _ = hm.get(torch.from_numpy(q).to(cuda), fallback_value=-5)
    rv2, _ = ref.get(q, fallback_value=-5)
    assert np.array_equal(v2.cpu().numpy(), rv2)

    gone = present[rng.permutation(n)[: n // 2]][:, None]
    m = hm.remove(torch.from_numpy(gone).to(cuda))
    rm = ref.remove(gone)
    assert np.array_equal(m.cpu().numpy(), rm)
    assert hm.n_elements == ref.n_elements == n - n // 2
    v, f = hm.get(torch.from_numpy(q).to(cuda))
    rv, rf = ref.get(q)
    assert np.array_equal(f.cpu().numpy(), rf)
    assert np.array_equal(v.cpu().numpy(), rv)
    _assert_same_map(hm, ref)


def _to(dev, *arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in arrays]


def _check_get(hm, ref, q, dev, fallback=None):
    v, f = hm.get(torch.from_numpy(q).to(dev), fallback_value=fallback)
    rv, rf = ref.get(q, fallback_value=fallback)
    assert np.array_equal(f.cpu().numpy(), rf)
    assert np.array_equal(np.ascontiguousarray(v.cpu().numpy()).view(np.uint8), np.ascontiguousarray(rv).view(np.uint8))


@pytest.mark.parametrize("n,capacity", [(131072, 2**18), (1_000_000, 2**21)])
def test_cfg2_float_triple_keys_wide_values(cuda, n, capacity):
    """README-shaped map, at 1/8 scale and at its full size (1,000,000 keys, capacity 2^21):
    float32[3] keys hashed over raw bytes, int64[5] values (tagged layout): set, get of as many
    hits as misses, remove 25 %, get again, overwrite + re-insert."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(1002)
    keys = rng.random((n, 3), dtype=np.float32)
    keys = np.unique(keys, axis=0)
    rng.shuffle(keys)
    n = keys.shape[0]
    vals = rng.integers(0, 2**63 - 1, size=(n, 5), dtype=np.int64)
    misses = rng.random((n, 3), dtype=np.float32) + 1.0            # disjoint from [0, 1)

    hm = CudaClosedHashmap(n_buckets=capacity, device=cuda)
    ref = RefClosedHashmap(n_buckets=capacity, rng=np.random.default_rng(8))
    k, v = _to(cuda, keys, vals)
    hm.set(k, v)
    ref.set(keys, vals)
    assert hm.n_elements == ref.n_elements == n and hm.n_buckets == ref.n_buckets
    q = np.concatenate([keys, misses])[rng.permutation(2 * n)]
    _check_get(hm, ref, q, cuda)
    _check_get(hm, ref, q, cuda, fallback=-1)
    gone = keys[rng.permutation(n)[: n // 4]]
    m = hm.remove(torch.from_numpy(gone).to(cuda))
    rm = ref.remove(gone)
    assert np.array_equal(m.cpu().numpy(), rm) and hm.n_elements == ref.n_elements
    _check_get(hm, ref, q, cuda)
    _assert_same_map(hm, ref)
    # overwrite half of the survivors and re-insert the removed quarter
    again = np.unique(np.concatenate([keys[: n // 2], gone]), axis=0)    # no repeats inside the batch
    vals2 = rng.integers(0, 2**63 - 1, size=(again.shape[0], 5), dtype=np.int64)
    a, b = _to(cuda, again, vals2)
    hm.set(a, b)
    ref.set(again, vals2)
    assert hm.n_elements == ref.n_elements
    _assert_same_map(hm, ref)


@pytest.mark.parametrize("key_shape,key_dtype,value_shape,value_dtype", [
    ((1,), np.int64, (1,), np.float32),
    ((1,), np.int64, (1,), np.float64),
    ((1,), np.int64, (1,), np.float16),
    ((1,), np.int64, (1,), np.int8),
    ((1,), np.int32, (1,), np.int32),
    ((2,), np.int32, (1,), np.int64),
    ((1,), np.int16, (2,), np.int16),
    ((2,), np.int64, (1,), np.float32),
    ((4,), np.int64, (1,), np.float16),
    ((3,), np.int16, (3,), np.int8),
    ((5,), np.int8, (7,), np.int8),
    ((1,), np.float64, (3,), np.float32),
])
def test_random_op_sequences_all_layouts(cuda, key_shape, key_dtype, value_shape, value_dtype):
    """Random interleaved set / get / remove batches with many repeated keys, growing from 16
    slots through several rehashes; state compared with the oracle after every step."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(77)
    hm = CudaClosedHashmap(n_buckets=16, device=cuda)
    ref = RefClosedHashmap(n_buckets=16, rng=np.random.default_rng(3))
    universe = rng.integers(0, 40, size=(400, *key_shape)).astype(key_dtype)
    for step in range(30):
        op = rng.integers(0, 3)
        idx = rng.permutation(universe.shape[0])[: rng.integers(0, 90)]
        ks = int(np.prod(key_shape))
        keys = np.unique(universe[idx].reshape(idx.shape[0], ks), axis=0).reshape(-1, *key_shape)
        if op <= 1:
            vals = rng.integers(-100, 100, size=(keys.shape[0], *value_shape)).astype(value_dtype)
            k, v = _to(cuda, keys, vals)
            hm.set(k, v)
            ref.set(keys, vals)
        elif hm._allocated:
            m = hm.remove(torch.from_numpy(keys).to(cuda))
            rm = ref.remove(keys)
            assert np.array_equal(m.cpu().numpy(), rm)
        if hm._allocated:
            assert hm.n_elements == ref.n_elements
            assert hm.n_buckets == ref.n_buckets
            _check_get(hm, ref, universe, cuda, fallback=-7)
            _assert_same_map(hm, ref)


def test_equal_keys_inside_one_batch(cuda):
    """Every key 64 times in one set batch: one slot per key, holding one of its values."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(5)
    for key_shape, vshape, vdtype in [((1,), (1,), np.int64), ((3,), (5,), np.int64)]:
        base = np.unique(rng.integers(0, 2**40, size=(3000, *key_shape), dtype=np.int64), axis=0)[:2048]
        keys = np.repeat(base, 64, axis=0)
        perm = rng.permutation(keys.shape[0])
        keys = keys[perm]
        # value rows carry (key id, copy id) so that a torn row would be visible
        ids = np.repeat(np.arange(base.shape[0]), 64)[perm]
        copy = rng.integers(0, 2**30, size=keys.shape[0])
        vals = np.stack([ids * 2**32 + copy] * int(np.prod(vshape)), axis=1).reshape(-1, *vshape).astype(vdtype)
        hm = CudaClosedHashmap(n_buckets=8192, device=cuda)
        k, v = _to(cuda, keys, vals)
        hm.set(k, v)
        assert hm.n_elements == base.shape[0]
        gk, gv = hm.items()
        assert gk.shape[0] == base.shape[0]
        out, found = hm.get(torch.from_numpy(base).to(cuda))
        assert bool(found.all())
        out = out.cpu().numpy().reshape(base.shape[0], -1)
        assert (out == out[:, :1]).all(), "a value row mixes two writers"
        written = {}
        for i_, c_ in zip(ids, copy):
            written.setdefault(int(i_), set()).add(int(c_))
        for i_ in range(base.shape[0]):
            assert out[i_, 0] >> 32 == i_ and int(out[i_, 0] & (2**32 - 1)) in written[i_]
        # a second identical batch changes nothing but values
        hm.set(k, v)
        assert hm.n_elements == base.shape[0]
        # removing with repeats removes each key once
        m = hm._remove_rows(k)
        assert int(m.sum().item()) == base.shape[0] and hm.n_elements == 0


def test_reserved_patterns_and_extreme_keys(cuda):
    """The packed layout keeps two key patterns in side slots; they and the extreme integers
    must behave like any other key."""
    from doksparse_amd import CudaClosedHashmap
    X = np.uint64(0x9E3779B97F4A7C15)
    special = np.array([X, X ^ np.uint64(1), 0, 1, np.uint64(2**64 - 1), np.uint64(2**63), np.uint64(2**63 - 1),
                        np.uint64(2**64 - 3)], dtype=np.uint64).view(np.int64)[:, None]
    vals = np.arange(1, special.shape[0] + 1, dtype=np.float32)[:, None]
    hm = CudaClosedHashmap(n_buckets=64, device=cuda)
    ref = RefClosedHashmap(n_buckets=64)
    k, v = _to(cuda, special, vals)
    hm.set(k, v)
    ref.set(special, vals)
    assert hm.n_elements == ref.n_elements == special.shape[0]
    _check_get(hm, ref, special, cuda)
    _assert_same_map(hm, ref)
    hm.set(k, v * 2)                                    # overwrite: still 8 entries
    ref.set(special, vals * 2)
    assert hm.n_elements == special.shape[0]
    _check_get(hm, ref, special, cuda)
    m = hm.remove(k[:3])
    rm = ref.remove(special[:3])
    assert np.array_equal(m.cpu().numpy(), rm) and hm.n_elements == ref.n_elements
    _check_get(hm, ref, special, cuda, fallback=9)
    _assert_same_map(hm, ref)
    hm.rehash(256)                                      # side slots survive a rehash
    assert hm.n_elements == ref.n_elements
    _check_get(hm, ref, special, cuda)


def test_tiny_and_full_tables(cuda):
    from doksparse_amd import CudaClosedHashmap
    for vdtype in (np.float32, np.float64):
        for cap in (1, 2, 3, 8):
            hm = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=1.0)
            ref = RefClosedHashmap(n_buckets=cap, rehash_threshold=1.0)
            keys = (np.arange(cap, dtype=np.int64) * 1000003 + 17)[:, None]
            vals = np.arange(cap, dtype=vdtype)[:, None] + 0.5
            k, v = _to(cuda, keys, vals)
            hm.set(k, v)
            ref.set(keys, vals)
            assert hm.n_elements == ref.n_elements == cap and hm.n_buckets == cap
            q = np.concatenate([keys, keys + 1])
            _check_get(hm, ref, q, cuda)
            # tombstone everything, then reuse the slots
            assert bool(hm.remove(k).all()) and hm.n_elements == 0
            v2, f2 = hm.get(torch.from_numpy(q).to(cuda))
            assert not bool(f2.any())
            hm.set(k + 5, v)
            assert hm.n_elements == cap
            v3, f3 = hm.get(k + 5)
            assert bool(f3.all()) and torch.equal(v3, v)
    # a table that is physically full reports it
    hm = CudaClosedHashmap(n_buckets=8, device=cuda, rehash_threshold=100.0)
    n_slots = 10   # one packed bucket of 8-byte keys / 4-byte values
    keys = torch.arange(n_slots + 6, device=cuda)[:, None]
    with pytest.raises(RuntimeError, match="full: 6 rows"):      # raised by the call that overflowed
        hm.set(keys, torch.ones(n_slots + 6, 1, device=cuda))
    assert hm.n_elements == n_slots                               # reported once; the map stays usable
    _, f = hm.get(keys)
    assert int(f.sum().item()) == n_slots


def test_api_edges(cuda):
    from doksparse_amd import CudaClosedHashmap
    hm = CudaClosedHashmap(n_buckets=32, device=cuda)
    hm.set(torch.zeros(0, 1, dtype=torch.long, device=cuda), torch.zeros(0, 1, device=cuda))
    assert hm.n_elements == 0 and hm.key_shape == (1,) and hm.value_type == torch.float32
    v, f = hm.get(torch.zeros(0, 1, dtype=torch.long, device=cuda))
    assert v.shape == (0, 1) and f.shape == (0,) and f.dtype == torch.bool
    assert hm.remove(torch.zeros(0, 1, dtype=torch.long, device=cuda)).shape == (0,)
    with pytest.raises(AssertionError):
        hm.set(torch.zeros(2, 1, dtype=torch.int32, device=cuda), torch.zeros(2, 1, device=cuda))
    with pytest.raises(AssertionError):
        hm.get(torch.zeros(2, 2, dtype=torch.long, device=cuda))
    hm[torch.tensor([[4], [6]], device=cuda)] = torch.tensor([[1.0], [2.0]], device=cuda)
    v, f = hm[torch.tensor([[6], [5]], device=cuda)]
    assert v.flatten().tolist() == [2.0, 0.0] and f.tolist() == [True, False]
    mask = hm.remove(torch.tensor([[6], [9], [6], [4]], device=cuda))     # over sorted unique rows 4, 6, 9
    assert mask.tolist() == [True, True, False] and len(hm) == 0
    # clone: shallow shares the table, deep does not
    hm.set(torch.tensor([[1]], device=cuda), torch.tensor([[3.0]], device=cuda))
    sh, dp = hm.clone(), hm.clone(deepclone=True)
    hm.set(torch.tensor([[2]], device=cuda), torch.tensor([[4.0]], device=cuda))
    assert sh.n_elements == 2 and dp.n_elements == 1
    assert hm.load_factor == 2 / 32
    # non-contiguous inputs are accepted
    kk = torch.arange(20, device=cuda).reshape(10, 2)[:, :1]
    hm.set(kk, torch.ones(10, 1, device=cuda))
    assert bool(hm.get(kk)[1].all())
    assert hm.count_existing(torch.arange(0, 25, device=cuda)[:, None]).item() == sum(
        1 for x in range(25) if x in {1, 2} | set(range(0, 20, 2)))
    # del hm[keys]: rows may repeat and may be absent
    before = hm.n_elements
    del hm[torch.tensor([[2], [2], [18], [99]], device=cuda)]
    assert hm.n_elements == before - 2
    assert hm.get(torch.tensor([[2], [18], [1]], device=cuda))[1].tolist() == [False, False, True]
    del hm[torch.zeros(0, 1, dtype=torch.long, device=cuda)]
    with pytest.raises(AssertionError):
        del hm[torch.zeros(2, 2, dtype=torch.long, device=cuda)]


def test_probe_stats_are_in_the_expected_band(cuda):
    """Mean buckets visited per lookup at load factor 0.5 with 10-slot buckets is barely above 1."""
    from doksparse_amd import CudaClosedHashmap
    g = torch.Generator(device=cuda).manual_seed(3)
    n = 1 << 20
    keys = torch.unique(torch.randint(0, 2**62, (n + 4096,), generator=g, device=cuda))[:n, None]
    hm = CudaClosedHashmap(n_buckets=2 * n, device=cuda, rehash_threshold=1.0)
    hm.set(keys, torch.randn(n, 1, device=cuda))
    hits = hm.probe_stats(keys)
    misses = hm.probe_stats(torch.randint(0, 2**62, (n, 1), generator=g, device=cuda))
    assert 1.0 <= hits < 1.05 and 1.0 <= misses < 1.1


def test_get_and_set_inside_a_hip_graph(cuda):
    """The entry points allocate nothing and only enqueue kernels, so they can be captured: a
    captured clear + set + get is replayed several times, with eager work and synchronisation
    between the replays, and every replay must equal the eager result."""
    import ctypes
    from doksparse_amd import CudaClosedHashmap, _lib
    lib = _lib.load()
    g = torch.Generator(device=cuda).manual_seed(11)
    n = 100_000
    keys = torch.unique(torch.randint(0, 2**62, (n + 1000,), generator=g, device=cuda))[:n].contiguous()
    vals = torch.randn(n, generator=g, device=cuda)
    q = torch.cat([keys[: n // 2], torch.randint(0, 2**62, (n // 2,), generator=g, device=cuda)]).contiguous()
    hm = CudaClosedHashmap(n_buckets=2 * n, device=cuda, rehash_threshold=1.0)
    hm.set(keys[:, None], vals[:, None])
    eager_v, eager_f = hm.get(q[:, None])
    out_v = torch.zeros(n, 1, device=cuda)
    out_f = torch.zeros(n, device=cuda, dtype=torch.bool)
    desc = ctypes.byref(hm._desc)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            assert lib.dok_table_clear(desc, st) == 0
            assert lib.dok_map_set(desc, keys.data_ptr(), vals.data_ptr(), n, None, st) == 0
            assert lib.dok_map_get(desc, q.data_ptr(), n, out_v.data_ptr(), None, out_f.data_ptr(), st) == 0
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(4):
        out_v.zero_()
        out_f.zero_()
        if rep == 2:
            vals.mul_(2.0)                      # the graph reads the buffers, not a snapshot
            eager_v = eager_v * 2.0
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_f, eager_f) and torch.equal(out_v, eager_v)
        assert hm.n_elements == n               # the captured clear + set rebuilt the table
        (torch.randn(1000, device=cuda) @ torch.randn(1000, device=cuda)).item()   # unrelated eager work


def test_growth_from_a_small_table_counts_distinct_keys_like_the_reference(cuda):
    """A large batch with repeats into a 1024-slot map: the growth target is computed from the
    number of distinct new keys, exactly as the reference's get + unique pre-pass does."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(21)
    base = np.unique(rng.integers(0, 2**62, size=200_000, dtype=np.int64))
    keys = base[rng.integers(0, base.shape[0], size=400_000)][:, None]      # many repeats
    n_distinct = np.unique(keys).shape[0]
    for coord in (False, True):
        if coord:
            k = np.stack([keys[:, 0] % 100_003, (keys[:, 0] >> 20) % 99_991], axis=1)
            n_distinct = np.unique(k, axis=0).shape[0]
            hm = CudaClosedHashmap(n_buckets=1024, device=cuda, coord_dims=(100_003, 99_991))
        else:
            k = keys
            hm = CudaClosedHashmap(n_buckets=1024, device=cuda)
        vals = np.zeros((k.shape[0], 1), dtype=np.float32)
        hm.set(torch.from_numpy(k).to(cuda), torch.from_numpy(vals).to(cuda))
        assert hm.n_elements == n_distinct
        assert hm.n_buckets == int(n_distinct * 2.0)
        # a second batch: half known keys, half new ones, again with repeats
        k2 = np.concatenate([k[:50_000], k[:50_000] + 1])
        hm.set(torch.from_numpy(k2).to(cuda), torch.from_numpy(np.ones((k2.shape[0], 1), dtype=np.float32)).to(cuda))
        merged = np.unique(np.concatenate([k, k2]), axis=0).shape[0]
        assert hm.n_elements == merged


def test_permute_keys(cuda):
    from doksparse_amd import CudaClosedHashmap
    g = torch.Generator(device=cuda).manual_seed(5)
    keys = torch.unique(torch.randint(0, 50, (400, 3), generator=g, device=cuda), dim=0)
    vals = torch.arange(keys.shape[0], device=cuda, dtype=torch.float32)[:, None]
    hm = CudaClosedHashmap(n_buckets=2048, device=cuda)
    hm.set(keys, vals)
    hm.permute_keys([2, 0, 1])
    v, f = hm.get(keys[:, [2, 0, 1]])
    assert bool(f.all()) and torch.equal(v, vals) and hm.n_elements == keys.shape[0]
    assert not bool(hm.get(keys + 100)[1].any())


@pytest.mark.parametrize("vdtype", [np.float32, np.int64, np.float16])
def test_completely_full_tables_exercise_far_displacements(cuda, vdtype):
    """Tables filled to the last physical slot: the last keys land dozens of buckets past their
    home, beyond the 31 displacements the home bucket's map can name, so lookups take the far
    walk.  Then tombstone churn at 100 % load."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(31)
    probe = CudaClosedHashmap(n_buckets=1, device=cuda)
    probe.set(torch.zeros(1, 1, dtype=torch.long, device=cuda), torch.zeros(1, 1, device=cuda).to(torch.from_numpy(np.zeros(1, vdtype)).dtype))
    slots = probe._slots_per_bucket
    # (buckets, rows per set call).  One call for all rows: the waves race, and where the last keys
    # end up differs from run to run.  One row per call: a fixed order, the same table every
    # time - that case must show a far displacement.
    # (700 buckets: displacements beyond the 254 the metadata records, where the walk runs to the
    # ring's end)
    for n_phys, step in ((40, None), (64, None), (200, None), (700, None), (120, 1)):
        cap = n_phys * slots                                   # every physical slot
        keys = np.unique(rng.integers(0, 2**62, size=cap + 64, dtype=np.int64))[:cap, None]
        vals = rng.integers(-100, 100, size=(cap, 1)).astype(vdtype)
        hm = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=1.0, seed=77)
        ref = RefClosedHashmap(n_buckets=cap, rehash_threshold=1.0, rng=np.random.default_rng(1))
        k, v = _to(cuda, keys, vals)
        for lo in range(0, cap, step or cap):
            hm.set(k[lo: lo + (step or cap)], v[lo: lo + (step or cap)])
        ref.set(keys, vals)
        assert hm.n_elements == ref.n_elements == cap
        assert hm._n_phys == n_phys
        meta = hm._table.view(torch.int64).reshape(n_phys, 16)[:, 15].cpu().numpy()
        if step:
            assert (meta & 1).any(), "no far displacement was produced; the test lost its point"
        q = np.concatenate([keys, rng.integers(0, 2**62, size=(cap, 1), dtype=np.int64)])
        _check_get(hm, ref, q, cuda, fallback=-3)
        assert hm.probe_stats(torch.from_numpy(q).to(cuda)) >= 1.0
        for _ in range(3):                                      # churn at full load
            gone = keys[rng.permutation(cap)[: cap // 3]]
            m = hm.remove(torch.from_numpy(gone).to(cuda))
            assert np.array_equal(m.cpu().numpy(), ref.remove(gone))
            fresh = np.unique(rng.integers(0, 2**62, size=cap, dtype=np.int64))[: gone.shape[0], None]
            fv = rng.integers(-100, 100, size=(fresh.shape[0], 1)).astype(vdtype)
            a, b = _to(cuda, fresh, fv)
            hm.set(a, b)
            ref.set(fresh, fv)
            keys = np.concatenate([np.setdiff1d(keys[:, 0], gone[:, 0]), fresh[:, 0]])[:, None]
            assert hm.n_elements == ref.n_elements == cap
            _check_get(hm, ref, q, cuda)
            _check_get(hm, ref, keys, cuda)
        _assert_same_map(hm, ref)


@pytest.mark.parametrize("granule", [128, 64, 32])
def test_line_gather_measurement_kernel_reads_the_lines_it_claims(cuda, granule):
    """dok_line_gather / dok_line_gather_granule: out[i] = XOR of the 8-byte words (folded to 32 bits)
    of granule (fmix64(i ^ seed) >> 32) * n_granules >> 32 of the bucket array, recomputed here from
    a copy of the table."""
    import ctypes
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    rng = np.random.default_rng(77)
    k = _unique_i64(rng, 5000)
    hm = CudaClosedHashmap(n_buckets=10000, device=cuda)
    hm.set(torch.from_numpy(k[:, None]).to(cuda), torch.from_numpy(k[:, None].astype(np.float32)).to(cuda))
    n, seed = 4099, 987654321
    out = torch.zeros(n, device=cuda, dtype=torch.int32)
    lib = _lib.load()
    if granule == 128:
        _lib.check(lib.dok_line_gather(ctypes.byref(hm._desc), n, seed, out.data_ptr(), _stream_ptr(cuda)), "line_gather")
    else:
        _lib.check(lib.dok_line_gather_granule(ctypes.byref(hm._desc), n, seed, granule, out.data_ptr(),
                                               _stream_ptr(cuda)), "line_gather")
    words = granule // 8
    n_gran = hm._n_phys * (128 // granule)
    table = hm._table.view(torch.int64).reshape(n_gran, words).cpu().numpy().view(np.uint64)
    M = (1 << 64) - 1
    expect = np.empty(n, dtype=np.uint32)
    for i in range(n):
        x = (i ^ seed) & M
        x ^= x >> 33; x = (x * 0xff51afd7ed558ccd) & M
        x ^= x >> 33; x = (x * 0xc4ceb9fe1a85ec53) & M
        x ^= x >> 33
        line = ((x >> 32) * n_gran) >> 32
        w = int(np.bitwise_xor.reduce(table[line]))
        expect[i] = (w ^ (w >> 32)) & 0xffffffff
    assert np.array_equal(out.cpu().numpy().view(np.uint32), expect)
    assert lib.dok_line_gather_granule(ctypes.byref(hm._desc), n, seed, 48, out.data_ptr(), None) == _lib.DOK_EINVAL


def test_calls_replay_inside_a_hip_graph(cuda):
    """The library neither allocates nor synchronises, so get / set / remove can be captured in a
    HIP graph.  Every replay (with eager work and synchronisation between replays) must equal the
    eager result and the oracle."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(4242)
    n = 20000
    allk = _unique_i64(rng, 5 * n)
    hm = CudaClosedHashmap(n_buckets=8 * n, device=cuda, rehash_threshold=1.0)
    ref = RefClosedHashmap(n_buckets=8 * n, rng=np.random.default_rng(3), rehash_threshold=1.0)
    k0 = allk[:n, None]
    v0 = rng.standard_normal((n, 1)).astype(np.float32)
    hm.set(torch.from_numpy(k0).to(cuda), torch.from_numpy(v0).to(cuda))
    ref.set(k0, v0)

    sk = torch.zeros(n, 1, device=cuda, dtype=torch.int64)      # static inputs of the graph
    sv = torch.zeros(n, 1, device=cuda, dtype=torch.float32)
    sq = torch.zeros(2 * n, 1, device=cuda, dtype=torch.int64)
    sg = torch.zeros(n // 2, 1, device=cuda, dtype=torch.int64)
    sk.copy_(torch.from_numpy(k0)); sv.copy_(torch.from_numpy(v0)); sq[:n].copy_(sk); sg.copy_(sk[: n // 2])
    # eager warm-up of every kernel the graph will hold (module load must not happen in capture)
    hm._launch_set(sk, sv)
    hm.get(sq)
    hm._remove_rows(sg)
    hm._launch_set(sk, sv)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hm._launch_set(sk, sv)
        removed = hm._remove_rows(sg)
        values, found = hm.get(sq)
    torch.cuda.synchronize()

    for r in range(1, 4):
        newk = allk[r * n:(r + 1) * n, None]
        newv = rng.standard_normal((n, 1)).astype(np.float32)
        gone = np.concatenate([allk[(r - 1) * n:(r - 1) * n + n // 4, None], newk[: n // 4]])
        q = np.concatenate([allk[: 2 * n: 2, None], allk[3 * n:4 * n, None]])
        sk.copy_(torch.from_numpy(newk)); sv.copy_(torch.from_numpy(newv))
        sg.copy_(torch.from_numpy(gone)); sq.copy_(torch.from_numpy(q))
        graph.replay()
        torch.cuda.synchronize()
        ref.set(newk, newv)
        rrem = ref.remove(gone)            # unique rows: the mask is a permutation of the aligned one
        rv, rf = ref.get(q)
        assert int(removed.sum().item()) == int(rrem.sum())
        assert np.array_equal(found.cpu().numpy(), rf)
        assert np.array_equal(values.cpu().numpy()[rf], rv[rf])
        ev, ef = hm.get(sq.clone())        # eager work between replays
        assert torch.equal(ef, found) and torch.equal(ev[ef], values[found])
        assert hm.n_elements == ref.n_elements
        _assert_same_map(hm, ref)


@pytest.mark.parametrize("capacity", [150, 3000, 20000])
def test_keys_beyond_freed_slots_are_overwritten_not_duplicated(cuda, capacity):
    """At 95 % load many keys sit buckets past their home.  Removing other keys leaves tombstones
    in front of them; a later set of such a key meets a free slot before it reaches the key and
    must still find the key (through the home bucket's displacement map), not store it twice.
    Three rounds of remove / overwrite / re-insert with equal keys in the batches."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(capacity)
    n = int(capacity * 0.95)
    keys = _unique_i64(rng, n)[:, None]
    vals = rng.integers(-1000, 1000, size=(n, 1)).astype(np.int32)
    hm = CudaClosedHashmap(n_buckets=capacity, device=cuda, rehash_threshold=1.0)
    ref = RefClosedHashmap(n_buckets=capacity, rehash_threshold=1.0, rng=np.random.default_rng(1))
    hm.set(*_to(cuda, keys, vals)); ref.set(keys, vals)
    for rnd in range(3):
        gone = keys[rng.permutation(n)[: n // 2]]
        m = hm.remove(torch.from_numpy(gone).to(cuda))
        assert np.array_equal(m.cpu().numpy(), ref.remove(gone))
        # every key again, each twice with the same value: half are overwrites of keys that now
        # have tombstones in front of them, half go back into tombstones
        again = np.concatenate([keys, keys])[rng.permutation(2 * n)]
        v2 = ((again * 7 + rnd) % 1000).astype(np.int32)
        hm.set(*_to(cuda, again, v2)); ref.set(again, v2)
        assert hm.n_elements == ref.n_elements == n
        _assert_same_map(hm, ref)
        ks, _ = hm.items()
        assert np.unique(ks.cpu().numpy()).shape[0] == n       # no key in two slots
        _check_get(hm, ref, keys, cuda, fallback=0)


def test_tagged_map_grows_on_the_device_like_the_reference(cuda):
    """A multi-word map that starts small: every growth re-inserts the entries with the
    device-side rehash; sizes, contents and lookups follow the oracle through the growths,
    through removals and through an explicit rehash."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(77)
    hm = CudaClosedHashmap(n_buckets=64, device=cuda)
    ref = RefClosedHashmap(n_buckets=64, rng=np.random.default_rng(9))
    pool = np.unique(rng.integers(-2**40, 2**40, size=(60000, 3), dtype=np.int64), axis=0)
    rng.shuffle(pool)
    done = 0
    for step, n in enumerate((10, 100, 1000, 7000, 30000)):
        keys = pool[done: done + n]
        done += n
        vals = rng.standard_normal((n, 2)).astype(np.float32)
        hm.set(*_to(cuda, keys, vals)); ref.set(keys, vals)
        assert hm.n_buckets == ref.n_buckets and hm.n_elements == ref.n_elements == done
        if step == 3:
            gone = pool[:done][rng.permutation(done)[: done // 3]]
            m = hm.remove(torch.from_numpy(gone).to(cuda))
            assert np.array_equal(m.cpu().numpy(), ref.remove(gone))
            done_live = hm.n_elements
            assert done_live == ref.n_elements
            # the removed keys go back in with the next batch
            pool = np.concatenate([pool[:done][~_isin_rows(pool[:done], gone)], pool[done:], gone])
            done = done_live
    _assert_same_map(hm, ref)
    q = np.concatenate([pool[:done], rng.integers(2**41, 2**42, size=(5000, 3), dtype=np.int64)])
    _check_get(hm, ref, q, cuda)
    hm.rehash(3 * hm.n_buckets); ref.rehash(3 * ref.n_buckets)
    assert hm.n_buckets == ref.n_buckets and hm.n_elements == ref.n_elements
    _check_get(hm, ref, q, cuda)
    _assert_same_map(hm, ref)


def _isin_rows(a, b):
    """Mask over the rows of `a` that occur among the rows of `b`."""
    va = np.ascontiguousarray(a).view([("", a.dtype)] * a.shape[1]).ravel()
    vb = np.ascontiguousarray(b).view([("", b.dtype)] * b.shape[1]).ravel()
    return np.isin(va, vb)


@pytest.mark.parametrize("kshape,kdt,vshape,vdt", [
    ((3,), np.float32, (5,), np.int64),        # 2 slots of 8 words per bucket
    ((2,), np.int64, (1,), np.float32),        # 4 slots of 4 words
    ((13,), np.int64, (1,), np.float16),       # 1 slot of 15 words (no filter word)
])
def test_full_multiword_tables_take_the_far_walk(cuda, kshape, kdt, vshape, vdt):
    """Multi-word tables filled to the last physical slot: the last keys land dozens to hundreds of
    buckets past their home - beyond the 23 displacements with a bit of their own, and (in the
    larger tables) beyond the 254 the metadata can record, where a lookup walks on to the ring's
    end.  Then tombstone churn at 100 % load.  Everything against the oracle."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(41)
    probe = CudaClosedHashmap(n_buckets=1, device=cuda)
    probe.set(torch.zeros((1, *kshape), dtype=torch.from_numpy(np.zeros(1, kdt)).dtype, device=cuda),
              torch.zeros((1, *vshape), dtype=torch.from_numpy(np.zeros(1, vdt)).dtype, device=cuda))
    slots = probe._slots_per_bucket
    for n_phys, step in ((40, None), (200, None), (700, None), (90, 1)):
        cap = n_phys * slots
        if kdt == np.float32:
            keys = rng.random((cap + 64, *kshape), dtype=np.float32)
        else:
            keys = rng.integers(-2**40, 2**40, size=(cap + 64, *kshape)).astype(kdt)
        keys = np.unique(keys, axis=0)
        rng.shuffle(keys)
        keys = keys[:cap]
        assert keys.shape[0] == cap
        vals = rng.integers(-100, 100, size=(cap, *vshape)).astype(vdt)
        hm = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=1.0, seed=77)
        ref = RefClosedHashmap(n_buckets=cap, rehash_threshold=1.0, rng=np.random.default_rng(1))
        k, v = _to(cuda, keys, vals)
        for lo in range(0, cap, step or cap):
            hm.set(k[lo: lo + (step or cap)], v[lo: lo + (step or cap)])
        ref.set(keys, vals)
        assert hm.n_elements == ref.n_elements == cap and hm._n_phys == n_phys
        words = hm._table.view(torch.int64).reshape(n_phys, 16).cpu().numpy()
        meta = (words[:, 0] >> 32) & 0xffffffff
        if step:
            assert (meta & 1).any(), "no far displacement was produced; the test lost its point"
        if kdt == np.float32:
            absent = rng.random((cap, *kshape), dtype=np.float32) + 1.0
        else:
            absent = rng.integers(2**41, 2**42, size=(cap, *kshape)).astype(kdt)
        q = np.concatenate([keys, absent])
        _check_get(hm, ref, q, cuda, fallback=-3)
        assert hm.probe_stats(torch.from_numpy(q).to(cuda)) >= 1.0
        for _ in range(3):                                      # churn at full load
            gone = keys[rng.permutation(cap)[: cap // 3]]
            m = hm.remove(torch.from_numpy(gone).to(cuda))
            assert np.array_equal(m.cpu().numpy(), ref.remove(gone))
            if kdt == np.float32:
                fresh = rng.random((gone.shape[0], *kshape), dtype=np.float32) + 2.0 + _
            else:
                fresh = np.unique(rng.integers(2**43 + _ * 2**41, 2**43 + (_ + 1) * 2**41, size=(cap, *kshape)).astype(kdt),
                                  axis=0)[: gone.shape[0]]
            fresh = np.unique(fresh, axis=0)
            assert fresh.shape[0] == gone.shape[0]
            fv = rng.integers(-100, 100, size=(fresh.shape[0], *vshape)).astype(vdt)
            a, b = _to(cuda, fresh, fv)
            hm.set(a, b)
            ref.set(fresh, fv)
            keys = np.concatenate([keys[~_isin_rows(keys, gone)], fresh])
            assert hm.n_elements == ref.n_elements == cap
            _check_get(hm, ref, q, cuda)
            _check_get(hm, ref, keys, cuda)
        _assert_same_map(hm, ref)


def test_multiword_layout_random_geometries_against_a_dict(cuda):
    """Differential test of the multi-word layout against a Python dict: random key / value widths
    (one to five slots per bucket), loads up to 99 % or growth from 64 slots, batches with equal
    keys, removals with repeats, several rounds.  After every round the whole key pool is looked
    up and compared."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(2024)
    geoms = [((3,), np.float32, (5,), np.int64), ((2,), np.int64, (1,), np.float32), ((13,), np.int64, (1,), np.float16),
             ((3,), np.int32, (1,), np.int8), ((4,), np.int64, (2,), np.int64), ((1,), np.int64, (3,), np.float32),
             ((5,), np.int16, (3,), np.int16)]
    for case in range(14):
        ks, kdt, vs, vdt = geoms[case % len(geoms)]
        universe = int(10 ** rng.uniform(2, 4.3))
        grow = case % 3 == 2
        cap = 64 if grow else int(universe / float(rng.uniform(0.3, 0.99))) + 4
        lim = 2**14 if kdt == np.int16 else 2**30
        pool = np.unique(rng.integers(-lim, lim, size=(universe, *ks)).astype(kdt), axis=0)
        universe = pool.shape[0]
        hm = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=0.75 if grow else 1e9,
                               seed=int(rng.integers(1, 1 << 40)))
        model = {}
        for rnd in range(int(rng.integers(2, 5))):
            n = int(universe * rng.uniform(0.1, 0.9)) + 1
            idx = rng.integers(0, universe, size=n)
            v = rng.integers(-100, 100, size=(n, *vs)).astype(vdt)
            hm.set(*_to(cuda, pool[idx], v))
            rows_of = {}
            for i, key in enumerate(idx.tolist()):
                rows_of.setdefault(key, []).append(i)
            uk = np.array(sorted(rows_of))
            got, f = hm.get(torch.from_numpy(pool[uk]).to(cuda))
            got = got.cpu().numpy()
            assert bool(f.all())
            for j, key in enumerate(uk.tolist()):       # each key holds the value of ONE of its rows, untorn
                assert any(np.array_equal(v[r].view(np.uint8), got[j].view(np.uint8)) for r in rows_of[key]), (case, rnd, key)
                model[key] = got[j].copy()
            assert hm.n_elements == len(model)
            gidx = rng.integers(0, universe, size=int(universe * rng.uniform(0.05, 0.6)) + 1)
            mask = hm._remove_rows(torch.from_numpy(pool[gidx]).to(cuda).contiguous()).cpu().numpy()
            gone = set(gidx.tolist())
            assert int(mask.sum()) == len(gone & set(model))       # repeated keys are removed once
            for key in gone:
                model.pop(key, None)
            assert hm.n_elements == len(model)
            allv, allf = hm.get(torch.from_numpy(pool).to(cuda))
            allv, allf = allv.cpu().numpy(), allf.cpu().numpy()
            present = np.zeros(universe, dtype=bool)
            present[list(model)] = True
            assert np.array_equal(allf, present), (case, rnd)
            for key, val in model.items():
                assert np.array_equal(allv[key].view(np.uint8), val.view(np.uint8)), (case, rnd, key)
        assert hm.items()[0].shape[0] == len(model)


@pytest.mark.parametrize("kshape,kdt,vshape,vdt", [((3,), np.float32, (5,), np.int64), ((2,), np.int64, (1,), np.float32),
                                                   ((9,), np.int64, (3,), np.int16)])
def test_multiword_rehash_into_a_table_without_a_free_slot_to_spare(cuda, kshape, kdt, vshape, vdt):
    """rehash(n_elements): the device-side rehash fills the new table to (nearly) its last slot, so
    rows walk far from their home buckets and leave far displacement records; every key must still
    be found, absent keys must not, and the map must keep working afterwards."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(31)
    n = 5000
    keys = np.unique(rng.integers(-2**20, 2**20, size=(n, *kshape)).astype(kdt), axis=0)
    n = keys.shape[0]
    vals = rng.integers(-1000, 1000, size=(n, *vshape)).astype(vdt)
    absent = (rng.integers(2**21, 2**22, size=(2000, *kshape))).astype(kdt)
    hm = CudaClosedHashmap(n_buckets=4 * n, device=cuda, rehash_threshold=1e9)
    hm.set(*_to(cuda, keys, vals))
    gone = rng.permutation(n)[: n // 5]
    hm._remove_rows(torch.from_numpy(keys[gone]).to(cuda).contiguous())       # tombstones do not travel
    live = np.ones(n, dtype=bool); live[gone] = False
    hm.rehash(int(live.sum()))
    assert hm.n_elements == int(live.sum()) and hm.n_buckets == int(live.sum())
    got, found = hm.get(torch.from_numpy(keys).to(cuda))
    assert np.array_equal(found.cpu().numpy(), live)
    assert np.array_equal(got.cpu().numpy()[live], vals[live])
    assert not bool(hm.get(torch.from_numpy(absent).to(cuda))[1].any())
    # the removed keys fit again only after a growth; overwrites work in the full table
    hm.set(*_to(cuda, keys[live][:100], vals[live][:100] + 1))
    assert np.array_equal(hm.get(torch.from_numpy(keys[live][:100]).to(cuda))[0].cpu().numpy(), vals[live][:100] + 1)
    hm.rehash(2 * n)
    hm.set(*_to(cuda, keys[gone], vals[gone]))
    assert hm.n_elements == n
    got, found = hm.get(torch.from_numpy(keys).to(cuda))
    assert bool(found.all())
    expect = vals.copy(); idx = np.flatnonzero(live)[:100]; expect[idx] += 1
    assert np.array_equal(got.cpu().numpy(), expect)


def test_raw_table_attributes_and_set_values(cuda):
    """The reference's raw-table surface (cuda_closed_hashmap.py:157-177, 233-273): keys() /
    values() / uuid() / nonempty_mask / _keys / _values / _uuid / _n_elements and set_values, whose
    selectors address the live entries in values() order."""
    from doksparse_amd import CudaClosedHashmap
    hm = CudaClosedHashmap(n_buckets=64, device=cuda)
    assert hm._keys is None and hm._values is None
    assert hm._uuid.shape == (64,) and bool((hm._uuid == hm._empty_marker).all())
    assert hm.nonempty_mask.shape == (0,)
    k = torch.arange(10, 40, device=cuda)[:, None]
    v = torch.arange(30, device=cuda, dtype=torch.float32)[:, None] * 2
    hm.set(k, v)
    hm.remove(k[:5])
    assert hm.key_type == torch.int64 and hm.value_type == torch.float32
    assert hm.key_shape == (1,) and hm.value_shape == (1,)
    assert int(hm._n_elements) == len(hm) == 25 and hm._n_elements.device.type == "cuda"
    keys, values = hm.keys(), hm.values()
    assert keys.shape == (25, 1) and values.shape == (25, 1)
    assert torch.equal(values, (keys - 10).float() * 2)                   # the two read-outs agree row by row
    assert torch.equal(hm._keys, keys) and torch.equal(hm._values, values)
    assert hm.nonempty_mask.shape == (25,) and bool(hm.nonempty_mask.all())
    assert hm.uuid().shape == (25,) and torch.equal(hm.uuid(), hm.get_uuid(keys))
    assert torch.unique(hm.uuid()).numel() == 25
    # set_values: by position in values() order, boolean or integer selectors
    sel = torch.zeros(25, dtype=torch.bool, device=cuda); sel[::3] = True
    hm.set_values(sel, torch.full((int(sel.sum()), 1), -1.0, device=cuda))
    got, found = hm.get(keys)
    assert bool(found.all())
    expect = values.clone(); expect[sel] = -1.0
    assert torch.equal(got, expect) and len(hm) == 25
    hm.set_values(torch.tensor([0, 24], device=cuda), torch.tensor([[5.0], [6.0]], device=cuda))
    keys2, values2 = hm.items()
    look = dict(zip(keys2.flatten().tolist(), values2.flatten().tolist()))
    assert look[int(keys[0])] == 5.0 and look[int(keys[24])] == 6.0


def _bytes_dict(keys, vals):
    return {k.tobytes(): v.tobytes() for k, v in zip(np.ascontiguousarray(keys), np.ascontiguousarray(vals))}


@pytest.mark.parametrize("kshape,vshape", [((1,), (1,)), ((3,), (5,))])
def test_remove_tells_float_keys_apart_by_bit_pattern(cuda, kshape, vshape):
    """The table's key identity is the key row's bytes.  `remove` must agree with it: a NaN key
    given twice in one batch is ONE key (removed once, counted once), and -0.0 / +0.0 are TWO keys
    (both removed) - `torch.unique` on the float values has both the other way round.  Checked
    against a dict keyed by the rows' bytes, on the packed layout (one float32 per key) and on the
    multi-word layout (float32[3] keys)."""
    from doksparse_amd import CudaClosedHashmap
    from doksparse_amd.closed_hashmap import unique_rows
    nan = np.float32("nan")
    width = kshape[0]
    base = np.array([nan, 0.0, -0.0, 1.5, -2.0, np.inf, -np.inf], dtype=np.float32)
    keys = np.stack([np.roll(base, s) for s in range(width)], axis=1)            # [7, width], distinct by bytes
    rng = np.random.default_rng(3)
    vals = rng.integers(1, 2**31, size=(keys.shape[0],) + vshape).astype(np.int64 if vshape[0] > 1 else np.int32)
    hm = CudaClosedHashmap(n_buckets=64, device=cuda)
    k, v = _to(cuda, keys, vals)
    hm.set(k, v)
    model = _bytes_dict(keys, vals)
    assert hm.n_elements == len(model) == 7
    got_v, got_f = hm.get(k)
    assert bool(got_f.all()) and np.array_equal(got_v.cpu().numpy(), vals)

    # the batch: the NaN row twice, both zeros, one absent key, one ordinary key twice
    absent = np.full((1, width), 7.25, dtype=np.float32)
    batch = np.concatenate([keys[0:1], keys[0:1], keys[1:2], keys[2:3], absent, keys[3:4], keys[3:4]])
    uniq = unique_rows(torch.from_numpy(batch)).numpy()
    assert uniq.shape[0] == 5                                                  # NaN once, -0.0 and +0.0 apart
    assert len({r.tobytes() for r in uniq}) == 5
    expect = np.array([r.tobytes() in model for r in uniq])
    m = hm.remove(torch.from_numpy(batch).to(cuda))
    assert np.array_equal(m.cpu().numpy(), expect)
    for r in uniq:
        model.pop(r.tobytes(), None)
    assert hm.n_elements == len(model) == 3
    rk, rv = hm.items()
    assert _bytes_dict(rk.cpu().numpy().reshape(-1, width), rv.cpu().numpy()) == model
    _, f = hm.get(k)
    assert f.cpu().numpy().tolist() == [False, False, False, False, True, True, True]
    # a batch holding a key twice that would cross the growth threshold: the exact count of distinct
    # new keys (multi-word layout: a sort of the rows) goes by bit pattern as well
    small = CudaClosedHashmap(n_buckets=8, device=cuda)
    rep = np.concatenate([keys[0:1]] * 4 + [keys[1:3]] + [keys[0:1]] * 4)       # 3 distinct keys in 10 rows
    small.set(torch.from_numpy(rep).to(cuda), torch.from_numpy(np.concatenate([vals[0:1]] * 4 + [vals[1:3]] + [vals[0:1]] * 4)).to(cuda))
    assert small.n_elements == 3 and small.n_buckets == 8                       # 3 <= int(0.75 * 8): no growth


@pytest.mark.parametrize("vshape,vdt", [((1,), np.float32), ((5,), np.int64), ((1,), np.int64), ((3,), np.int16)])
def test_device_resident_fallback_row(cuda, vshape, vdt):
    """A fallback row given as a device tensor is read by the kernel (dok_map_get_dev_fallback): same
    results as the host-side fallback, and a captured get sees the row's contents at replay time."""
    import ctypes
    from doksparse_amd import CudaClosedHashmap, _lib
    lib = _lib.load()
    rng = np.random.default_rng(17)
    n = 5000
    keys = _unique_i64(rng, 2 * n)
    vals = rng.integers(-1000, 1000, size=(n,) + vshape).astype(vdt)
    hm = CudaClosedHashmap(n_buckets=4 * n, device=cuda)
    k, v = _to(cuda, keys[:n, None], vals)
    hm.set(k, v)
    q = torch.from_numpy(keys[rng.permutation(2 * n)][:, None]).to(cuda)
    fb_host = (np.arange(vshape[0]) - 7).astype(vdt)
    want_v, want_f = hm.get(q, fallback_value=torch.from_numpy(fb_host))        # a CPU tensor: passed by value
    fb = torch.from_numpy(fb_host).to(cuda)
    got_v, got_f = hm.get(q, fallback_value=fb)
    assert torch.equal(got_f, want_f) and torch.equal(got_v, want_v)
    assert bool((got_v[~got_f] == fb).all()) and int((~got_f).sum()) == n
    # broadcast of a one-element device tensor over the value row
    one = torch.tensor([-9], device=cuda, dtype=fb.dtype)
    b_v, _ = hm.get(q, fallback_value=one)
    assert bool((b_v[~got_f] == -9).all()) and torch.equal(b_v[got_f], want_v[got_f])
    # captured: the row changes between replays
    out_v = torch.zeros_like(want_v)
    out_f = torch.zeros_like(want_f)
    desc = ctypes.byref(hm._desc)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            assert lib.dok_map_get_dev_fallback(desc, q.data_ptr(), q.shape[0], out_v.data_ptr(), fb.data_ptr(),
                                                out_f.data_ptr(), st) == 0
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(4):
        out_v.zero_()
        out_f.zero_()
        if rep % 2 == 1:
            fb.add_(100)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_f, want_f) and torch.equal(out_v[want_f], want_v[want_f])
        assert bool((out_v[~want_f] == fb).all())
        (torch.randn(1000, device=cuda) @ torch.randn(1000, device=cuda)).item()   # unrelated eager work
    # a NULL device row is refused
    assert lib.dok_map_get_dev_fallback(desc, q.data_ptr(), q.shape[0], out_v.data_ptr(), None, out_f.data_ptr(),
                                        None) == _lib.DOK_EINVAL


def test_rows_wider_than_a_bucket_against_a_dict(cuda):
    """Key + value rows that do not fit a 128-byte bucket (the reference compiles its kernels for
    any KeySize / ValueSize, closed_hashmap_impl_class.cu:7): the values then live in a side array
    and the table holds row numbers.  Differential test against a Python dict over several rounds of
    set (with equal keys in a batch), get (hits, misses, fallback row), remove (mask over the sorted
    distinct keys) and growth from 64 slots; then read-out, set_values, clones and the compaction of
    the side array after heavy churn."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(77)
    geoms = [((1,), np.int64, (40,), np.float32), ((3,), np.float32, (20,), np.int64), ((8,), np.int64, (64,), np.int16),
             ((2,), np.int64, (4, 8), np.float32), ((), np.int64, (33,), np.float64)]
    for case, (ks, kdt, vs, vdt) in enumerate(geoms):
        universe = int(10 ** rng.uniform(2.5, 3.8))
        grow = case % 2 == 0
        cap = 64 if grow else 2 * universe
        pool = rng.integers(-2**30, 2**30, size=(universe, *ks)).astype(kdt)
        pool = np.unique(pool.reshape(universe, -1), axis=0).reshape(-1, *ks)
        universe = pool.shape[0]
        hm = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=0.75 if grow else 1e9)
        model = {}
        for rnd in range(4):
            n = int(universe * rng.uniform(0.2, 0.9)) + 1
            idx = rng.integers(0, universe, size=n)
            v = rng.integers(-100, 100, size=(n, *vs)).astype(vdt)
            hm.set(*_to(cuda, pool[idx], v))
            assert tuple(hm.value_shape) == vs and hm.value_type == torch.from_numpy(v).dtype
            rows_of = {}
            for i, key in enumerate(idx.tolist()):
                rows_of.setdefault(key, []).append(i)
            uk = np.array(sorted(rows_of))
            got, f = hm.get(torch.from_numpy(pool[uk]).to(cuda))
            got = got.cpu().numpy()
            assert bool(f.all()) and got.shape == (len(uk), *vs)
            for j, key in enumerate(uk.tolist()):       # each key holds the value of ONE of its rows, untorn
                assert any(np.array_equal(v[r], got[j]) for r in rows_of[key]), (case, rnd, key)
                model[key] = got[j].copy()
            assert hm.n_elements == len(model) == len(hm)
            # remove: mask over the sorted distinct keys of the batch
            gidx = rng.integers(0, universe, size=int(universe * rng.uniform(0.05, 0.6)) + 1)
            gk = torch.from_numpy(pool[gidx]).to(cuda)
            mask = hm.remove(gk).cpu().numpy()
            distinct = np.unique(pool[gidx].reshape(len(gidx), -1), axis=0)
            index_of = {bytes(np.ascontiguousarray(pool[i]).reshape(-1)): i for i in set(gidx.tolist())}
            expect = np.array([index_of[bytes(np.ascontiguousarray(r.astype(kdt)))] in model for r in distinct])
            assert mask.shape == expect.shape and np.array_equal(mask, expect), (case, rnd)
            for key in set(gidx.tolist()):
                model.pop(key, None)
            assert hm.n_elements == len(model)
            # every key of the pool, with a fallback row for the absent ones
            fb = np.full(vs, 7, dtype=vdt)
            allv, allf = hm.get(torch.from_numpy(pool).to(cuda), fallback_value=torch.from_numpy(fb).to(cuda))
            allv, allf = allv.cpu().numpy(), allf.cpu().numpy()
            present = np.zeros(universe, dtype=bool)
            present[list(model)] = True
            assert np.array_equal(allf, present), (case, rnd)
            for key in range(universe):
                assert np.array_equal(allv[key], model[key] if key in model else fb), (case, rnd, key)
        # read-out: keys() / values() / items() in one order, equal to the model as a set of rows
        k, vals = hm.items()
        assert k.shape[0] == len(model) and vals.shape == (len(model), *vs)
        assert torch.equal(hm.values(), vals) and torch.equal(hm.keys(), k)
        back = {bytes(np.ascontiguousarray(pool[i]).reshape(-1)): val for i, val in model.items()}
        kn, vn = k.cpu().numpy(), vals.cpu().numpy()
        for j in range(kn.shape[0]):
            assert np.array_equal(vn[j], back[bytes(np.ascontiguousarray(kn[j]))])
        # clones: the shallow one shares the entries, the deep one keeps its own
        shallow, deep = hm.clone(), hm.clone(deepclone=True)
        some = pool[: min(50, universe)]
        nv = rng.integers(-5, 5, size=(some.shape[0], *vs)).astype(vdt)
        hm.set(*_to(cuda, some, nv))
        assert torch.equal(shallow.get(torch.from_numpy(some).to(cuda))[0].cpu(), torch.from_numpy(nv))
        dv, df = deep.get(torch.from_numpy(some).to(cuda))
        for j in range(some.shape[0]):
            if j in model:
                assert bool(df[j]) and np.array_equal(dv[j].cpu().numpy(), model[j])
            else:
                assert not bool(df[j])
        # set_values: overwrite the first entry of the read-out order
        k, vals = hm.items()
        first = rng.integers(-9, 9, size=vs).astype(vdt)
        hm.set_values(slice(0, 1), torch.from_numpy(first).to(cuda))
        assert torch.equal(hm.get(k[:1].reshape(1, *ks))[0][0].cpu(), torch.from_numpy(first))
        # churn: remove everything and insert again, several times - the side array is compacted instead of growing
        for _ in range(6):
            del hm[torch.from_numpy(pool).to(cuda)]
            assert hm.n_elements == 0
            v = rng.integers(-100, 100, size=(universe, *vs)).astype(vdt)
            hm.set(*_to(cuda, pool, v))
            assert hm.n_elements == universe
        assert hm._rows.shape[0] <= 6 * universe + 2048
        got, f = hm.get(torch.from_numpy(pool).to(cuda))
        assert bool(f.all()) and np.array_equal(got.cpu().numpy(), v)


def test_keys_wider_than_a_bucket_are_refused(cuda):
    """A key row of more than 112 bytes cannot be stored whatever the value width."""
    from doksparse_amd import CudaClosedHashmap
    hm = CudaClosedHashmap(n_buckets=64, device=cuda)
    with pytest.raises((RuntimeError, NotImplementedError, ValueError, AssertionError)):
        hm.set(torch.zeros(4, 15, device=cuda, dtype=torch.long), torch.zeros(4, 1, device=cuda))


@pytest.mark.parametrize("vdt", [np.float32, np.int64, np.float16])
def test_update_existing_overwrites_present_keys_and_counts_the_rest(cuda, vdt):
    """dok_map_update_existing through the C ABI: present keys take their new values, absent keys
    are counted and not inserted (the two side-slot keys included); and `set` in a table too full
    to skip the growth check: a batch of present keys only changes values and keeps the count, a
    batch with new keys still grows the table by the reference's rule."""
    import ctypes
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    from oracle.ref_hashmap import RefClosedHashmap
    rng = np.random.default_rng(5)
    n = 20_000
    keys = _unique_i64(rng, n)
    keys[:2] = np.array([0x9E3779B97F4A7C15, 0x9E3779B97F4A7C14], dtype=np.uint64).view(np.int64)   # the side-slot keys
    vals = rng.integers(-1000, 1000, size=(n, 1)).astype(vdt)
    hm = CudaClosedHashmap(n_buckets=16_000, device=cuda)          # (threshold 12,000 entries)
    ref = RefClosedHashmap(n_buckets=16_000)
    half = n // 2
    hm.set(*_to(cuda, keys[:half, None], vals[:half]))
    ref.set(keys[:half, None], vals[:half])
    # C ABI: rows 0 .. n-1, of which the first half is present
    newv = rng.integers(-1000, 1000, size=(n, 1)).astype(vdt)
    k, v = _to(cuda, keys[:, None], newv)
    missing = torch.zeros((), device=cuda, dtype=torch.long)
    lib = _lib.load()
    _lib.check(lib.dok_map_update_existing(ctypes.byref(hm._desc), k.data_ptr(), v.data_ptr(), n, missing.data_ptr(),
                                           _stream_ptr(cuda)), "update")
    assert int(missing.item()) == n - half and hm.n_elements == half
    ref.set(keys[:half, None], newv[:half])
    _assert_same_map(hm, ref)
    _check_get(hm, ref, keys[:, None], cuda)
    # a batch of present keys in a table whose growth check cannot be skipped
    assert hm._n_upper + half > hm._growth_limit()
    again = rng.integers(-1000, 1000, size=(half, 1)).astype(vdt)
    buckets_before = hm.n_buckets
    hm.set(*_to(cuda, keys[:half, None], again))
    ref.set(keys[:half, None], again)
    assert hm.n_buckets == buckets_before == ref.n_buckets and hm._n_exact and hm.n_elements == half
    _assert_same_map(hm, ref)
    # and one with new keys among them: grows like the reference
    hm.set(*_to(cuda, keys[:, None], newv))
    ref.set(keys[:, None], newv)
    assert hm.n_buckets == ref.n_buckets and hm.n_elements == ref.n_elements == n
    _assert_same_map(hm, ref)


def test_update_pass_on_a_coordinate_keyed_map(cuda):
    """The same pre-pass of `set` on a map whose keys are coordinate rows linearised by the table:
    a batch of present coordinates in a table too full to skip the growth check only changes
    values; one with new coordinates grows the table."""
    from doksparse_amd import CudaClosedHashmap
    rng = np.random.default_rng(6)
    dims = (300, 200, 7)
    lin = rng.permutation(int(np.prod(dims)))[:20_000]
    rows = np.stack(np.unravel_index(lin, dims), axis=1).astype(np.int64)
    vals = rng.standard_normal((20_000, 1)).astype(np.float32)
    hm = CudaClosedHashmap(n_buckets=16_000, device=cuda, coord_dims=dims)
    k, v = _to(cuda, rows, vals)
    hm.set(k[:10_000], v[:10_000])
    assert hm.n_elements == 10_000 and hm._n_upper + 10_000 > hm._growth_limit()
    v2 = torch.from_numpy(rng.standard_normal((10_000, 1)).astype(np.float32)).to(cuda)
    hm.set(k[:10_000], v2)                                   # only present coordinates
    assert hm.n_buckets == 16_000 and hm.n_elements == 10_000 and hm._n_exact
    got, found = hm.get(k)
    assert bool(found[:10_000].all()) and not bool(found[10_000:].any()) and torch.equal(got[:10_000], v2)
    hm.set(k, v)                                             # half of them new: the table grows
    assert hm.n_elements == 20_000 and hm.n_buckets == int((10_000 + 10_000) * 2.0)
    got, found = hm.get(k)
    assert bool(found.all()) and torch.equal(got, v)
