"""GPU checks at the full sizes of the benchmark configurations, through properties that do not
need the CPU oracle: a sorted-array lookup (torch.sort + searchsorted over linearised
coordinates) as the independent map, entry counts, and read-out round trips."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


class SortedMap:
    """key -> value by binary search over sorted unique int64 keys (independent of the table)."""
    def __init__(self, keys, values):
        self.keys, order = torch.sort(keys)
        self.values = values[order]

    def get(self, q):
        pos = torch.searchsorted(self.keys, q).clamp_(max=self.keys.numel() - 1)
        hit = self.keys[pos] == q
        return torch.where(hit, self.values[pos], torch.zeros((), dtype=self.values.dtype, device=q.device)), hit


def unique_coords(gen, dev, n, size):
    """~n distinct coordinates uniform over `size` (duplicates of the draw are dropped)."""
    strides = torch.tensor(np.cumprod((list(size[1:]) + [1])[::-1])[::-1].copy(), device=dev)
    coords = torch.stack([torch.randint(0, s, (n,), generator=gen, device=dev) for s in size])
    lin = (coords * strides[:, None]).sum(0)
    lin = torch.unique(lin)
    lin = lin[torch.randperm(lin.numel(), generator=gen, device=dev)]
    coords = torch.stack([(lin // st) % s for st, s in zip(strides.tolist(), size)])
    return coords, lin


def test_cfg4_full_size(cuda):
    """2-D 1e6 x 1e6 float32, 50M entries: construct, 4096 x 256 advanced-index gather (uniform and
    planted), scatter of 10M coordinates (overwrites + inserts), read-out round trip."""
    from doksparse_amd import SparseDOKTensor
    gen = torch.Generator(device=cuda).manual_seed(1004)
    size = (1_000_000, 1_000_000)
    coords, lin = unique_coords(gen, cuda, 50_000_000, size)
    vals = torch.randn(lin.numel(), generator=gen, device=cuda)
    dok = SparseDOKTensor(size, coords, vals, device=cuda)
    nnz = lin.numel()
    assert dok._nnz() == nnz
    assert dok.storage().n_buckets == 2**26              # 50M <= int(0.75 * 2^26): no growth
    smap = SortedMap(lin, vals)

    rows = torch.randint(0, size[0], (4096,), generator=gen, device=cuda)
    cols = torch.randint(0, size[1], (256,), generator=gen, device=cuda)
    prow, pcol = coords[0, :4096], coords[1, 1000:1256]
    for rr, cc in ((rows, cols), (prow, pcol)):
        got = dok[rr[:, None], cc[None, :]]
        exp, hit = smap.get((rr[:, None] * size[1] + cc[None, :]).reshape(-1))
        assert got.shape == (4096, 256) and torch.equal(got.reshape(-1), exp)
    assert int(hit.sum()) >= 200                          # the planted gather really hits

    # scatter: 5M stored coordinates + ~5M fresh ones
    fresh, flin = unique_coords(gen, cuda, 5_000_000, size)
    keep = ~smap.get(flin)[1]
    fresh, flin = fresh[:, keep], flin[keep]
    sc = torch.cat([coords[:, :5_000_000], fresh], dim=1)
    sv = torch.randn(sc.shape[1], generator=gen, device=cuda)
    dok[sc[0], sc[1]] = sv
    assert dok._nnz() == nnz + flin.numel()
    assert dok.storage().n_buckets == int(np.ceil((nnz + sc.shape[1]) * 2.0))   # grown as the reference would
    lin2 = torch.cat([lin[5_000_000:], lin[:5_000_000], flin])
    val2 = torch.cat([vals[5_000_000:], sv])
    smap2 = SortedMap(lin2, val2)
    probe = torch.randint(0, lin2.numel(), (4_000_000,), generator=gen, device=cuda)
    got = dok[lin2[probe] // size[1], lin2[probe] % size[1]]
    assert torch.equal(got, smap2.get(lin2[probe])[0])
    del smap, got, probe

    # read-out: the entries, sorted by coordinate, are exactly what went in
    idx, v = dok.indices(), dok.values()
    assert idx.shape == (2, lin2.numel())
    out_lin = idx[0] * size[1] + idx[1]
    order = torch.argsort(out_lin)
    assert torch.equal(out_lin[order], smap2.keys) and torch.equal(v[order], smap2.values)


def test_cfg5_full_size_churn(cuda):
    """4-D (4096, 4096, 64, 8) float16, 100M entries at load factor 0.85: mixed indexing
    dok[i, :512, idx, mask] for 64 values of i, then remove 20 % / insert as many fresh / repeat."""
    from doksparse_amd import SparseDOKTensor, CudaClosedHashmap
    gen = torch.Generator(device=cuda).manual_seed(1005)
    size = (4096, 4096, 64, 8)
    strides = (4096 * 64 * 8, 64 * 8, 8, 1)
    coords, lin = unique_coords(gen, cuda, 100_000_000, size)
    vals = torch.randn(lin.numel(), generator=gen, device=cuda).half()
    nnz = lin.numel()
    cap = int(np.ceil(nnz / 0.85))
    store = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=0.9, coord_dims=size)
    dok = SparseDOKTensor(size, coords, vals, device=cuda, storage=store)
    del coords
    assert dok._nnz() == nnz and dok.storage().n_buckets == cap

    i_list = torch.randint(0, 4096, (64,), generator=gen, device=cuda).tolist()
    sel_idx = torch.randint(0, 64, (128,), generator=gen, device=cuda)
    mask = torch.tensor([True, False, True, True, False, False, True, False], device=cuda)
    mcols = mask.nonzero()[:, 0]

    def run_gets(smap):
        hits = 0
        for i in i_list:
            got = dok[i, :512, sel_idx[:, None], mask]
            q = (i * strides[0] + torch.arange(512, device=cuda)[None, None, :] * strides[1]
                 + sel_idx[:, None, None] * strides[2] + mcols[None, :, None])
            exp, hit = smap.get(q.reshape(-1))
            assert got.shape == (128, 4, 512) and got.dtype == torch.float16
            assert torch.equal(got.reshape(-1), exp)
            hits += int(hit.sum())
        return hits

    smap = SortedMap(lin, vals)
    assert run_gets(smap) > 100            # density 1.8e-4 over 16.8M lookups
    # churn: remove 20 %, insert as many fresh coordinates
    n_gone = nnz // 5
    gone = lin[:n_gone]
    gc = torch.stack([(gone // st) % s for st, s in zip(strides, size)], dim=1)
    removed = dok.storage()._remove_rows(gc.contiguous())
    assert bool(removed.all()) and dok._nnz() == nnz - n_gone
    del gc, removed
    fresh, flin = unique_coords(gen, cuda, n_gone + n_gone // 50, size)
    keep = ~smap.get(flin)[1]
    fresh, flin = fresh[:, keep][:, :n_gone], flin[keep][:n_gone]
    fv = torch.randn(flin.numel(), generator=gen, device=cuda).half()
    dok.storage().set(fresh.T.contiguous(), fv[:, None])
    assert dok._nnz() == nnz - n_gone + flin.numel()
    assert dok.storage().n_buckets == cap
    del smap
    smap = SortedMap(torch.cat([lin[n_gone:], flin]), torch.cat([vals[n_gone:], fv]))
    assert run_gets(smap) > 100
    # removed keys are gone, fresh keys are there
    q = torch.cat([gone[:1_000_000], flin[:1_000_000]])
    qc = torch.stack([(q // st) % s for st, s in zip(strides, size)], dim=1).contiguous()
    v, f = dok.storage().get(qc)
    assert not bool(f[:1_000_000].any()) and bool(f[1_000_000:].all())
    assert torch.equal(v[1_000_000:, 0], fv[:1_000_000])


@pytest.mark.parametrize("load_factor", [0.5, 0.9])
def test_cfg3_full_size_int64_to_float32(cuda, load_factor):
    """The headline configuration: 2^26 unique int64 keys -> float32 at load factor 0.5 and 0.9.
    Build (bulk path, uninitialised table), bulk upsert on top, get of 2^26 queries (half hits, half
    misses), read-out round trip, removal of a random half, per-row re-insert of a quarter.  Every
    result is compared with the sorted-array map."""
    from doksparse_amd import CudaClosedHashmap
    gen = torch.Generator(device=cuda); gen.manual_seed(1003)
    n = 1 << 26
    draw = torch.unique(torch.randint(0, 2**62, (2 * n + (1 << 20),), generator=gen, device=cuda))
    draw = draw[torch.randperm(draw.numel(), generator=gen, device=cuda)]
    assert draw.numel() >= 2 * n
    keys, absent = draw[:n].contiguous(), draw[n: 2 * n].contiguous()
    del draw
    values = torch.randn(n, generator=gen, device=cuda)
    capacity = 2 * n if load_factor == 0.5 else int(np.ceil(n / 0.9))
    hm = CudaClosedHashmap(n_buckets=capacity, device=cuda, rehash_threshold=1.0)

    hm.set(keys[:, None], values[:, None])                       # first set: build
    assert hm.n_elements == n and hm.n_buckets == capacity
    model = SortedMap(keys, values)

    def check(queries):
        got_v, got_f = hm.get(queries[:, None])
        exp_v, exp_f = model.get(queries)
        assert torch.equal(got_f, exp_f)
        assert torch.equal(got_v[:, 0], exp_v)
        return int(exp_f.sum())

    mixed = torch.cat([keys[: n // 2], absent[: n // 2]])
    mixed = mixed[torch.randperm(n, generator=gen, device=cuda)]
    assert check(mixed) == n // 2
    del mixed

    # the batch of the configuration itself: 2^26 queries, half of them hits whose rank among the
    # stored keys is drawn Zipf(1.1), half uniform misses, shuffled; every row is compared
    from bench import make_queries
    zipf, n_hit = make_queries(keys, n, gen, cuda)
    assert abs(check(zipf) - n_hit) <= 64          # (a uniform "miss" can hit a stored key by chance)
    del zipf

    # bulk upsert into the populated table: a quarter overwritten, nothing new
    values[: n // 4] += 1.0
    hm.set(keys[: n // 4, None], values[: n // 4, None])
    assert hm.n_elements == n
    model = SortedMap(keys, values)
    assert check(keys) == n

    # read-out: exactly the stored pairs, each once
    ks, vs = hm.items()
    assert ks.shape[0] == n
    order = torch.argsort(ks[:, 0])
    assert torch.equal(ks[order, 0], model.keys) and torch.equal(vs[order, 0], model.values)
    del ks, vs, order

    # removal of a random half (the keys are in random order), then a per-row re-insert of a quarter
    gone = hm._remove_rows(keys[: n // 2, None].contiguous())
    assert bool(gone.all()) and hm.n_elements == n - n // 2
    model = SortedMap(keys[n // 2:], values[n // 2:])
    assert check(keys) == n - n // 2
    assert check(absent[: n // 4]) == 0
    back = keys[: n // 4]
    from doksparse_amd import closed_hashmap as ch
    old = ch.BULK_MIN_ROWS
    ch.BULK_MIN_ROWS = 1 << 62
    try:
        hm.set(back[:, None], values[: n // 4, None])
    finally:
        ch.BULK_MIN_ROWS = old
    assert hm.n_elements == n - n // 2 + n // 4
    model = SortedMap(torch.cat([keys[n // 2:], back]), torch.cat([values[n // 2:], values[: n // 4]]))
    assert check(keys) == n - n // 2 + n // 4


def test_table_beyond_four_gib(cuda, monkeypatch):
    """A table of 7 GiB: bucket byte offsets pass 2^32 (the reference's kernels index with 32-bit
    ints, closed_hashmap_impl.cu:72).  Per-row insert, bulk upsert on top, get, removal and
    read-out are checked through closed forms: key i is i times an odd constant (a bijection of
    the 64-bit integers, so the keys are distinct) and its value is i mod 2^24."""
    from doksparse_amd import CudaClosedHashmap
    from doksparse_amd import closed_hashmap as ch
    odd = -7046029254386353131                              # 0x9E3779B97F4A7C15 as int64
    def rows(lo, hi):
        i = torch.arange(lo, hi, device=cuda, dtype=torch.long)
        return (i * odd)[:, None], (i % (1 << 24)).float()[:, None]

    capacity = 560_000_000
    hm = CudaClosedHashmap(n_buckets=capacity, device=cuda, rehash_threshold=1.0)
    n1, n2, n_miss = 30_000_000, 150_000_000, 20_000_000
    monkeypatch.setattr(ch, "BULK_MIN_ROWS", 1 << 62)      # first batch: the per-row kernel
    k1, v1 = rows(0, n1)
    hm.set(k1, v1)
    assert hm._n_phys * 128 > 6 * 2**30
    assert hm.n_elements == n1
    got, found = hm.get(k1)
    assert bool(found.all()) and torch.equal(got, v1)
    del got, found

    # second batch through the bulk path: the last third of the first batch again (new values)
    # and n2 new keys
    monkeypatch.setattr(ch, "BULK_MIN_ROWS", 0)
    monkeypatch.setattr(ch, "BULK_MIN_ROWS_PER_BUCKET", 0.0)
    k2, v2 = rows(n1 - n1 // 3, n1 + n2)
    v2 += 1.0
    assert hm._bulk_workspace(k2.shape[0]) is not None
    hm.set(k2, v2)
    total = n1 + n2
    assert hm.n_elements == total
    got, found = hm.get(k2)
    assert bool(found.all()) and torch.equal(got, v2)
    del got, found
    head = n1 - n1 // 3
    got, found = hm.get(k1[:head])
    assert bool(found.all()) and torch.equal(got, v1[:head])
    km, _ = rows(total, total + n_miss)
    got, found = hm.get(km)
    assert not bool(found.any()) and not bool(got.any())
    del got, found, km

    # read-out: every key once (the wrapped sum of the keys is a checksum of the set)
    ks = hm.keys()
    assert ks.shape[0] == total
    i_sum = total * (total - 1) // 2
    expect = (i_sum * odd) % (1 << 64)
    assert int(ks.sum()) % (1 << 64) == expect
    del ks

    # removal of the first batch's head, then those keys are gone and the rest is there
    gone = hm._remove_rows(k1[:head].contiguous())
    assert bool(gone.all()) and hm.n_elements == total - head
    assert not bool(hm.get(k1[:head])[1].any())
    assert bool(hm.get(k2[-n_miss:])[1].all())


def test_bulk_path_with_the_wide_second_level(cuda, monkeypatch):
    """Between 2^26 and 2^28 buckets the bulk path partitions 1024 ranges per first-level bin
    instead of 256.  A table of 100M buckets (12.8 GB): bulk build of 200M rows into uninitialised
    memory, bulk upsert of 50M stored + 50M new keys, then get / read-out checksum / count."""
    from doksparse_amd import CudaClosedHashmap
    from doksparse_amd import closed_hashmap as ch
    monkeypatch.setattr(ch, "BULK_MIN_ROWS", 0)
    monkeypatch.setattr(ch, "BULK_MIN_ROWS_PER_BUCKET", 0.0)
    odd = -7046029254386353131
    def rows(lo, hi, bump):
        i = torch.arange(lo, hi, device=cuda, dtype=torch.long)
        return (i * odd)[:, None], ((i % (1 << 24)).float() + bump)[:, None]

    hm = CudaClosedHashmap(n_buckets=1_000_000_000, device=cuda, rehash_threshold=1.0)
    n1 = 200_000_000
    k1, v1 = rows(0, n1, 0.0)
    hm.set(k1, v1)                                          # build
    assert 2**26 < hm._n_phys <= 2**28 and hm._bulk_workspace(n1) is not None
    assert hm.n_elements == n1
    got, found = hm.get(k1)
    assert bool(found.all()) and torch.equal(got, v1)
    del got, found
    k2, v2 = rows(n1 - 50_000_000, n1 + 50_000_000, 1.0)
    hm.set(k2, v2)                                          # upsert into the populated table
    total = n1 + 50_000_000
    assert hm.n_elements == total
    got, found = hm.get(k2)
    assert bool(found.all()) and torch.equal(got, v2)
    got, found = hm.get(k1[: n1 - 50_000_000])
    assert bool(found.all()) and torch.equal(got, v1[: n1 - 50_000_000])
    del got, found
    assert not bool(hm.get(rows(total, total + 10_000_000, 0.0)[0])[1].any())
    ks = hm.keys()
    assert ks.shape[0] == total
    assert int(ks.sum()) % (1 << 64) == (total * (total - 1) // 2 * odd) % (1 << 64)


def test_table_of_several_bulk_windows(cuda, monkeypatch):
    """More than 2^28 buckets (a table of 36 GB): the two partition levels address 1024 x 1024
    ranges, so the bulk path works through such a table in windows of 2^28 buckets, one run of its
    passes per window.  Bulk build of 700M rows, bulk upsert of 50M stored + 50M new keys, bulk
    removal of 100M (half of them absent), then get / count / read-out checksum; bulk rehash of a
    smaller table into one of two windows."""
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd import closed_hashmap as ch
    monkeypatch.setattr(ch, "BULK_MIN_ROWS", 0)
    monkeypatch.setattr(ch, "BULK_MIN_ROWS_PER_BUCKET", 0.0)
    monkeypatch.setattr(ch, "BULK_REMOVE_MIN_ROWS_PER_BUCKET", 0.0)
    odd = -7046029254386353131
    # the two keys whose stored word would read EMPTY / TOMBSTONE - 0x9E3779B97F4A7C15 (which is `odd`
    # as an int64) and the same ^ 1 - live in side slots of the header: they take the places of keys
    # 0 and 1 of the first batch (with several windows only the first one may handle them)
    specials = [odd, odd ^ 1]
    def rows(lo, hi, bump):
        i = torch.arange(lo, hi, device=cuda, dtype=torch.long)
        k = i * odd
        if lo == 0:
            k[0], k[1] = specials[0], specials[1]
        return k[:, None], ((i % (1 << 24)).float() + bump)[:, None]
    key_sum = lambda total: (total * (total - 1) // 2 * odd - odd + specials[0] + specials[1]) % (1 << 64)

    hm = CudaClosedHashmap(n_buckets=2_800_000_000, device=cuda, rehash_threshold=1.0)
    n1 = 700_000_000
    k1, v1 = rows(0, n1, 0.0)
    hm.set(k1, v1)                                          # build
    assert hm._n_phys > 2**28 and hm._bulk_workspace(n1) is not None
    assert hm.n_elements == n1
    got, found = hm.get(k1)
    assert bool(found.all()) and torch.equal(got, v1)
    del got, found
    k2, v2 = rows(n1 - 50_000_000, n1 + 50_000_000, 1.0)
    hm.set(k2, v2)                                          # upsert into the populated table
    total = n1 + 50_000_000
    assert hm.n_elements == total
    got, found = hm.get(k2)
    assert bool(found.all()) and torch.equal(got, v2)
    got, found = hm.get(k1[: n1 - 50_000_000])
    assert bool(found.all()) and torch.equal(got, v1[: n1 - 50_000_000])
    del got, found, k2, v2
    assert not bool(hm.get(rows(total, total + 10_000_000, 0.0)[0])[1].any())
    k3 = rows(total - 50_000_000, total + 50_000_000, 0.0)[0]
    del hm[k3]                                              # bulk removal: 50M stored, 50M absent
    total -= 50_000_000
    assert hm.n_elements == total
    assert not bool(hm.get(k3)[1].any())
    del k3
    got, found = hm.get(k1[: n1 - 50_000_000])
    assert bool(found.all()) and torch.equal(got, v1[: n1 - 50_000_000])
    del got, found
    ks = hm.keys()
    assert ks.shape[0] == total
    assert int(ks.sum()) % (1 << 64) == key_sum(total)
    del ks, hm

    # bulk rehash from a table of one window (the source's words are the rows: 2^27 buckets at
    # most) into one of two
    hm = CudaClosedHashmap(n_buckets=1_300_000_000, device=cuda, rehash_threshold=1.0)
    hm.set(k1, v1)
    assert hm._n_phys <= 2**27
    lib = _lib.load()
    calls = []
    real = lib.dok_map_rehash_bulk
    monkeypatch.setattr(lib, "dok_map_rehash_bulk", lambda *a: (calls.append(1), real(*a))[1])
    hm.rehash(2_700_000_000)                                # (2.5 entries per bucket and more: the bulk rehash)
    assert calls and hm._n_phys > 2**28 and hm.n_elements == n1
    got, found = hm.get(k1)
    assert bool(found.all()) and torch.equal(got, v1)
    del got, found
    ks = hm.keys()
    assert ks.shape[0] == n1
    assert int(ks.sum()) % (1 << 64) == key_sum(n1)


def test_coordinate_row_tensor_10m_entries(cuda):
    """A (2^40, 2^40) tensor - its coordinates cannot be linearised into one 8-byte key and are
    stored as two-word keys - with 10M entries: construct, gather of 4M elements (half stored, half
    absent), scatter of 4M (half present, half new, with a growth of the table), sparse-valued
    gather, read-out.  The independent map is a sorted array: the coordinates are drawn as
    c = (r << 20) | f(r) with r < 2^20, so that a pair of them has a 40-bit name (r0, r1) of its
    own that the table never sees."""
    from doksparse_amd import SparseDOKTensor, _lib
    gen = torch.Generator(device=cuda).manual_seed(4040)
    size = (2**40, 2**40)

    def spread(r):
        return (r << 20) | ((r * 0x9E3779B1) & 0xFFFFF)

    def names(n):
        lin = torch.unique(torch.randint(0, 2**40, (n,), generator=gen, device=cuda))
        return lin[torch.randperm(lin.numel(), generator=gen, device=cuda)]

    lin = names(10_000_000)
    nnz = lin.numel()
    coords = torch.stack([spread(lin >> 20), spread(lin & 0xFFFFF)])
    assert int(coords.max()) >= 2**39
    vals = torch.randn(nnz, generator=gen, device=cuda)
    dok = SparseDOKTensor(size, coords, vals, device=cuda)
    hm = dok.storage()
    assert hm._coord_rows and hm._layout == _lib.DOK_LAYOUT_TAGGED and hm._desc.key_bytes == 16
    assert dok._nnz() == nnz
    smap = SortedMap(lin, vals)

    # gather: 2M stored coordinates, 1M absent pairs of the same form, 1M arbitrary coordinates
    pick = torch.randint(0, nnz, (2_000_000,), generator=gen, device=cuda)
    other = torch.randint(0, 2**40, (1_000_000,), generator=gen, device=cuda)
    qlin = torch.cat([lin[pick], other])
    q = torch.stack([spread(qlin >> 20), spread(qlin & 0xFFFFF)])
    q = torch.cat([q, torch.randint(0, 2**40, (2, 1_000_000), generator=gen, device=cuda)], dim=1)
    exp = torch.cat([smap.get(qlin)[0], torch.zeros(1_000_000, device=cuda)])
    order = torch.randperm(q.shape[1], generator=gen, device=cuda)
    q, exp = q[:, order].contiguous(), exp[order]
    got = dok[q[0], q[1]]
    assert torch.equal(got, exp) and int((exp != 0).sum()) >= 2_000_000
    # the same as a 2-D expression: 2048 stored rows x 2048 columns (mostly absent cells)
    rr, cc = coords[0, :2048], coords[1, 5000:7048]
    got2 = dok[rr[:, None], cc[None, :]]
    lin2 = ((rr >> 20)[:, None] << 20) + (cc >> 20)[None, :]
    assert torch.equal(got2.reshape(-1), smap.get(lin2.reshape(-1))[0])

    # scatter: 2M stored + 2M fresh coordinates; the table has to grow
    flin = names(2_200_000)
    flin = flin[~smap.get(flin)[1]][:2_000_000]
    wl = torch.cat([lin[:2_000_000], flin])
    wl = wl[torch.randperm(wl.numel(), generator=gen, device=cuda)]
    wc = torch.stack([spread(wl >> 20), spread(wl & 0xFFFFF)])
    wv = torch.randn(wl.numel(), generator=gen, device=cuda)
    n_before = hm.n_buckets
    dok[wc[0], wc[1]] = wv
    assert dok._nnz() == nnz + flin.numel()
    assert hm.n_buckets == int(np.ceil((nnz + wl.numel()) * 2.0)) > n_before      # grown as the reference would
    keep = ~SortedMap(wl, wv).get(lin)[1]
    smap2 = SortedMap(torch.cat([lin[keep], wl]), torch.cat([vals[keep], wv]))
    assert torch.equal(dok[q[0], q[1]][order.argsort()][:3_000_000], smap2.get(qlin)[0])

    # read-out: exactly the entries, each once
    idx, v = dok.indices(), dok.values()
    assert idx.shape == (2, nnz + flin.numel())
    assert torch.equal(spread(idx[0] >> 20), idx[0]) and torch.equal(spread(idx[1] >> 20), idx[1])
    rl = ((idx[0] >> 20) << 20) + (idx[1] >> 20)
    so = torch.argsort(rl)
    assert torch.equal(rl[so], smap2.keys) and torch.equal(v[so], smap2.values)

    # count / remove of the first gather's elements
    n_stored = int(smap2.get(qlin)[1].sum())
    assert int(dok.count_items((q[0], q[1])).item()) == n_stored
    dok.zero_items((q[0], q[1]))
    assert dok._nnz() == nnz + flin.numel() - int(smap2.get(torch.unique(qlin))[1].sum())
    assert int(dok.count_items((q[0], q[1])).item()) == 0
