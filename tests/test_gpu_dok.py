"""GPU parity: SparseDOKTensor indexing through the fused HIP kernels against the CPU oracle
(oracle/ref_dok.py) and dense torch tensors on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle.ref_dok import RefSparseDOKTensor

pytestmark = pytest.mark.gpu


def make(shape, nnz, seed, dev, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    flat = torch.randperm(int(np.prod(shape)), generator=g)[:nnz]
    idx = torch.stack(torch.unravel_index(flat, shape))
    vals = (torch.randn(nnz, generator=g) * 10).to(dtype)
    vals[vals == 0] = 1
    from doksparse_amd import SparseDOKTensor
    dok = SparseDOKTensor(shape, idx.to(dev), vals.to(dev), device=dev)
    ref = RefSparseDOKTensor(shape, idx, vals, rng=np.random.default_rng(seed))
    return dok, ref


def sorted_coo(indices, values):
    indices, values = indices.cpu().numpy(), values.cpu().numpy()
    order = np.lexsort(indices[::-1])
    return indices[:, order], values[order]


def same_entries(dok, ref):
    a = sorted_coo(dok.indices(), dok.values())
    b = sorted_coo(ref.indices(), ref.values())
    return np.array_equal(a[0], b[0]) and np.array_equal(a[1].view(np.uint8), b[1].view(np.uint8))


def test_construct_readout_to_dense(cuda):
    for dtype in (torch.float32, torch.float16, torch.float64, torch.int64):
        dok, ref = make((13, 17), 60, 1, cuda, dtype)
        assert dok._nnz() == ref._nnz() == 60
        assert dok.storage().n_buckets == ref._hashmap.n_buckets == 120
        assert same_entries(dok, ref)
        assert torch.equal(dok.to_dense().cpu(), ref.to_dense())
        assert torch.equal(dok.to_sparse_coo().to_dense().cpu(), ref.to_dense())
        assert dok.indices().shape == (2, 60) and dok.values().shape == (60,)


@pytest.mark.parametrize("size", [
    (7, 1, 1000003, 3, 1),                    # dimensions of 1 (strides that repeat), a prime
    (2147483647, 2147483629),                 # two primes below 2^31: keys up to 2^62
    (3, 5, 7, 11, 13, 17, 19, 23),            # eight dimensions, no stride a power of two
    (4096, 4096, 64, 8),                      # every stride a power of two
    (1, 1, 1),                                # a single cell
    (1000000, 1000000),
    (9223372036854775807,),                   # one dimension of 2^63 - 1
])
def test_readout_recovers_coordinates_for_awkward_shapes(cuda, size):
    """indices() turns the stored linear keys back into coordinates by multiply-and-shift
    division by the row-major strides: it must return exactly the coordinates that went in,
    the largest coordinate of every dimension included."""
    from doksparse_amd import SparseDOKTensor
    g = torch.Generator().manual_seed(len(size))
    n = 1 if all(s == 1 for s in size) else 4000
    coords = torch.stack([torch.randint(0, s, (n,), generator=g) if s > 1 else torch.zeros(n, dtype=torch.long)
                          for s in size])
    coords[:, 0] = torch.tensor([s - 1 for s in size])              # the far corner
    if n > 1:
        coords[:, 1] = 0                                             # and the origin
    coords = torch.unique(coords, dim=1)
    vals = torch.arange(1, coords.shape[1] + 1, dtype=torch.float32)
    dok = SparseDOKTensor(size, coords.to(cuda), vals.to(cuda), device=cuda)
    idx, v = dok.indices().cpu(), dok.values().cpu()
    assert idx.shape == coords.shape
    order = torch.argsort(v)                                         # the values number the input columns
    assert torch.equal(v[order], vals)
    assert torch.equal(idx[:, order], coords)


GET_CASES = [
    lambda r, c, m: (r, c),
    lambda r, c, m: (r[:, None], c[None, :]),
    lambda r, c, m: (r,),
    lambda r, c, m: (slice(None), c),
    lambda r, c, m: (slice(2, 9), slice(None, 5)),
    lambda r, c, m: (slice(None), slice(None)),
    lambda r, c, m: (r.tolist(), slice(1, 4)),
    lambda r, c, m: (r.to(torch.int32), c.to(torch.int16)),
    lambda r, c, m: (slice(5, 3), c),
    lambda r, c, m: (3, c),
    lambda r, c, m: (3, slice(None)),
    lambda r, c, m: (slice(None), m),
]


@pytest.mark.parametrize("case", range(len(GET_CASES)))
def test_getitem_2d(cuda, case):
    dok, ref = make((13, 17), 120, 2, cuda)
    g = torch.Generator().manual_seed(case)
    r = torch.randint(0, 13, (6,), generator=g)
    c = torch.randint(0, 17, (6,), generator=g)
    m = torch.rand(17, generator=g) < 0.5
    sel = GET_CASES[case](r, c, m)
    dsel = tuple(s.to(cuda) if isinstance(s, torch.Tensor) else s for s in sel)
    got, exp = dok[dsel], ref[sel]
    assert got.shape == exp.shape and got.dtype == exp.dtype
    assert torch.equal(got.cpu(), exp)


def test_getitem_4d_axis_rule_masks_scalars(cuda):
    dok, ref = make((6, 7, 5, 4), 700, 3, cuda)
    i, k = torch.tensor([0, 5, 2]), torch.tensor([3, 0, 1])
    mask = torch.tensor([True, False, True, True])
    m2 = torch.rand(6, 7, generator=torch.Generator().manual_seed(1)) < 0.3
    cases = [(slice(None), i, slice(None), k), (i, slice(None), k), (4, slice(0, 3), i[:2] % 5, k[:2]),
             (2, slice(0, 5), i[:, None], mask), (slice(None), slice(None), slice(None), mask),
             (m2,), (m2, slice(1, 3)), (3,), (3, 2), (0, slice(3, 4), slice(None))]
    for sel in cases:
        dsel = tuple(s.to(cuda) if isinstance(s, torch.Tensor) else s for s in sel)
        got, exp = dok[dsel], ref[sel]
        assert got.shape == exp.shape, sel
        assert torch.equal(got.cpu(), exp), sel
    # the reference raises IndexError here by accident (it squeezes an axis that does not
    # exist); the build returns what the expression means
    with pytest.raises(IndexError):
        ref[:, 2, 3]
    got = dok[:, 2, 3]
    dense = ref.to_dense()
    assert torch.equal(got.cpu(), dense[:, 2, 3])
    with pytest.raises(IndexError):
        ref[1, 2, 3, 0]                       # all-scalar indexing: same accident
    assert dok[1, 2, 3, 0].shape == () and dok[1, 2, 3, 0].item() == dense[1, 2, 3, 0].item()


def test_getitem_out_of_range_coordinates_read_zero(cuda):
    dok, ref = make((13, 17), 100, 4, cuda)
    r = torch.tensor([0, 12, 13, -1, 5, 2**40])
    c = torch.tensor([0, 16, 0, 3, 17, 1])
    got, exp = dok[r.to(cuda), c.to(cuda)], ref[r, c]
    assert torch.equal(got.cpu(), exp)
    assert got[2:].abs().sum().item() == 0


def test_setitem_parity(cuda):
    dok, ref = make((13, 17), 40, 6, cuda)
    g = torch.Generator().manual_seed(0)
    flat = torch.randperm(13 * 17, generator=g)[:50]
    r, c = flat // 17, flat % 17
    v = torch.randn(50, generator=g)
    dok[r.to(cuda), c.to(cuda)] = v.to(cuda)
    ref[r, c] = v
    assert dok._nnz() == ref._nnz()
    assert dok.storage().n_buckets == ref._hashmap.n_buckets
    assert same_entries(dok, ref)
    rows, cols = torch.tensor([1, 4, 7]), torch.tensor([0, 16])
    dok[rows[:, None].to(cuda), cols[None, :].to(cuda)] = torch.tensor([5.0, 6.0], device=cuda)
    ref[rows[:, None], cols[None, :]] = torch.tensor([5.0, 6.0])
    dok[2:4, 5:9] = 3.5
    ref[2:4, 5:9] = 3.5
    dok[:, 3] = torch.arange(13.0, device=cuda)
    ref[:, 3] = torch.arange(13.0)
    assert dok._nnz() == ref._nnz() and dok.storage().n_buckets == ref._hashmap.n_buckets
    assert same_entries(dok, ref)
    assert torch.equal(dok.to_dense().cpu(), ref.to_dense())
    # a strided (transposed) source view is read through its strides
    src = torch.randn(9, 13, generator=g)
    dok[:, 4:13] = src.T.to(cuda)
    ref[:, 4:13] = src.T
    assert torch.equal(dok.to_dense().cpu(), ref.to_dense())
    assert dok._nnz() == ref._nnz()


def test_setitem_from_empty_stores_zeros_and_grows_like_the_reference(cuda):
    from doksparse_amd import SparseDOKTensor
    dok = SparseDOKTensor((100, 100), device=cuda, dtype=torch.float)
    ref = RefSparseDOKTensor((100, 100))
    idx = torch.arange(100)
    dok[idx.to(cuda), idx.to(cuda)] = torch.zeros(100, device=cuda)
    ref[idx, idx] = torch.zeros(100)
    assert dok._nnz() == ref._nnz() == 100
    assert dok.storage().n_buckets == ref._hashmap.n_buckets == 202
    dok[idx.to(cuda), idx.to(cuda)] = 1
    assert torch.equal(dok.to_dense(), torch.eye(100, device=cuda))
    assert dok._nnz() == 100


def test_setitem_with_repeated_coordinates(cuda):
    """Equal coordinates inside one assignment: one entry, holding one of the assigned values
    (the reference over-counts its element counter here; the build counts entries)."""
    from doksparse_amd import SparseDOKTensor
    dok = SparseDOKTensor((50, 60), device=cuda)
    g = torch.Generator().manual_seed(2)
    r = torch.randint(0, 50, (5000,), generator=g)
    c = torch.randint(0, 60, (5000,), generator=g)
    v = torch.arange(1.0, 5001.0)
    dok[r.to(cuda), c.to(cuda)] = v.to(cuda)
    lin = (r * 60 + c)
    assert dok._nnz() == lin.unique().numel()
    dense = dok.to_dense().cpu().flatten()
    allowed = {}
    for p, x in zip(lin.tolist(), v.tolist()):
        allowed.setdefault(p, set()).add(x)
    for p in range(3000):
        assert (dense[p].item() in allowed[p]) if p in allowed else dense[p].item() == 0
    with pytest.raises(IndexError):
        dok[torch.tensor([1, 50], device=cuda), torch.tensor([1, 1], device=cuda)] = 1.0


def test_count_and_zero_items(cuda):
    dok, ref = make((13, 17), 100, 8, cuda)
    dense = ref.to_dense()
    r = torch.arange(13)[:, None]
    c = torch.arange(0, 17, 2)[None, :]
    assert dok.count_items((r.to(cuda), c.to(cuda))).item() == int((dense[r, c] != 0).sum())
    dok.zero_items((r.to(cuda), c.to(cuda)))
    dense[r, c] = 0
    assert torch.equal(dok.to_dense().cpu(), dense)
    assert dok._nnz() == int((dense != 0).sum())


def test_cfg4_shape_scaled(cuda):
    """2-D 1e6 x 1e6 float32 tensor at 1/1024 of the entry count: advanced-index gather of
    rows x cols (uniform and planted on stored coordinates) and a scatter of mixed overwrites
    and inserts."""
    from doksparse_amd import SparseDOKTensor
    g = torch.Generator().manual_seed(1004)
    nnz = 50_000_000 // 1024
    size = (1_000_000, 1_000_000)
    idx = torch.randint(0, 1_000_000, (2, nnz), generator=g)
    lin = idx[0] * 1_000_000 + idx[1]
    keep = torch.from_numpy(np.unique(lin.numpy(), return_index=True)[1])
    idx = idx[:, keep]
    vals = torch.randn(idx.shape[1], generator=g)
    dok = SparseDOKTensor(size, idx.to(cuda), vals.to(cuda), device=cuda)
    ref = RefSparseDOKTensor(size, idx, vals, rng=np.random.default_rng(4))
    assert dok._nnz() == ref._nnz() == idx.shape[1]
    assert dok.storage().n_buckets == ref._hashmap.n_buckets
    rows = torch.randint(0, 1_000_000, (128,), generator=g)
    cols = torch.randint(0, 1_000_000, (256,), generator=g)
    prow, pcol = idx[0, :128], idx[1, 100:356]              # planted: rows/cols that hold entries
    for rr, cc in ((rows, cols), (prow, pcol)):
        got = dok[rr[:, None].to(cuda), cc[None, :].to(cuda)]
        exp = ref[rr[:, None], cc[None, :]]
        assert got.shape == (128, 256) and torch.equal(got.cpu(), exp)
    assert int((dok[prow[:, None].to(cuda), pcol[None, :].to(cuda)] != 0).sum()) >= 28
    # scatter: half overwrites, half new coordinates
    n_set = 10_000_000 // 1024
    new = torch.randint(0, 1_000_000, (2, n_set // 2), generator=g)
    coords = torch.cat([idx[:, : n_set // 2], new], dim=1)
    lin = coords[0] * 1_000_000 + coords[1]
    coords = coords[:, torch.from_numpy(np.unique(lin.numpy(), return_index=True)[1])]
    x = torch.randn(coords.shape[1], generator=g)
    dok[coords[0].to(cuda), coords[1].to(cuda)] = x.to(cuda)
    ref[coords[0], coords[1]] = x
    assert dok._nnz() == ref._nnz()
    assert dok.storage().n_buckets == ref._hashmap.n_buckets
    assert same_entries(dok, ref)


def test_cfg5_shape_scaled_with_tombstone_churn(cuda):
    """4-D (4096, 4096, 64, 8) float16 tensor at 1/1024 of the entry count and load factor 0.85:
    mixed indexing dok[i, :512, idx, mask], then remove 20 % / insert as many fresh / repeat."""
    from doksparse_amd import SparseDOKTensor, CudaClosedHashmap
    g = torch.Generator().manual_seed(1005)
    size = (4096, 4096, 64, 8)
    nnz = 100_000_000 // 1024
    i_list = torch.randint(0, 4096, (8,), generator=g)

    def draw(n):
        # half of the entries are planted inside the region the gets address
        a = torch.stack([torch.randint(0, s, (n // 2,), generator=g) for s in size])
        b = torch.stack([i_list[torch.randint(0, 8, (n - n // 2,), generator=g)],
                         torch.randint(0, 512, (n - n // 2,), generator=g),
                         torch.randint(0, 64, (n - n // 2,), generator=g),
                         torch.randint(0, 8, (n - n // 2,), generator=g)])
        return torch.cat([a, b], dim=1)

    def dedupe(idx):
        lin = ((idx[0] * 4096 + idx[1]) * 64 + idx[2]) * 8 + idx[3]
        return idx[:, torch.from_numpy(np.unique(lin.numpy(), return_index=True)[1])]

    idx = dedupe(draw(nnz))
    vals = torch.randn(idx.shape[1], generator=g).half()
    cap = int(np.ceil(idx.shape[1] / 0.85))
    store = CudaClosedHashmap(n_buckets=cap, device=cuda, rehash_threshold=0.9, coord_dims=size)
    dok = SparseDOKTensor(size, idx.to(cuda), vals.to(cuda), device=cuda, storage=store)
    ref = RefSparseDOKTensor(size, dtype=torch.float16, rng=np.random.default_rng(5))
    ref._hashmap.__init__(n_buckets=cap, rehash_threshold=0.9, rng=np.random.default_rng(5))
    ref._hashmap.set(idx.T.contiguous().numpy(), vals[:, None].numpy())
    assert dok._nnz() == ref._nnz() == idx.shape[1] and dok.storage().n_buckets == cap

    sel_idx = torch.randint(0, 64, (128,), generator=g)
    mask = torch.tensor([True, False, True, True, False, False, True, False])

    def run_gets():
        hits = 0
        for i in i_list.tolist():
            got = dok[i, :512, sel_idx[:, None].to(cuda), mask.to(cuda)]
            exp = ref[i, :512, sel_idx[:, None], mask]
            assert got.shape == exp.shape == (128, 4, 512) and got.dtype == torch.float16
            assert torch.equal(got.cpu(), exp)
            hits += int((exp != 0).sum())
        return hits

    assert run_gets() > 1000
    # churn
    n_gone = idx.shape[1] // 5
    perm = torch.randperm(idx.shape[1], generator=g)
    gone = idx[:, perm[:n_gone]]
    m = dok.storage().remove(gone.T.contiguous().to(cuda))
    rm = ref._hashmap.remove(gone.T.contiguous().numpy())
    assert np.array_equal(m.cpu().numpy(), rm) and bool(m.all())
    fresh = dedupe(draw(n_gone))
    fv = torch.randn(fresh.shape[1], generator=g).half()
    dok.storage().set(fresh.T.contiguous().to(cuda), fv[:, None].to(cuda))
    ref._hashmap.set(fresh.T.contiguous().numpy(), fv[:, None].numpy())
    assert dok._nnz() == ref._nnz() and dok.storage().n_buckets == ref._hashmap.n_buckets
    assert run_gets() > 1000
    assert same_entries(dok, ref)


def test_sparse_valued_getitem(cuda):
    dok, ref = make((9, 11, 6), 250, 9, cuda)
    sels = [(slice(2, 7), torch.tensor([1, 3, 5, 10]), slice(None)),
            (torch.tensor([0, 8, 3])[:, None], torch.tensor([2, 2, 9])[None, :], 4),
            (slice(None), slice(None), slice(None)),
            (torch.tensor([1, 1, 2]), slice(0, 0), slice(None))]
    for sel in sels:
        dsel = tuple(s.to(cuda) if isinstance(s, torch.Tensor) else s for s in sel)
        got, exp = dok.__spgetitem__(dsel), ref.__spgetitem__(sel)
        assert tuple(got.shape) == tuple(exp.shape)
        assert got._nnz() == exp._nnz()
        assert got.storage().n_buckets == exp._hashmap.n_buckets
        assert same_entries(got, exp)
        assert torch.equal(got.to_dense().cpu(), exp.to_dense())
    # explicit zeros are entries: they survive the sparse gather
    dok[0, 0, 0] = 0.0
    ref[0, 0, 0] = 0.0
    got, exp = dok.__spgetitem__((slice(0, 2),)), ref.__spgetitem__((slice(0, 2),))
    assert got._nnz() == exp._nnz() and same_entries(got, exp)


def test_sparse_valued_setitem(cuda):
    from doksparse_amd import SparseDOKTensor
    dok, ref = make((9, 11), 40, 10, cuda)
    src = torch.zeros(5, 4)
    src[0, 1], src[3, 2], src[4, 0], src[2, 2] = 7.0, -2.0, 5.0, 1.5
    cols = torch.tensor([1, 3, 5, 10])
    dok[2:7, cols.to(cuda)] = src.to_sparse().to(cuda)
    ref[2:7, cols] = src.to_sparse()
    assert dok.storage().n_buckets == ref._hashmap.n_buckets
    assert same_entries(dok, ref)
    dense = ref.to_dense()
    assert torch.equal(dok.to_dense().cpu(), dense)
    assert dok._nnz() == int((dense != 0).sum())
    # a DOK tensor as the source, into an empty destination
    sdok = SparseDOKTensor.from_dense(src.to(cuda))
    rsrc = RefSparseDOKTensor((5, 4), src.nonzero().T, src[tuple(src.nonzero().T)])
    d2 = SparseDOKTensor((20, 20), device=cuda)
    r2 = RefSparseDOKTensor((20, 20))
    rows = torch.tensor([3, 19, 0, 7, 8])
    d2[rows.to(cuda), 4:8] = sdok
    r2[rows, 4:8] = rsrc
    assert torch.equal(d2.to_dense().cpu(), r2.to_dense())
    assert d2.storage().n_buckets == r2._hashmap.n_buckets
    # minus zero in a floating source counts as zero
    s3 = torch.sparse_coo_tensor(torch.tensor([[0, 1], [0, 1]]), torch.tensor([-0.0, 4.0]), (5, 4))
    d2[rows.to(cuda), 4:8] = s3.to(cuda)
    r2[rows, 4:8] = s3
    assert torch.equal(d2.to_dense().cpu(), r2.to_dense())
    assert same_entries(d2, r2)


def test_views_share_storage(cuda):
    """permute / transpose / T give views over the same table: reads follow the permuted
    dimensions, writes through a view land in the base tensor and vice versa."""
    dok, ref = make((6, 7, 5), 120, 11, cuda)
    dense = ref.to_dense()
    v = dok.permute(2, 0, 1)
    assert tuple(v.shape) == (5, 6, 7) and v._nnz() == dok._nnz()
    assert torch.equal(v.to_dense().cpu(), dense.permute(2, 0, 1))
    i, j = torch.tensor([0, 4, 2]), torch.tensor([5, 1, 3])
    assert torch.equal(v[i.to(cuda), j.to(cuda)].cpu(), dense.permute(2, 0, 1)[i, j])
    assert torch.equal(v[1:4, :, 2].cpu(), dense.permute(2, 0, 1)[1:4, :, 2])
    order = np.lexsort(v.indices().cpu().numpy()[::-1])
    assert torch.equal(v.indices().cpu()[:, order], dense.permute(2, 0, 1).nonzero().T)
    # write through the view, read through the base
    v[4, 5, 6] = 42.0
    dense[5, 6, 4] = 42.0
    assert dok[5, 6, 4].item() == 42.0 and torch.equal(dok.to_dense().cpu(), dense)
    # write through the base (enough to force a rehash), read through the view
    g = torch.Generator().manual_seed(3)
    flat = torch.randperm(6 * 7 * 5, generator=g)[:150]
    a, b, c = flat // 35, (flat // 5) % 7, flat % 5
    x = torch.randn(150, generator=g)
    dok[a.to(cuda), b.to(cuda), c.to(cuda)] = x.to(cuda)
    dense[a, b, c] = x
    assert torch.equal(v.to_dense().cpu(), dense.permute(2, 0, 1))
    assert v._nnz() == dok._nnz() == int((dense != 0).sum())
    # transpose of a view composes; T on 2-D
    w = v.transpose(0, 2)
    assert tuple(w.shape) == (7, 6, 5) and torch.equal(w.to_dense().cpu(), dense.permute(1, 0, 2))
    d2, r2 = make((8, 9), 30, 12, cuda)
    t = d2.T
    assert torch.equal(t.to_dense().cpu(), r2.to_dense().T)
    t[torch.arange(9, device=cuda), torch.arange(9, device=cuda) % 8] = 1.0
    dd = r2.to_dense()
    dd[torch.arange(9) % 8, torch.arange(9)] = 1.0
    assert torch.equal(d2.to_dense().cpu(), dd)
    # in-place permutation moves nothing
    table_ptr = d2.storage()._table.data_ptr()
    d2.permute_(1, 0)
    assert tuple(d2.shape) == (9, 8) and d2.storage()._table.data_ptr() == table_ptr
    assert torch.equal(d2.to_dense().cpu(), dd.T)
    # flatten / reshape / unary ops go through the view order
    assert torch.equal(v.flatten().to_dense().cpu(), dense.permute(2, 0, 1).reshape(-1))
    assert torch.equal(v.reshape(30, 7).to_dense().cpu(), dense.permute(2, 0, 1).reshape(30, 7))
    assert torch.equal(v.abs().to_dense().cpu(), dense.permute(2, 0, 1).abs())


def test_repeated_mask_selectors_follow_in_place_changes(cuda):
    """The index tensors of a boolean mask are kept between calls; an in-place write to the mask
    and a different mask object must both be seen."""
    from doksparse_amd import SparseDOKTensor
    g = torch.Generator().manual_seed(8)
    dense = torch.zeros(40, 16)
    flat = torch.randperm(40 * 16, generator=g)[:200]
    dense.view(-1)[flat] = torch.randn(200, generator=g)
    dok = SparseDOKTensor.from_dense(dense.to(cuda))
    mask = torch.zeros(16, dtype=torch.bool, device=cuda)
    mask[[1, 4, 9]] = True
    rows = torch.arange(0, 40, 3, device=cuda)
    for _ in range(3):
        assert torch.equal(dok[rows[:, None], mask].cpu(), dense[rows.cpu()[:, None], mask.cpu()])
    mask[4] = False                                   # in-place change: the version counter moves
    mask[12] = True
    assert torch.equal(dok[rows[:, None], mask].cpu(), dense[rows.cpu()[:, None], mask.cpu()])
    for k in range(12):                                # fresh mask objects, more than the cache holds
        m2 = torch.zeros(16, dtype=torch.bool, device=cuda)
        m2[[k, (k + 5) % 16]] = True
        assert torch.equal(dok[rows[:, None], m2].cpu(), dense[rows.cpu()[:, None], m2.cpu()])
        del m2


def test_reductions_and_elementwise_glue(cuda):
    """The methods that stay torch glue over the read-out (reference: sparse_dok_tensor.py:352-561):
    sum, norm, normalize, softmax, log_softmax, index_select, select and the element-wise maps,
    against the same operations on the dense tensor (softmax and normalize run over the stored
    entries only, as torch.sparse does)."""
    from doksparse_amd import SparseDOKTensor
    gen = torch.Generator(device="cpu"); gen.manual_seed(9)
    dense = torch.zeros(40, 30)
    mask = torch.rand(40, 30, generator=gen) < 0.3
    dense[mask] = torch.randn(int(mask.sum()), generator=gen) * 3
    dok = SparseDOKTensor.from_dense(dense.to(cuda))
    assert torch.allclose(dok.sum().cpu(), dense.sum(), atol=1e-4)
    assert torch.allclose(dok.sum(dim=1).to_dense().cpu(), dense.sum(dim=1), atol=1e-4)
    for p in (1, 2, 3):
        assert torch.allclose(dok.norm(dim=1, p=p).cpu(), dense.norm(dim=1, p=p), atol=1e-4)
        n = dok.normalize(dim=1, p=p).to_dense().cpu()
        expect = dense.abs() / dense.norm(dim=1, p=p, keepdim=True).clamp_min(1e-30)
        assert torch.allclose(n, expect, atol=1e-5)
        assert torch.allclose(dok.normalize_(dim=1, p=p).to_dense().cpu(), expect, atol=1e-5)
    assert torch.equal(dok.to_dense().cpu(), dense)                       # normalize_ leaves the tensor alone
    sm = dok.softmax(dim=1).to_dense().cpu()
    e = torch.where(mask, dense.exp(), torch.zeros(()))
    assert torch.allclose(sm, e / e.sum(dim=1, keepdim=True).clamp_min(1e-30), atol=1e-5)
    lsm = dok.log_softmax(dim=1).coalesce()
    assert torch.allclose(lsm.values().cpu().exp(), sm[tuple(lsm.indices().cpu())], atol=1e-5)
    idx = torch.tensor([3, 0, 17], device=cuda)
    assert torch.equal(dok.index_select(0, idx).to_dense().cpu(), dense[idx.cpu()])
    assert torch.equal(dok.select(1, 4).to_dense().cpu(), dense[:, 4])
    assert torch.equal(dok.abs().to_dense().cpu(), dense.abs())
    assert torch.equal(dok.ceil().to_dense().cpu(), dense.ceil())
    assert torch.equal(dok.floor().to_dense().cpu(), dense.floor())
    assert torch.equal(dok.round().to_dense().cpu(), dense.round())
    assert torch.allclose(dok.abs().sqrt().to_dense().cpu(), dense.abs().sqrt())
    assert torch.equal(dok.flatten().to_dense().cpu(), dense.flatten())
    assert torch.equal(dok.reshape(20, 60).to_dense().cpu(), dense.reshape(20, 60))


def test_constructors_clone_resize_and_conversions(cuda):
    """from_sparse_coo / from_storage / clone / resize / to_sparse_csr / __torch_function__ / repr
    (reference: sparse_dok_tensor.py:71-118, 195-215), against the dense tensor."""
    from doksparse_amd import SparseDOKTensor, sparse_dok_tensor
    gen = torch.Generator(device="cpu"); gen.manual_seed(21)
    dense = torch.zeros(24, 18)
    mask = torch.rand(24, 18, generator=gen) < 0.25
    dense[mask] = torch.randn(int(mask.sum()), generator=gen)
    coo = dense.to_sparse().to(cuda)
    dok = SparseDOKTensor.from_sparse_coo(coo)
    assert torch.equal(dok.to_dense().cpu(), dense) and dok._nnz() == int(mask.sum())
    assert torch.equal(sparse_dok_tensor((24, 18), coo.indices(), coo.values(), device=cuda).to_dense().cpu(), dense)
    # the storage of one tensor makes another: same table, same entries
    twin = SparseDOKTensor.from_storage(dok.storage())
    assert tuple(twin.shape) == (24, 18) and torch.equal(twin.to_dense().cpu(), dense)
    # deep clone is independent, shallow clone shares the table
    deep, shallow = dok.clone(), dok.clone(deepclone=False)
    dok[torch.tensor([0], device=cuda), torch.tensor([0], device=cuda)] = torch.tensor([7.0], device=cuda)
    changed = dense.clone(); changed[0, 0] = 7.0
    assert torch.equal(deep.to_dense().cpu(), dense)
    assert torch.equal(shallow.to_dense().cpu(), changed) and torch.equal(dok.to_dense().cpu(), changed)
    # conversions
    csr = dok.to_sparse_csr()
    assert csr.layout == torch.sparse_csr and torch.equal(csr.to_dense().cpu(), changed)
    assert torch.equal(dok.to_sparse_coo().to_dense().cpu(), changed)
    assert torch.allclose(torch.sparse.sum(dok).cpu(), changed.sum(), atol=1e-5)      # via __torch_function__
    text = repr(dok)
    assert "SparseDOKTensor" in text and f"nnz={dok._nnz()}" in text
    # resize: growing keeps every entry, shrinking keeps the entries inside the new size
    grown = deep.clone().resize(30, 40)
    assert tuple(grown.shape) == (30, 40)
    big = torch.zeros(30, 40); big[:24, :18] = dense
    assert torch.equal(grown.to_dense().cpu(), big)
    shrunk = deep.clone().resize(10)                       # second dimension unchanged
    assert tuple(shrunk.shape) == (10, 18) and torch.equal(shrunk.to_dense().cpu(), dense[:10])
    assert shrunk._nnz() == int(mask[:10].sum())


def _new_dok(shape, idx, vals, dev, rows):
    """A tensor from COO entries; rows=True: on a storage that keeps the int64 coordinate rows as
    multi-word keys (what tensors of 2^63 elements and more, or of more than 8 dimensions, get by
    themselves), so that the kernels of that key format meet every small case as well."""
    from doksparse_amd import SparseDOKTensor, CudaClosedHashmap
    from doksparse_amd.util import next_power_of_2
    from doksparse_amd import _lib
    storage = None
    if rows:
        storage = CudaClosedHashmap(n_buckets=next_power_of_2(vals.shape[0]), device=dev, coord_dims=shape, coord_rows=True)
    dok = SparseDOKTensor(shape, idx.to(dev), vals.to(dev), device=dev, storage=storage)
    if rows and len(shape) >= 2:
        assert dok.storage()._layout == _lib.DOK_LAYOUT_TAGGED and dok.storage()._desc.key_bytes == 8 * len(shape)
    return dok


def _random_selectors(rng, shape):
    """A random indexing expression over the leading dimensions of `shape`: integers, slices,
    index tensors that broadcast to one shape, lists, and at most one 1-D mask (kept apart
    from the index tensors)."""
    n_sel = int(rng.integers(1, len(shape) + 1))
    bshape = tuple(int(x) for x in rng.integers(1, 5, size=int(rng.integers(1, 3))))
    use_mask, mask_done, sel = rng.random() < 0.25, False, []
    for d in range(n_sel):
        s = shape[d]
        kind = rng.choice(["int", "slice", "tensor", "mask", "full", "list"], p=[0.2, 0.2, 0.3, 0.1, 0.15, 0.05])
        if kind == "mask" and (not use_mask or mask_done):
            kind = "slice"
        if kind in ("tensor", "list") and use_mask:
            kind = "slice"
        if kind == "int":
            sel.append(int(rng.integers(0, s)))
        elif kind == "full":
            sel.append(slice(None))
        elif kind == "slice":
            a, b = sorted(int(x) for x in rng.integers(0, s + 1, size=2))
            sel.append(slice(a if rng.random() < 0.8 else None, b if rng.random() < 0.8 else None))
        elif kind == "tensor":
            shp = tuple(x if rng.random() < 0.7 else 1 for x in bshape)
            sel.append(torch.from_numpy(rng.integers(0, s, size=shp)).long())
        elif kind == "list":
            sel.append([int(x) for x in rng.integers(0, s, size=bshape[-1])])
        else:
            m = torch.from_numpy(rng.random(s) < 0.5)
            m[0] = m[0] or not bool(m.any())
            sel.append(m)
            mask_done = True
    return tuple(sel)


@pytest.mark.parametrize("rows", [False, True, "fast"])
def test_random_selectors_against_the_oracle(cuda, rows, monkeypatch):
    """Differential test: random shapes (1 to 5 dimensions), random contents and random indexing
    expressions; every expression the oracle accepts is read through the HIP path and compared,
    then assigned one value through both and the tensors compared.  (Equal coordinates inside
    one assignment: the reference over-counts its element counter, so the entry count is compared
    with the oracle's distinct coordinates.)"""
    from doksparse_amd import SparseDOKTensor, closed_hashmap as ch
    if rows == "fast":
        # every insert through the form with one compare-and-swap per new row and a deferred list
        # (by itself only batches of tens of thousands of rows take it)
        monkeypatch.setattr(ch, "TAGGED_FAST_MIN_ROWS", 0)
    rng = np.random.default_rng(20)
    compared = 0
    for case in range(80):
        # (one to eight dimensions: up to four take the small index descriptor, more the large one)
        nd = int(rng.integers(1, 9))
        shape = tuple(int(x) for x in rng.integers(1, 9 if nd <= 5 else 4, size=nd))
        vol = int(np.prod(shape))
        nnz = max(1, int(rng.integers(0, vol + 1)))
        idx = torch.stack(torch.unravel_index(torch.from_numpy(rng.permutation(vol)[:nnz]), shape))
        vals = torch.from_numpy(rng.integers(1, 100, size=nnz)).float()
        dok = _new_dok(shape, idx, vals, cuda, rows)
        ref = RefSparseDOKTensor(shape, idx, vals, rng=np.random.default_rng(case))
        assert same_entries(dok, ref)
        for _ in range(4):
            sel = _random_selectors(rng, shape)
            dsel = tuple(s.to(cuda) if isinstance(s, torch.Tensor) else s for s in sel)
            try:
                exp = ref[sel]
            except Exception:
                continue                          # rejected by the oracle, as by the reference
            try:
                got = dok[dsel]
            except NotImplementedError as err:    # (an index space of more axes than a descriptor holds)
                assert "axes" in str(err) and len(shape) >= 6
                continue
            assert got.shape == exp.shape and torch.equal(got.cpu(), exp), (shape, sel)
            val = float(rng.integers(-50, 50))
            try:
                ref[sel] = torch.full(exp.shape, val)
            except Exception:
                continue
            dok[dsel] = torch.full(exp.shape, val, device=cuda)
            assert torch.equal(dok.to_dense().cpu(), ref.to_dense()), (shape, sel)
            assert dok._nnz() == np.unique(ref.indices().cpu().numpy(), axis=1).shape[1], (shape, sel)
            compared += 1
    assert compared > 200


@pytest.mark.parametrize("rows", [False, True])
def test_random_selectors_through_permuted_views(cuda, rows):
    """The same differential test through `permute` views: reads and writes through the view must
    equal an oracle tensor built from the permuted coordinates, and the base tensor must see
    the writes (the view shares its table)."""
    from doksparse_amd import SparseDOKTensor
    rng = np.random.default_rng(21)
    compared = 0
    for case in range(50):
        nd = int(rng.integers(2, 6))
        shape = tuple(int(x) for x in rng.integers(1, 8, size=nd))
        vol = int(np.prod(shape))
        nnz = max(1, int(rng.integers(0, vol + 1)))
        idx = torch.stack(torch.unravel_index(torch.from_numpy(rng.permutation(vol)[:nnz]), shape))
        vals = torch.from_numpy(rng.integers(1, 100, size=nnz)).float()
        dok = _new_dok(shape, idx, vals, cuda, rows)
        perm = [int(x) for x in rng.permutation(nd)]
        view = dok.permute(*perm) if case % 2 else dok.permute(perm)
        pshape = tuple(shape[p] for p in perm)
        inverse = [perm.index(d) for d in range(nd)]
        ref = RefSparseDOKTensor(pshape, idx[perm], vals, rng=np.random.default_rng(case))
        assert tuple(view.shape) == pshape
        for _ in range(4):
            sel = _random_selectors(rng, pshape)
            dsel = tuple(s.to(cuda) if isinstance(s, torch.Tensor) else s for s in sel)
            try:
                exp = ref[sel]
            except Exception:
                continue
            got = view[dsel]
            assert got.shape == exp.shape and torch.equal(got.cpu(), exp), (shape, perm, sel)
            val = float(rng.integers(-50, 50))
            try:
                ref[sel] = torch.full(exp.shape, val)
            except Exception:
                continue
            view[dsel] = torch.full(exp.shape, val, device=cuda)
            assert torch.equal(view.to_dense().cpu(), ref.to_dense()), (shape, perm, sel)
            assert torch.equal(dok.to_dense().cpu(), ref.to_dense().permute(*inverse)), (shape, perm, sel)
            assert dok._nnz() == view._nnz()
            compared += 1
    assert compared > 100


@pytest.mark.parametrize("rows", [False, True])
def test_random_sparse_valued_indexing_against_the_oracle(cuda, rows):
    """Differential test of the sparse-valued paths: `__spgetitem__` of random expressions and
    `__setitem__` with a sparse source of the selection's shape (without repeated coordinates,
    where the winner among equal coordinates is not defined)."""
    from doksparse_amd import SparseDOKTensor

    def has_repeats(sel):
        for s in sel:
            s = torch.tensor(s) if isinstance(s, list) else s
            if isinstance(s, torch.Tensor) and s.dtype != torch.bool and s.numel() != s.unique().numel():
                return True
        return False

    rng = np.random.default_rng(22)
    n_get = n_set = 0
    for case in range(60):
        shape = tuple(int(x) for x in rng.integers(1, 8, size=int(rng.integers(1, 5))))
        vol = int(np.prod(shape))
        nnz = max(1, int(rng.integers(0, vol + 1)))
        idx = torch.stack(torch.unravel_index(torch.from_numpy(rng.permutation(vol)[:nnz]), shape))
        vals = torch.from_numpy(rng.integers(1, 100, size=nnz)).float()
        dok = _new_dok(shape, idx, vals, cuda, rows)
        ref = RefSparseDOKTensor(shape, idx, vals, rng=np.random.default_rng(case))
        for _ in range(4):
            sel = _random_selectors(rng, shape)
            dsel = tuple(s.to(cuda) if isinstance(s, torch.Tensor) else s for s in sel)
            try:
                exp = ref.__spgetitem__(sel)
            except Exception:
                continue
            if tuple(exp.shape) == ():
                with pytest.raises(NotImplementedError):     # a result without axes: documented deviation
                    dok.__spgetitem__(dsel)
                continue
            got = dok.__spgetitem__(dsel)
            assert tuple(got.shape) == tuple(exp.shape) and got._nnz() == exp._nnz(), (shape, sel)
            assert torch.equal(got.to_dense().cpu(), exp.to_dense()), (shape, sel)
            n_get += 1
            if has_repeats(sel):
                continue
            src = torch.from_numpy(rng.integers(-9, 10, size=tuple(exp.shape))).float()
            src[torch.from_numpy(rng.random(tuple(exp.shape)) < 0.6)] = 0
            try:
                ref[sel] = src.to_sparse()
            except Exception:
                continue
            dok[dsel] = src.to_sparse().to(cuda)
            assert torch.equal(dok.to_dense().cpu(), ref.to_dense()), (shape, sel)
            n_set += 1
    assert n_get > 150 and n_set > 100


# ---- wide tensors: index spaces of 2^63 elements or more, or more than 8 dimensions ---------------

def _wide_pair(size, nnz, seed, dev, dtype=torch.float32):
    from doksparse_amd import SparseDOKTensor
    rng = np.random.default_rng(seed)
    idx = np.stack([rng.integers(0, s, size=nnz, dtype=np.int64) for s in size])
    idx = np.unique(idx, axis=1)
    idx = torch.from_numpy(idx[:, rng.permutation(idx.shape[1])])
    vals = torch.from_numpy(rng.integers(1, 1000, size=idx.shape[1])).to(dtype)
    dok = SparseDOKTensor(size, idx.to(dev), vals.to(dev), device=dev)
    ref = RefSparseDOKTensor(size, idx, vals, rng=np.random.default_rng(seed))
    return dok, ref, idx, vals


@pytest.mark.parametrize("size", [(2**40, 2**40), (2**31, 2**31, 2**31), (2**62, 5), (2**21,) * 4])
def test_wide_index_space_construct_getitem_setitem_roundtrip(cuda, size):
    """Tensors whose volume is 2^63 or more keep their coordinates as multi-word keys: construct,
    gather (hits, misses, broadcast and slice selectors), scatter (new and present coordinates,
    with growth), read-out - all against the oracle."""
    dok, ref, idx, vals = _wide_pair(size, 5000, 11, cuda)
    assert dok.storage()._coord_rows and dok._nnz() == ref._nnz() == idx.shape[1]
    assert dok.storage().n_buckets == ref._hashmap.n_buckets
    assert same_entries(dok, ref)
    rng = np.random.default_rng(12)
    nd = len(size)
    # gather: stored coordinates mixed with random ones
    pick = torch.from_numpy(rng.integers(0, idx.shape[1], size=3000))
    rand = torch.from_numpy(np.stack([rng.integers(0, s, size=3000, dtype=np.int64) for s in size]))
    q = torch.cat([idx[:, pick], rand], dim=1)[:, torch.from_numpy(rng.permutation(6000))]
    sel = tuple(q[d] for d in range(nd))
    exp = ref[sel]
    got = dok[tuple(x.to(cuda) for x in sel)]
    assert got.shape == exp.shape and torch.equal(got.cpu(), exp) and int((exp != 0).sum()) >= 3000
    # a broadcast block with a slice at the end: rows of stored first coordinates x a window
    first = idx[0, :7]
    last0 = int(idx[-1, 0])
    lo = max(0, min(last0 - 3, size[-1] - 8))
    sel = (first[:, None],) + tuple(idx[d, :5][None, :] for d in range(1, nd - 1)) + (slice(lo, lo + 8),)
    exp = ref[sel]
    got = dok[tuple(x.to(cuda) if isinstance(x, torch.Tensor) else x for x in sel)]
    assert got.shape == exp.shape and torch.equal(got.cpu(), exp)
    # scalar selectors
    one = tuple(int(idx[d, 0]) for d in range(nd))
    assert dok[one].item() == vals[0].item()       # (the reference, and so the oracle, raises here by accident)
    # scatter: half present, half new coordinates; enough to grow the table
    new = torch.from_numpy(np.stack([rng.integers(0, s, size=4000, dtype=np.int64) for s in size]))
    w = torch.cat([idx[:, :4000], new], dim=1)
    wv = torch.from_numpy(rng.integers(-500, 500, size=8000)).float()
    wsel = tuple(w[d] for d in range(nd))
    ref[wsel] = wv
    dok[tuple(x.to(cuda) for x in wsel)] = wv.to(cuda)
    assert dok.storage().n_buckets == ref._hashmap.n_buckets
    a = sorted_coo(dok.indices(), dok.values())
    b = sorted_coo(ref.indices(), ref.values())
    ub, first_of = np.unique(b[0], axis=1, return_index=True)       # (the oracle may hold a repeated coordinate twice)
    assert np.array_equal(a[0], ub) and dok._nnz() == ub.shape[1]
    assert torch.equal(dok[tuple(x.to(cuda) for x in wsel)].cpu(), ref[wsel])
    # out-of-range coordinates: reads give 0, writes raise
    far = tuple(torch.tensor([s + 5]) for s in size)
    assert dok[tuple(x.to(cuda) for x in far)].item() == 0
    with pytest.raises(IndexError):
        dok[tuple(x.to(cuda) for x in far)] = torch.ones(1, device=cuda)
    # count / remove
    csel = tuple(q[d].to(cuda) for d in range(nd))
    n_before = dok._nnz()
    cnt = int(dok.count_items(csel).item())
    dok.zero_items(csel)
    assert int(dok.count_items(csel).item()) == 0
    def rows(a):                                       # [nd, n] coordinates -> n comparable records
        return np.ascontiguousarray(a.T).view([("", np.int64)] * nd).ravel()
    stored_q = np.isin(rows(q.numpy()), rows(ub))
    assert cnt == int(stored_q.sum()) >= 3000
    assert n_before - dok._nnz() == np.unique(rows(q.numpy())[stored_q]).shape[0]
    assert "nnz=" in repr(dok)


def test_wide_many_dimensions_against_the_oracle(cuda):
    """A 10-dimensional tensor (more dimensions than the fused kernels take): random expressions,
    assignments, views, dense read-out and sparse-valued indexing against the oracle."""
    from doksparse_amd import SparseDOKTensor
    size = (3, 2, 4, 3, 2, 3, 2, 2, 3, 2)
    dok, ref, idx, vals = _wide_pair(size, 3000, 21, cuda)
    assert dok.storage()._coord_rows and dok.ndim == 10 and same_entries(dok, ref)
    assert torch.equal(dok.to_dense().cpu(), ref.to_dense())
    rng = np.random.default_rng(22)
    compared = 0
    for _ in range(40):
        sel = _random_selectors(rng, size)
        dsel = tuple(s.to(cuda) if isinstance(s, torch.Tensor) else s for s in sel)
        try:
            exp = ref[sel]
        except Exception:
            continue
        got = dok[dsel]
        assert got.shape == exp.shape and torch.equal(got.cpu(), exp), sel
        val = float(rng.integers(-50, 50))
        try:
            ref[sel] = torch.full(exp.shape, val)
        except Exception:
            continue
        dok[dsel] = torch.full(exp.shape, val, device=cuda)
        assert torch.equal(dok.to_dense().cpu(), ref.to_dense()), sel
        compared += 1
    assert compared >= 15
    # a permuted view shares the storage
    order = (9, 0, 5, 2, 7, 1, 8, 3, 6, 4)
    v = dok.permute(*order)
    dense = ref.to_dense()
    assert torch.equal(v.to_dense().cpu(), dense.permute(*order))
    pos = tuple(int(x) for x in idx[:, 0])
    vpos = tuple(pos[o] for o in order)
    v[vpos] = 777.0
    assert dok[pos].item() == 777.0
    dense[pos] = 777.0
    # sparse-valued gather and scatter
    sel = (torch.tensor([0, 2, 1])[:, None], slice(None), torch.tensor([3, 0])[None, :], 1, 0, 2, 1, 0, 2, 1)
    dsel = tuple(s.to(cuda) if isinstance(s, torch.Tensor) else s for s in sel)
    sp = dok.__spgetitem__(dsel)
    want = dok[dsel]
    assert torch.equal(sp.to_dense().cpu().reshape(want.shape), want.cpu())
    # (result axes: the 3 x 2 broadcast block at the first tensor selector's position, then the slice)
    assert tuple(want.shape) == (3, 2, 2)
    src = torch.zeros(3, 2, 2)
    src[0, 1, 0], src[2, 0, 1] = 5.0, -6.0
    dok[dsel] = src.to_sparse().to(cuda)
    for bi, c0 in enumerate((0, 2, 1)):
        for bj, c2 in enumerate((3, 0)):
            for sl in range(2):
                dense[c0, sl, c2, 1, 0, 2, 1, 0, 2, 1] = src[bi, bj, sl]
    assert torch.equal(dok.to_dense().cpu(), dense)


def test_permuted_dok_tensor_as_sparse_source(cuda):
    """`a[sel] = b.t()` with a DOK source that is a permuted view: the source's coordinates are
    taken in the view's dimension order."""
    from doksparse_amd import SparseDOKTensor
    g = torch.Generator().manual_seed(5)
    b_dense = torch.zeros(6, 4)
    b_dense[torch.randint(0, 6, (9,), generator=g), torch.randint(0, 4, (9,), generator=g)] = torch.randn(9, generator=g)
    b = SparseDOKTensor.from_dense(b_dense.to(cuda))
    a = SparseDOKTensor((10, 12), device=cuda)
    a_dense = torch.zeros(10, 12)
    a[2:6, 3:9] = b.t()
    a_dense[2:6, 3:9] = b_dense.t()
    assert torch.equal(a.to_dense().cpu(), a_dense)
    a[torch.tensor([7, 1, 0, 9])[:, None].to(cuda), torch.tensor([0, 11, 5, 2, 3, 8])[None, :].to(cuda)] = b.permute(1, 0)
    a_dense[torch.tensor([7, 1, 0, 9])[:, None], torch.tensor([0, 11, 5, 2, 3, 8])[None, :]] = b_dense.t()
    assert torch.equal(a.to_dense().cpu(), a_dense)


def test_dok_entry_points_on_coordinate_rows_through_the_c_abi(cuda):
    """The C entry points themselves on a table of int64 coordinate rows (key_bytes = 8 * ndim):
    dok_coo_set, dok_getitem_dense, dok_setitem_dense, dok_count_items, dok_zero_items,
    dok_coo_compact and dok_to_dense called through ctypes with hand-filled descriptors, on a
    (2^40, 2^40) index space and on a small one that a dense torch tensor can mirror."""
    import ctypes
    from doksparse_amd import _lib
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def table(dims, n_buckets, vbytes=4):
        t = _lib.DokTable()
        mem = torch.empty(n_buckets * 128, device=cuda, dtype=torch.uint8)
        header = torch.empty(16, device=cuda, dtype=torch.long)
        t.buckets, t.header, t.n_phys_buckets, t.seed = mem.data_ptr(), header.data_ptr(), n_buckets, 99
        t.key_bytes, t.value_bytes, t.lin_ndim = 8 * len(dims), vbytes, len(dims)
        for i, d in enumerate(dims):
            t.lin_dims[i] = d
        assert lib.dok_table_clear(ctypes.byref(t), st) == 0
        return t, mem, header

    def index(ndim, shape, sels):
        ix = _lib.DokIndex()
        ix.ndim, ix.sel_ndim = ndim, len(shape)
        for j, s in enumerate(shape):
            ix.shape[j] = s
        for d, (ptr, base, strides) in enumerate(sels):
            ix.sel[d].data, ix.sel[d].base = ptr, base
            for j, sd in enumerate(strides):
                ix.sel[d].strides[j] = sd
        return ix

    # ---- (2^40, 2^40): 20,000 entries
    rng = np.random.default_rng(31)
    n = 20000
    coords = np.ascontiguousarray(np.unique(rng.integers(0, 2**40, size=(2, n), dtype=np.int64), axis=1))
    n = coords.shape[1]
    vals = rng.standard_normal(n).astype(np.float32)
    t, mem, header = table((2**40, 2**40), 16384)
    ci, cv = torch.from_numpy(coords).to(cuda), torch.from_numpy(vals).to(cuda)
    assert ci.is_contiguous()
    assert lib.dok_coo_set(ctypes.byref(t), ci.data_ptr(), cv.data_ptr(), n, st) == 0
    assert int(header[_lib.DOK_H_NELEM]) == n and int(header[_lib.DOK_H_NOOB]) == 0
    # gather: every stored coordinate in reverse order, plus misses, through two 1-D selectors
    q = np.concatenate([coords[:, ::-1], rng.integers(0, 2**40, size=(2, 500), dtype=np.int64)], axis=1)
    qd = torch.from_numpy(np.ascontiguousarray(q)).to(cuda)
    out = torch.full((q.shape[1],), -1.0, device=cuda)
    ix = index(2, (q.shape[1],), [(qd[0].data_ptr(), 0, (1,)), (qd[1].data_ptr(), 0, (1,))])
    assert lib.dok_getitem_dense(ctypes.byref(t), ctypes.byref(ix), out.data_ptr(), st) == 0
    expect = np.concatenate([vals[::-1], np.zeros(500, dtype=np.float32)])
    assert np.array_equal(out.cpu().numpy(), expect)
    cnt = torch.zeros(1, device=cuda, dtype=torch.long)
    assert lib.dok_count_items(ctypes.byref(t), ctypes.byref(ix), cnt.data_ptr(), st) == 0
    assert int(cnt) == n
    # an affine selector without a device tensor: row coords[0, 0], columns coords[1, 0] - 3 .. + 4
    r0, c0 = int(coords[0, 0]), int(coords[1, 0])
    lo = max(c0 - 3, 0)
    ix2 = index(2, (8,), [(None, r0, (0,)), (None, lo, (1,))])
    out8 = torch.full((8,), -1.0, device=cuda)
    assert lib.dok_getitem_dense(ctypes.byref(t), ctypes.byref(ix2), out8.data_ptr(), st) == 0
    model = {(int(a), int(b)): float(v) for a, b, v in zip(coords[0], coords[1], vals)}
    assert out8.cpu().tolist() == [model.get((r0, lo + k), 0.0) for k in range(8)]
    # scatter through the same descriptor (8 cells of one row), then remove them again
    src = torch.arange(1, 9, device=cuda, dtype=torch.float32)
    view = _lib.DokView()
    view.data = src.data_ptr()
    view.strides[0] = 1
    before = sum((r0, lo + k) in model for k in range(8))
    assert lib.dok_setitem_dense(ctypes.byref(t), ctypes.byref(ix2), ctypes.byref(view), st) == 0
    assert int(header[_lib.DOK_H_NELEM]) == n + 8 - before
    assert lib.dok_getitem_dense(ctypes.byref(t), ctypes.byref(ix2), out8.data_ptr(), st) == 0
    assert out8.cpu().tolist() == list(range(1, 9))
    assert lib.dok_zero_items(ctypes.byref(t), ctypes.byref(ix2), st) == 0
    assert int(header[_lib.DOK_H_NELEM]) == n - before
    # rows outside the coordinate space: skipped and counted by the insert, absent for the lookups
    bad = torch.tensor([[2**40, -1, 5], [7, 7, 2**40 + 1]], device=cuda)
    assert lib.dok_coo_set(ctypes.byref(t), bad.data_ptr(), cv.data_ptr(), 3, st) == 0
    assert int(header[_lib.DOK_H_NOOB]) == 3 and int(header[_lib.DOK_H_NELEM]) == n - before
    # read-out in COO layout
    scratch = torch.empty(int(lib.dok_compact_scratch_bytes(ctypes.byref(t))) // 8, device=cuda, dtype=torch.long)
    live = n - before
    oi = torch.zeros(2, live, device=cuda, dtype=torch.long)
    ov = torch.zeros(live, device=cuda)
    assert lib.dok_coo_compact(ctypes.byref(t), oi.data_ptr(), ov.data_ptr(), live, cnt.data_ptr(), scratch.data_ptr(), st) == 0
    assert int(cnt) == live
    for k in range(8):
        model.pop((r0, lo + k), None)
    got = {(int(a), int(b)): float(v) for a, b, v in zip(oi[0].cpu(), oi[1].cpu(), ov.cpu())}
    assert got == model
    # a linear key cannot hold this space: the descriptor with key_bytes 8 is refused, not misread
    t.key_bytes = 8
    assert lib.dok_getitem_dense(ctypes.byref(t), ctypes.byref(ix), out.data_ptr(), st) == _lib.DOK_EUNSUPPORTED

    # ---- a small 3-D space mirrored by a dense tensor; float16 values
    dims = (6, 5, 7)
    dense = torch.zeros(dims, dtype=torch.float16)
    flat = torch.from_numpy(rng.permutation(6 * 5 * 7)[:90])
    c3 = torch.stack(torch.unravel_index(flat, dims))
    v3 = torch.from_numpy(rng.integers(1, 50, size=90)).to(torch.float16)
    dense[tuple(c3)] = v3
    t3, mem3, header3 = table(dims, 64, vbytes=2)
    c3d, v3d = c3.contiguous().to(cuda), v3.to(cuda)
    assert lib.dok_coo_set(ctypes.byref(t3), c3d.data_ptr(), v3d.data_ptr(), 90, st) == 0
    dd = torch.zeros(dims, device=cuda, dtype=torch.float16)
    assert lib.dok_to_dense(ctypes.byref(t3), dd.data_ptr(), st) == 0
    assert torch.equal(dd.cpu(), dense)
    # dok[rows[:, None], 1:4, cols[None, :]] -> (3, 2, 3) by the reference's axis rule: block first, slice after
    rows_ = torch.tensor([4, 0, 5], device=cuda)
    cols_ = torch.tensor([6, 2], device=cuda)
    ix3 = index(3, (3, 2, 3), [(rows_.data_ptr(), 0, (1, 0, 0)), (None, 1, (0, 0, 1)), (cols_.data_ptr(), 0, (0, 1, 0))])
    o3 = torch.zeros(3, 2, 3, device=cuda, dtype=torch.float16)
    assert lib.dok_getitem_dense(ctypes.byref(t3), ctypes.byref(ix3), o3.data_ptr(), st) == 0
    want = dense[rows_.cpu()[:, None, None], torch.arange(1, 4)[None, None, :], cols_.cpu()[None, :, None]]
    assert torch.equal(o3.cpu(), want)
