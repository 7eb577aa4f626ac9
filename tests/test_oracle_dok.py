"""Pins the CPU oracle of the DOK tensor (oracle/ref_dok.py) against dense torch indexing.

The reference's selector rule coincides with torch/numpy advanced indexing whenever the tensor
selectors are adjacent or there is at most one of them; where they are separated by a slice it
differs in a way that is a pure axis move, which is checked against the moved torch result."""
import numpy as np
import pytest
import torch

from oracle.ref_dok import RefSparseDOKTensor, next_power_of_2, shape_to_stride


def make(shape, nnz, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    flat = torch.randperm(int(np.prod(shape)), generator=g)[:nnz]
    idx = torch.stack(torch.unravel_index(flat, shape))
    vals = (torch.randn(nnz, generator=g) * 10).to(dtype)
    vals[vals == 0] = 1
    dense = torch.zeros(shape, dtype=dtype)
    dense[tuple(idx)] = vals
    return RefSparseDOKTensor(shape, idx, vals, rng=np.random.default_rng(seed)), dense


def test_helpers():
    assert [next_power_of_2(n) for n in (0, 1, 2, 3, 4, 5, 1023, 1024, 1025)] == [1, 1, 2, 4, 4, 8, 1024, 1024, 2048]
    for shape in [(7,), (3, 4), (2, 3, 5), (4, 1, 6, 2)]:
        assert shape_to_stride(shape) == torch.empty(shape).stride()
    assert shape_to_stride(()) == ()


def test_construct_and_to_dense():
    dok, dense = make((13, 17), 60, 1)
    assert dok._nnz() == 60
    # next_power_of_2(60) = 64 slots, then 60 > int(0.75 * 64) grows to int(60 * 2.0)
    assert dok._hashmap.n_buckets == 120
    assert torch.equal(dok.to_dense(), dense)
    order = np.lexsort(dok.indices().numpy()[::-1])
    assert torch.equal(dok.indices()[:, order], dense.nonzero().T)


CASES_2D = [
    lambda r, c: (r, c),                                   # paired coordinates
    lambda r, c: (r[:, None], c[None, :]),                 # outer product
    lambda r, c: (r,),                                     # rows, implicit full slice
    lambda r, c: (slice(None), c),
    lambda r, c: (slice(2, 9), slice(None, 5)),
    lambda r, c: (slice(None), slice(None)),
    lambda r, c: (r.tolist(), slice(1, 4)),
    lambda r, c: (r.to(torch.int32), c.to(torch.int16)),
    lambda r, c: (slice(5, 3), c),                         # empty range
]


@pytest.mark.parametrize("case", range(len(CASES_2D)))
def test_getitem_2d_matches_dense(case):
    dok, dense = make((13, 17), 80, 2)
    g = torch.Generator().manual_seed(case)
    r = torch.randint(0, 13, (6,), generator=g)
    c = torch.randint(0, 17, (6,), generator=g)
    sel = CASES_2D[case](r, c)
    tsel = tuple(s.long() if isinstance(s, torch.Tensor) else s for s in sel)
    assert torch.equal(dok[sel], dense[tsel])


def test_getitem_scalars_masks_and_higher_rank():
    dok, dense = make((6, 7, 5, 4), 700, 3)
    i = torch.tensor([0, 5, 2])
    j = torch.tensor([1, 1, 6])
    m = torch.tensor([True, False, True, True])
    assert torch.equal(dok[3], dense[3])                       # bare int: squeeze(0) of a size-? axis
    assert torch.equal(dok[3, 2], dense[3, 2])
    assert torch.equal(dok[i, j], dense[i, j])
    assert torch.equal(dok[i, j, 1:4], dense[i, j, 1:4])
    assert torch.equal(dok[:, :, :, m], dense[:, :, :, m])
    assert torch.equal(dok[i, :, :, torch.tensor([0, 2, 3])], dense[i, :, :, torch.tensor([0, 2, 3])])
    # 2-d boolean mask over the first two dimensions
    m2 = dense[:, :, 0, 0] != 0
    m2[0, 0] = True
    assert torch.equal(dok[m2], dense[m2])
    # scalar followed by a slice and tensors
    # (the scalar counts as the first tensor selector, so the broadcast axis comes first; torch
    # treats the int as a plain select and keeps the broadcast axis behind the slice)
    got = dok[4, :3, i[:2] % 5, j[:2] % 4]
    assert got.shape == (2, 3)
    assert torch.equal(got, dense[4, :3, i[:2] % 5, j[:2] % 4].T)


def test_axis_rule_when_a_slice_separates_tensor_selectors():
    dok, dense = make((6, 7, 5, 4), 700, 4)
    i = torch.tensor([0, 5, 2])
    k = torch.tensor([3, 0, 1])
    # numpy/torch put the broadcast axis first; the reference keeps it at the first tensor's place
    got = dok[:, i, :, k]
    assert got.shape == (6, 3, 5)
    assert torch.equal(got, dense[:, i, :, k].movedim(0, 1))
    # tensor first: both rules agree
    assert torch.equal(dok[i, :, k], dense[i, :, k])


def test_scalar_squeeze_quirks():
    dok, dense = make((6, 7, 5), 180, 5)
    # a scalar selector at position p squeezes result axis p when that axis has size 1 ...
    assert dok[0, 3:4, :].shape == (5,)                       # numpy would give (1, 5)
    assert torch.equal(dok[0, 3:4, :], dense[0, 3, :])
    # ... leaves it alone when it has another size ...
    assert torch.equal(dok[2, :, :], dense[2])
    # ... and raises, as the reference does, when the result has no such axis
    with pytest.raises(IndexError):
        dok[:, 2, 3]


def test_setitem_matches_dense_assignment():
    dok, dense = make((13, 17), 40, 6)
    g = torch.Generator().manual_seed(0)
    flat = torch.randperm(13 * 17, generator=g)[:50]
    r, c = flat // 17, flat % 17
    v = torch.randn(50, generator=g)
    n_existing = int((dense[r, c] != 0).sum())
    dok[r, c] = v
    dense[r, c] = v
    assert torch.equal(dok.to_dense(), dense)
    assert dok._nnz() == 40 + 50 - n_existing
    # broadcasting of the source over an outer-product selector, and scalar assignment
    rows, cols = torch.tensor([1, 4, 7]), torch.tensor([0, 16])
    dok[rows[:, None], cols[None, :]] = torch.tensor([5.0, 6.0])
    dense[rows[:, None], cols[None, :]] = torch.tensor([5.0, 6.0])
    dok[2:4, 5:9] = 3.5
    dense[2:4, 5:9] = 3.5
    assert torch.equal(dok.to_dense(), dense)
    assert torch.equal(dok[rows[:, None], :], dense[rows[:, None], :])


def test_setitem_stores_explicit_zeros_and_grows_like_the_reference():
    dok = RefSparseDOKTensor((100, 100), rng=np.random.default_rng(1))
    idx = torch.arange(100)
    dok[idx, idx] = torch.zeros(100)
    assert dok._nnz() == 100                                   # zeros are entries too
    # bootstrap insert (1 element, 32 buckets), then 1 + 100 > 32*0.75 -> ceil(101 * 2) buckets
    assert dok._hashmap.n_buckets == 202
    dok[idx, idx] = 1.0
    assert torch.equal(dok.to_dense(), torch.eye(100))
    assert dok._nnz() == 100


def test_empty_tensor_reads_zero():
    dok = RefSparseDOKTensor((5, 6))
    assert torch.equal(dok[1:3, :], torch.zeros(2, 6))
    assert dok.indices().shape == (2, 0) and dok.values().shape == (0,)


def test_sparse_valued_getitem_matches_dense_slice():
    dok, dense = make((9, 11, 6), 250, 9)
    for sel in [(slice(2, 7), torch.tensor([1, 3, 5, 10]), slice(None)),
                (torch.tensor([0, 8, 3])[:, None], torch.tensor([2, 2, 9])[None, :], 4),
                (slice(None), slice(None), slice(None))]:
        sp = dok.__spgetitem__(sel)
        exp = dense[sel]
        assert tuple(sp.shape) == tuple(exp.shape)
        assert torch.equal(sp.to_dense(), exp)
        assert sp._nnz() == int((exp != 0).sum())
        assert sp._hashmap.n_buckets == int(sp._nnz() * 2.0)
    # an explicitly stored zero is an entry of the result
    dok[0, 0, 0] = 0.0
    n0 = int((dense[0:2] != 0).sum()) + (1 if dense[0, 0, 0] == 0 else 0)
    assert dok.__spgetitem__((slice(0, 2),))._nnz() == n0


def test_sparse_valued_setitem_matches_dense_assignment():
    dok, dense = make((9, 11), 40, 10)
    src = torch.zeros(5, 4)
    src[0, 1], src[3, 2], src[4, 0], src[2, 2] = 7.0, -2.0, 5.0, 1.5
    cols = torch.tensor([1, 3, 5, 10])
    n_before = dok._nnz()
    n_removed = int((dense[2:7][:, cols] != 0).sum())
    dok[2:7, cols] = src.to_sparse()
    dense[2:7, cols] = src                      # zeros of the source clear the destination
    assert torch.equal(dok.to_dense(), dense)
    assert dok._nnz() == int((dense != 0).sum())
    assert dok._hashmap.n_buckets == int(np.ceil((n_before - n_removed + 4) * 2.0 * 2))
    # DOK source; minus zero in a floating source is skipped
    src2 = RefSparseDOKTensor((5, 4), torch.tensor([[0, 1, 4], [0, 1, 3]]), torch.tensor([-0.0, 4.0, 2.0]))
    dok[2:7, cols] = src2
    d2 = torch.zeros(5, 4)
    d2[1, 1], d2[4, 3] = 4.0, 2.0
    dense[2:7, cols] = d2
    assert torch.equal(dok.to_dense(), dense)
