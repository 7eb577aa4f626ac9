"""Committed regression vectors (tests/golden/*.npz, written by tests/golden/make_golden.py).

The CPU tests replay each case through the oracle; the GPU tests replay it through the HIP
library and compare with the recorded outputs directly, without the oracle in the loop."""
import glob
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
HASHMAP_CASES = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN, "hashmap_*.npz")))


def _load(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False)


def _same(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


def _sorted(keys, vals):
    n = keys.shape[0]
    kb = np.ascontiguousarray(keys).reshape(n, -1).view(np.uint8).reshape(n, -1)
    order = np.lexsort(kb.T[::-1])
    return keys[order], vals[order]


def test_fixtures_present():
    assert len(HASHMAP_CASES) == 3 and os.path.exists(os.path.join(GOLDEN, "dok_3d_f32.npz"))


def _replay_hashmap(g, make, to_dev, to_np):
    m = make()
    m.set(to_dev(g["keys"]), to_dev(g["vals"]))
    v, f = m.get(to_dev(g["q"]), fallback_value=-1)
    assert _same(to_np(f), g["get_f"]) and _same(to_np(v), g["get_v"])
    rem = m.remove(to_dev(np.concatenate([g["gone"], g["absent10"]])))
    assert _same(to_np(rem), g["rem"])
    v, f = m.get(to_dev(g["q"]))
    assert _same(to_np(f), g["get2_f"])
    assert _same(to_np(v)[g["get2_f"]], g["get2_v"][g["get2_f"]])
    m.set(to_dev(g["gone"][::-1].copy()), to_dev(g["vals2"]))
    v, f = m.get(to_dev(g["q"]))
    assert _same(to_np(f), g["get3_f"])
    assert _same(to_np(v)[g["get3_f"]], g["get3_v"][g["get3_f"]])
    assert m.n_buckets == int(g["n_buckets"]) and m.n_elements == int(g["n_elements"])
    return m


@pytest.mark.parametrize("name", HASHMAP_CASES)
def test_oracle_reproduces_hashmap_fixture(name):
    from oracle.ref_hashmap import RefClosedHashmap
    g = _load(name)
    m = _replay_hashmap(g, lambda: RefClosedHashmap(n_buckets=64, rng=np.random.default_rng(5)),
                        lambda a: a, lambda a: a)
    k, v = _sorted(m.keys(), m.values())
    assert _same(k, g["final_keys"]) and _same(v, g["final_vals"])


def _replay_dok(g, make):
    dok = make(torch.from_numpy(g["idx"]), torch.from_numpy(g["vals"]))
    dev = dok.device if hasattr(dok, "device") else "cpu"
    i, k = torch.from_numpy(g["i"]).to(dev), torch.from_numpy(g["k"]).to(dev)
    assert _same(dok[i, :, k].cpu().numpy(), g["g_pair"])
    assert _same(dok[:, i, k].cpu().numpy(), g["g_sep"])
    assert _same(dok[2:6, k[:, None], i[None, :] % 5].cpu().numpy(), g["g_mid"])
    assert _same(dok[3].cpu().numpy(), g["g_scalar"])
    r, c = torch.from_numpy(g["r"]).to(dev), torch.from_numpy(g["c"]).to(dev)
    dok[r, c, 1:4] = torch.arange(12.0).reshape(4, 3).to(dev)
    dok[5] = 2.5
    assert _same(dok.to_dense().cpu().numpy(), g["dense_after"])
    assert dok._nnz() == int(g["nnz_after"])
    assert dok._hashmap.n_buckets == int(g["n_buckets_after"])


def test_oracle_reproduces_dok_fixture():
    from oracle.ref_dok import RefSparseDOKTensor
    _replay_dok(_load("dok_3d_f32"),
                lambda idx, vals: RefSparseDOKTensor((7, 9, 5), idx, vals, rng=np.random.default_rng(9)))


@pytest.mark.gpu
@pytest.mark.parametrize("name", HASHMAP_CASES)
def test_hip_reproduces_hashmap_fixture(cuda, name):
    from doksparse_amd import CudaClosedHashmap
    g = _load(name)
    m = _replay_hashmap(g, lambda: CudaClosedHashmap(n_buckets=64, device=cuda),
                        lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(cuda),
                        lambda t: t.cpu().numpy())
    keys, vals = m.items()
    k, v = _sorted(keys.cpu().numpy(), vals.cpu().numpy())
    assert _same(k, g["final_keys"]) and _same(v, g["final_vals"])


@pytest.mark.gpu
def test_hip_reproduces_dok_fixture(cuda):
    from doksparse_amd import SparseDOKTensor
    _replay_dok(_load("dok_3d_f32"),
                lambda idx, vals: SparseDOKTensor((7, 9, 5), idx.to(cuda), vals.to(cuda)))
