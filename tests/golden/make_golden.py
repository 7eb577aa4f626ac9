"""Writes the regression vectors under tests/golden/.

The reference repository holds no tests, fixtures or golden vectors for the hashmap / DOK path
(its own `tests` directory is git-ignored upstream) and cannot be imported here (CuPy, nvcc and a
CUDA device are absent), so there is nothing of the reference to record.  What this script
records instead are small seeded input/output cases produced by the CPU oracle AFTER it has
been pinned by tests/test_oracle_*.py; they guard both the oracle and the HIP path against
regressions and let the GPU tests run even where the oracle's C library could not be built.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.ref_dok import RefSparseDOKTensor      # noqa: E402
from oracle.ref_hashmap import RefClosedHashmap    # noqa: E402


def hashmap_case(name, key_shape, key_dtype, value_shape, value_dtype, seed):
    rng = np.random.default_rng(seed)
    n = 300
    keys = np.unique(rng.integers(0, 1000, size=(2 * n, *key_shape)).astype(key_dtype).reshape(2 * n, -1), axis=0)
    rng.shuffle(keys)
    keys = keys[:n].reshape(-1, *key_shape)
    vals = rng.integers(-1000, 1000, size=(keys.shape[0], *value_shape)).astype(value_dtype)
    absent = (rng.integers(2000, 3000, size=(100, *key_shape))).astype(key_dtype)
    m = RefClosedHashmap(n_buckets=64, rng=np.random.default_rng(seed + 1))
    m.set(keys, vals)
    q = np.concatenate([keys[::2], absent])
    get_v, get_f = m.get(q, fallback_value=-1)
    gone = keys[: len(keys) // 3]
    rem = m.remove(np.concatenate([gone, absent[:10]]))
    get2_v, get2_f = m.get(q)
    vals2 = rng.integers(-1000, 1000, size=(gone.shape[0], *value_shape)).astype(value_dtype)
    m.set(gone[::-1], vals2)                                   # re-insert through the tombstones
    get3_v, get3_f = m.get(q)
    order = np.lexsort(m.keys().reshape(m.n_elements, -1).view(np.uint8).reshape(m.n_elements, -1).T[::-1])
    np.savez_compressed(os.path.join(HERE, name + ".npz"), keys=keys, vals=vals, q=q, get_v=get_v, get_f=get_f,
                        gone=gone, absent10=absent[:10], rem=rem, get2_v=get2_v, get2_f=get2_f, vals2=vals2,
                        get3_v=get3_v, get3_f=get3_f, n_buckets=m.n_buckets, n_elements=m.n_elements,
                        final_keys=m.keys()[order], final_vals=m.values()[order])


def dok_case(name, seed):
    g = torch.Generator().manual_seed(seed)
    shape = (7, 9, 5)
    flat = torch.randperm(int(np.prod(shape)), generator=g)[:120]
    idx = torch.stack(torch.unravel_index(flat, shape))
    vals = torch.randint(1, 100, (120,), generator=g).float()
    dok = RefSparseDOKTensor(shape, idx, vals, rng=np.random.default_rng(seed))
    i, k = torch.tensor([0, 6, 2]), torch.tensor([3, 0, 1])
    out = {"idx": idx.numpy(), "vals": vals.numpy(), "i": i.numpy(), "k": k.numpy()}
    out["g_pair"] = dok[i, :, k].numpy()
    out["g_sep"] = dok[:, i, k].numpy()
    out["g_mid"] = dok[2:6, k[:, None], i[None, :] % 5].numpy()
    out["g_scalar"] = dok[3].numpy()
    r, c = torch.tensor([1, 1, 4, 6]), torch.tensor([8, 0, 2, 2])
    dok[r, c, 1:4] = torch.arange(12.0).reshape(4, 3)
    dok[5] = 2.5
    out["r"], out["c"] = r.numpy(), c.numpy()
    out["dense_after"] = dok.to_dense().numpy()
    out["nnz_after"] = dok._nnz()
    out["n_buckets_after"] = dok._hashmap.n_buckets
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


if __name__ == "__main__":
    hashmap_case("hashmap_i64_f32", (1,), np.int64, (1,), np.float32, 101)
    hashmap_case("hashmap_f32x3_i64x5", (3,), np.float32, (5,), np.int64, 102)
    hashmap_case("hashmap_i64x2_f16", (2,), np.int64, (1,), np.float16, 103)
    dok_case("dok_3d_f32", 104)
    print("written:", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
