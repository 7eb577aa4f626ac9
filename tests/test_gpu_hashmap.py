"""GPU parity: the HIP hashmap (through the C ABI) against the CPU oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle.ref_hashmap import RefClosedHashmap

pytestmark = pytest.mark.gpu


def _sorted_items(keys, values):
    """Order-independent view of a key->value map: rows sorted by key bytes."""
    k = np.ascontiguousarray(keys).reshape(keys.shape[0], -1)
    v = np.ascontiguousarray(values).reshape(values.shape[0], -1)
    kb = k.view(np.uint8).reshape(k.shape[0], -1)
    order = np.lexsort(kb.T[::-1])
    return k[order], v[order]


def _assert_same_map(hm, ref):
    keys, values = hm.items()
    rk, rv = ref.keys(), ref.values()
    assert hm.n_elements == ref.n_elements == keys.shape[0] == rk.shape[0]
    a = _sorted_items(keys.cpu().numpy(), values.cpu().numpy())
    b = _sorted_items(rk, rv)
    assert a[0].tobytes() == b[0].tobytes()
    assert a[1].tobytes() == b[1].tobytes()


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
