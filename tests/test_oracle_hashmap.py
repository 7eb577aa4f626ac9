"""Pins the CPU oracle of the hashmap (oracle/closed_hashmap_ref.c + oracle/ref_hashmap.py).

The reference ships no tests, fixtures or golden vectors for this path, so the oracle is pinned
by what the mathematics fixes: an arbitrary-precision evaluation of the two universal hashes and
closed-form special cases; a Python dict as the model of the key->value map; and hand-derived
slot placements of linear probing with tombstones on tiny tables."""
import numpy as np
import pytest

from oracle.ref_hashmap import RefClosedHashmap, next_prime


def consts(ks, prime1, prime2, alpha1=1, beta1=0, alpha2=1, beta2=0):
    f = lambda v: np.array([v] * ks if np.isscalar(v) else v, dtype=np.int64)
    return dict(prime1=f(prime1), prime2=f(prime2), alpha1=f(alpha1), alpha2=f(alpha2),
                beta1=f(beta1), beta2=f(beta2))


def wrap64(x):
    x &= (1 << 64) - 1
    return x - (1 << 64) if x >= (1 << 63) else x


def c_rem(a, p):
    """C remainder: sign follows the dividend."""
    r = abs(a) % p
    return -r if a < 0 else r


def big_hash(words, alpha, beta, prime):
    h = None
    for w, a, b, p in zip(words, alpha, beta, prime):
        t = c_rem(wrap64(wrap64(int(w) * int(a)) + int(b)), int(p))
        h = t if h is None else wrap64(h * t)
    if h == -(1 << 63):
        return 0
    return abs(h)


def test_next_prime():
    assert [next_prime(n) for n in (0, 1, 2, 3, 13, 14, 89, 7919)] == [2, 2, 3, 5, 17, 17, 97, 7927]
    # strictly greater, also above 2^32 and for a Carmichael number
    assert next_prime(561) == 563 and next_prime(2**61 - 1) > 2**61 - 1
    assert next_prime(4294967291) == 4294967311


@pytest.mark.parametrize("ks", [1, 2, 3])
def test_hashes_match_big_integer_evaluation(ks):
    rng = np.random.default_rng(ks)
    c = dict(
        prime1=np.array([next_prime(int(rng.integers(1000, 2000))) for _ in range(ks)], dtype=np.int64),
        prime2=np.array([next_prime(int(rng.integers(0, 2**60))) for _ in range(ks)], dtype=np.int64),
        alpha1=rng.integers(-1, 2000, ks), alpha2=rng.integers(-1, 2**40, ks),
        beta1=rng.integers(-1, 2000, ks), beta2=rng.integers(-1, 2**40, ks),
    )
    c = {k: v.astype(np.int64) for k, v in c.items()}
    m = RefClosedHashmap(n_buckets=1024, constants=c)
    keys = rng.integers(-2**63, 2**63 - 1, size=(200, ks), dtype=np.int64)
    keys[0] = 0
    keys[1] = -1
    keys[2] = np.iinfo(np.int64).min
    m.set(keys[:1], np.zeros((1, 1), dtype=np.float32))
    h1, h2 = m.hashes_of(keys)
    for r in range(keys.shape[0]):
        assert h1[r] == big_hash(keys[r], c["alpha1"], c["beta1"], c["prime1"])
        assert h2[r] == big_hash(keys[r], c["alpha2"], c["beta2"], c["prime2"])


def test_hash_closed_forms():
    # alpha=1, beta=0, prime > key: the hash is the key; two words: the product; negative keys:
    # C remainder keeps the sign, then the absolute value is taken
    m = RefClosedHashmap(n_buckets=64, constants=consts(2, 1_000_003, 1_000_033))
    keys = np.array([[5, 7], [0, 9], [-5, 7], [1_000_003 + 4, 3]], dtype=np.int64)
    m.set(keys[:1], np.zeros((1, 1), dtype=np.int64))
    h1, h2 = m.hashes_of(keys)
    assert h1.tolist() == [35, 0, 35, 12]
    assert h2.tolist() == [35, 0, 35, (1_000_003 + 4) % 1_000_033 * 3]


def test_float_keys_hash_bit_patterns_and_keep_signed_zero_apart():
    m = RefClosedHashmap(n_buckets=64, constants=consts(1, 2_147_483_659, 2_147_483_659))
    keys = np.array([[1.0], [0.0], [-0.0], [2.5]], dtype=np.float32)
    m.set(keys, np.arange(4, dtype=np.int64)[:, None])
    h1, _ = m.hashes_of(keys)
    bits = keys.view(np.int32).astype(np.int64).ravel()
    assert h1[0] == bits[0] and h1[3] == bits[3]
    assert h1[1] == h1[2] == 0                      # minus zero hashes like plus zero ...
    v, f = m.get(keys)
    assert f.all() and v.ravel().tolist() == [0, 1, 2, 3]   # ... but is a key of its own
    assert m.n_elements == 4


def _dict_check(m, model, probe_keys):
    v, f = m.get(probe_keys, fallback_value=-7)
    for r, k in enumerate(probe_keys):
        kb = k.tobytes()
        assert bool(f[r]) == (kb in model)
        exp = model[kb] if kb in model else np.full(v.shape[1:], -7, dtype=v.dtype)
        assert np.array_equal(v[r], exp)
    assert m.n_elements == len(model)
    ks, vs = m.keys(), m.values()
    assert ks.shape[0] == len(model)
    assert {k.tobytes(): tuple(x.ravel().tolist()) for k, x in zip(ks, vs)} == \
        {k: tuple(x.ravel().tolist()) for k, x in model.items()}


@pytest.mark.parametrize("key_shape,key_dtype,value_shape,value_dtype", [
    ((1,), np.int64, (1,), np.int64),
    ((3,), np.float32, (5,), np.int64),
    ((2,), np.int64, (1,), np.float32),
    ((4,), np.int32, (2,), np.float64),
])
def test_random_sequences_against_dict(key_shape, key_dtype, value_shape, value_dtype):
    rng = np.random.default_rng(42)
    m = RefClosedHashmap(n_buckets=16, rng=np.random.default_rng(3))
    model = {}
    universe = rng.integers(0, 50, size=(120, *key_shape)).astype(key_dtype)   # small: many repeats
    for step in range(40):
        op = rng.integers(0, 3)
        idx = rng.integers(0, universe.shape[0], size=rng.integers(0, 25))
        keys = universe[idx]
        if op <= 1:
            vals = rng.integers(-100, 100, size=(keys.shape[0], *value_shape)).astype(value_dtype)
            n_before, b_before = m.n_elements, m.n_buckets
            m.set(keys, vals)
            n_new = len({k.tobytes() for k in keys} - set(model))
            for k, v in zip(keys, vals):
                model[k.tobytes()] = v                      # sequential: the last row wins
            # growth rule of CudaClosedHashmap.set
            if n_before + n_new > int(0.75 * b_before):
                assert m.n_buckets == int((n_before + n_new) * 2.0)
            else:
                assert m.n_buckets == b_before
        elif model or m._keys is not None:
            mask = m.remove(keys)
            uniq = np.unique(keys.reshape(keys.shape[0], -1), axis=0) if keys.shape[0] else keys
            assert mask.shape[0] == uniq.shape[0]
            for r, k in enumerate(uniq):
                assert bool(mask[r]) == (k.astype(key_dtype).tobytes() in model)
                model.pop(k.astype(key_dtype).tobytes(), None)
        if m._keys is not None:
            _dict_check(m, model, universe)


def test_placement_known_answers():
    # h1(key) = key (alpha 1, beta 0, big prime), B = 8: linear probing from key % 8
    m = RefClosedHashmap(n_buckets=8, rehash_threshold=2.0, constants=consts(1, 1_000_003, 1_000_033))
    val = lambda *xs: np.array(xs, dtype=np.int64)[:, None]
    m.set(val(0, 8, 16), val(10, 11, 12))
    assert m.slots_of(val(0, 8, 16)).tolist() == [0, 1, 2]           # one collision chain
    m.set(val(7, 15), val(13, 14))
    assert m.slots_of(val(7, 15)).tolist() == [7, 3]                 # 15 wraps past 0,1,2
    assert m.remove(val(8)).tolist() == [True]
    assert m._uuid[1] == -3
    assert m.slots_of(val(16)).tolist() == [2]                       # found across the tombstone
    m.set(val(24), val(15))
    assert m.slots_of(val(24)).tolist() == [1]                       # first tombstone is reused
    m.set(val(16), val(99))
    assert m.slots_of(val(16)).tolist() == [2] and m.n_elements == 5  # overwrite in place
    v, f = m.get(val(16, 8, 24, 15))
    assert f.tolist() == [True, False, True, True] and v.ravel().tolist() == [99, 0, 15, 14]
    # fill up: 3 free slots (4,5,6); a fourth new key finds no slot
    stored = m.set(val(4, 5, 6, 32), val(1, 2, 3, 4))
    assert stored.tolist() == [1, 1, 1, 0]
    v, f = m.get(val(32))
    assert not f[0]


def test_all_tombstone_table_still_terminates_and_reuses():
    m = RefClosedHashmap(n_buckets=4, rehash_threshold=2.0, constants=consts(1, 1_000_003, 1_000_033))
    k = np.arange(4, dtype=np.int64)[:, None]
    m.set(k, k)
    assert m.remove(k).all() and m.n_elements == 0
    assert (m._uuid == -3).all()
    v, f = m.get(k)
    assert not f.any()
    m.set(k[:2] + 100, k[:2])
    assert m.n_elements == 2 and (m.slots_of(k[:2] + 100) >= 0).all()


def test_uuid_aliases_are_not_confused():
    # prime2 = 2 leaves two possible uuids: the reference would confuse keys, the oracle must not
    m = RefClosedHashmap(n_buckets=64, constants=consts(1, 1_000_003, 2))
    k = np.arange(0, 40, 2, dtype=np.int64)[:, None]          # all even: identical uuid
    m.set(k, k * 3)
    _, h2 = m.hashes_of(k)
    assert len(set(h2.tolist())) == 1
    v, f = m.get(k)
    assert f.all() and np.array_equal(v, k * 3)
    v, f = m.get(k + 100)
    assert not f.any()
    assert m.n_elements == 20


def test_api_edges():
    m = RefClosedHashmap(n_buckets=8)
    with pytest.raises(RuntimeError):
        m.get(np.zeros((1, 1), dtype=np.int64))
    with pytest.raises(RuntimeError):
        m.remove(np.zeros((1, 1), dtype=np.int64))
    m.set(np.zeros((0, 1), dtype=np.int64), np.zeros((0, 1), dtype=np.float32))   # fixes types, stores nothing
    assert m.n_elements == 0
    v, f = m.get(np.zeros((0, 1), dtype=np.int64))
    assert v.shape == (0, 1) and f.shape == (0,)
    assert m.remove(np.zeros((0, 1), dtype=np.int64)).shape == (0,)
    with pytest.raises(AssertionError):
        m.set(np.zeros((1, 1), dtype=np.int32), np.zeros((1, 1), dtype=np.float32))
    # duplicates inside one batch occupy one slot; sequentially the last value wins
    k = np.array([[5], [5], [5]], dtype=np.int64)
    m.set(k, np.array([[1], [2], [3]], dtype=np.float32))
    assert m.n_elements == 1 and m.get(k[:1])[0].ravel().tolist() == [3.0]
    # remove reports over the sorted unique keys
    m.set(np.array([[9], [2]], dtype=np.int64), np.array([[1], [1]], dtype=np.float32))
    mask = m.remove(np.array([[9], [7], [9], [2]], dtype=np.int64))
    assert mask.tolist() == [True, False, True]                # rows: 2, 7, 9
    assert m.n_elements == 1


def test_parallel_drivers_agree_with_serial_on_unique_keys():
    rng = np.random.default_rng(9)
    keys = np.unique(rng.integers(0, 2**62, size=60000, dtype=np.int64))[:50000, None]
    vals = rng.standard_normal((keys.shape[0], 1)).astype(np.float32)
    q = np.concatenate([keys[:20000], rng.integers(0, 2**62, size=(20000, 1), dtype=np.int64)])
    out = []
    for threads in (1, 4):
        m = RefClosedHashmap(n_buckets=131072, rng=np.random.default_rng(1), n_threads=threads)
        m.set(keys, vals)
        out.append(m.get(q))
        assert m.n_elements == keys.shape[0]
    assert np.array_equal(out[0][0], out[1][0]) and np.array_equal(out[0][1], out[1][1])
