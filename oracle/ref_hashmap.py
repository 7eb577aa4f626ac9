"""TEST INFRASTRUCTURE - NOT PRODUCT CODE.

Host-side restatement of the reference's ``CudaClosedHashmap`` policy
(sparse_dok/components/cuda_closed_hashmap.py) on top of the C restatement of its kernels
(``closed_hashmap_ref.c``).  Everything lives in host memory as numpy arrays.

Restated, with the reference lines each method follows:
  __init__            :21-64    table = uuid[B] filled with -1, lazily allocated keys/values
  hash constants      :66-113   prime1 ~ nextprime(U[B,2B)), prime2 ~ nextprime(U[0,2^60)),
                                alpha/beta ~ U[0,prime1) - 1   (alpha2/beta2 also against prime1)
  set                 :321-384  pre-pass get -> count distinct new keys -> rehash when
                                n + n_new > int(threshold*B) to int((n+n_new)*factor) -> set kernel
  get                 :386-421  fallback row pre-fill, hit mask
  remove              :423-454  keys.unique(dim=0) first; mask is over the sorted unique rows
  rehash              :456-468  keys()/values() -> fresh table and constants -> set
  keys/values         :157-172  slots whose uuid is neither -1 nor -3, in slot order

Key identity is the key row's bytes (see the header of closed_hashmap_ref.c for this and the
other documented differences).  Parity pins: tests/test_oracle_hashmap.py.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libref_hashmap.so")
_lib = None

MAX_DIMS = 16


class RefTable(ctypes.Structure):
    _fields_ = [
        ("n_buckets", ctypes.c_int64),
        ("key_size", ctypes.c_int32),
        ("key_elem_bytes", ctypes.c_int32),
        ("key_is_float", ctypes.c_int32),
        ("value_bytes", ctypes.c_int32),
        ("prime1", ctypes.c_void_p), ("prime2", ctypes.c_void_p),
        ("alpha1", ctypes.c_void_p), ("alpha2", ctypes.c_void_p),
        ("beta1", ctypes.c_void_p), ("beta2", ctypes.c_void_p),
        ("uuid", ctypes.c_void_p), ("keys", ctypes.c_void_p), ("values", ctypes.c_void_p),
    ]


class RefAccessor(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("sizes", ctypes.c_int64 * MAX_DIMS),
        ("strides", ctypes.c_int64 * MAX_DIMS),
    ]


def build():
    """Compile the C restatement with the Makefile beside it."""
    import subprocess
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32
        T = ctypes.POINTER(RefTable)
        A = ctypes.POINTER(RefAccessor)
        L.ref_batch_get.restype = i64
        L.ref_batch_get.argtypes = [T, vp, i64, vp, vp, i32]
        L.ref_batch_set.restype = i64
        L.ref_batch_set.argtypes = [T, vp, vp, i64, vp, i32]
        L.ref_batch_remove.restype = i64
        L.ref_batch_remove.argtypes = [T, vp, i64, vp, i32]
        L.ref_batch_find.restype = None
        L.ref_batch_find.argtypes = [T, vp, i64, vp]
        L.ref_batch_hash.restype = None
        L.ref_batch_hash.argtypes = [T, vp, i64, vp, vp]
        L.ref_dok_count_items.restype = i64
        L.ref_dok_count_items.argtypes = [T, A, i32, i32, vp, vp, i64, i32]
        L.ref_dok_set_items_dense.restype = i64
        L.ref_dok_set_items_dense.argtypes = [T, A, A, i32, i32, vp, vp, i64, i32]
        L.ref_dok_get_items_dense.restype = None
        L.ref_dok_get_items_dense.argtypes = [T, A, i32, i32, vp, vp, i64, vp, vp, i32]
        L.ref_dok_zero_items.restype = i64
        L.ref_dok_zero_items.argtypes = [T, A, i32, i32, vp, vp, i64]
        L.ref_dok_get_items.restype = None
        L.ref_dok_get_items.argtypes = [T, T, A, i32, i32, vp, vp, i64]
        L.ref_dok_set_items_sparse_v1.restype = i64
        L.ref_dok_set_items_sparse_v1.argtypes = [T, A, i32, i32, vp, vp, i64, i32]
        L.ref_max_threads.restype = i32
        L.ref_max_threads.argtypes = []
        _lib = L
    return _lib


def next_prime(n):
    """Smallest prime strictly greater than n (what sympy.nextprime returns)."""
    def is_prime(m):
        if m < 2:
            return False
        for p in (2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37):
            if m % p == 0:
                return m == p
        d, r = m - 1, 0
        while d % 2 == 0:
            d, r = d // 2, r + 1
        for a in (2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37):
            x = pow(a, d, m)
            if x in (1, m - 1):
                continue
            for _ in range(r - 1):
                x = x * x % m
                if x == m - 1:
                    break
            else:
                return False
        return True
    m = int(n) + 1
    while not is_prime(m):
        m += 1
    return m


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _rows(a):
    """[N, ...] array -> contiguous [N, row_bytes] uint8 view."""
    a = np.ascontiguousarray(a)
    n = a.shape[0]
    return a.reshape(n, -1).view(np.uint8).reshape(n, -1)


class RefClosedHashmap:
    def __init__(self, n_buckets=1024, rehash_factor=2.0, rehash_threshold=0.75, rng=None,
                 n_threads=1, constants=None):
        self._n_buckets = int(n_buckets)
        self._rehash_factor = rehash_factor
        self._rehash_threshold = rehash_threshold
        self._rng = rng if rng is not None else np.random.default_rng(0)
        self.n_threads = n_threads
        self._uuid = np.full(self._n_buckets, -1, dtype=np.int64)          # :40
        self._keys = None
        self._values = None
        self._n_elements = 0
        self._consts = constants      # optional dict of the six constant vectors
        self._tab = None
        self.probes = 0               # slot probes of get calls, for mean-probe-length reports

    # -- constants (:66-113) --------------------------------------------------------------
    def _draw_constants(self, key_size):
        B = self._n_buckets
        r = self._rng
        prime1 = np.array([next_prime(int(r.integers(B, 2 * B))) for _ in range(key_size)], dtype=np.int64)
        prime2 = np.array([next_prime(int(r.integers(0, 2**60))) for _ in range(key_size)], dtype=np.int64)
        draw = lambda: np.array([int(r.integers(0, int(p))) - 1 for p in prime1], dtype=np.int64)
        return dict(prime1=prime1, prime2=prime2, alpha1=draw(), alpha2=draw(), beta1=draw(), beta2=draw())

    def _table(self):
        if self._tab is None:
            t = RefTable()
            t.n_buckets = self._n_buckets
            t.key_size = self._key_size
            t.key_elem_bytes = self._key_dtype.itemsize
            t.key_is_float = int(self._key_dtype.kind == "f")
            t.value_bytes = self._value_bytes
            for name in ("prime1", "prime2", "alpha1", "alpha2", "beta1", "beta2"):
                setattr(t, name, _ptr(self._consts[name]))
            t.uuid, t.keys, t.values = _ptr(self._uuid), _ptr(self._keys), _ptr(self._values)
            self._tab = t
        return ctypes.byref(self._tab)

    def _allocate(self, keys, values):
        self._key_shape, self._key_dtype = keys.shape[1:], keys.dtype
        self._value_shape, self._value_dtype = values.shape[1:], values.dtype
        self._key_size = int(np.prod(self._key_shape, dtype=np.int64))
        self._key_bytes = self._key_size * keys.dtype.itemsize
        self._value_bytes = int(np.prod(self._value_shape, dtype=np.int64)) * values.dtype.itemsize
        self._keys = np.zeros((self._n_buckets, self._key_bytes), dtype=np.uint8)
        self._values = np.zeros((self._n_buckets, self._value_bytes), dtype=np.uint8)
        if self._consts is None:
            self._consts = self._draw_constants(self._key_size)
        self._tab = None

    # -- properties -----------------------------------------------------------------------
    @property
    def n_elements(self):
        return self._n_elements

    @property
    def n_buckets(self):
        return self._n_buckets

    def __len__(self):
        return self._n_elements

    @property
    def nonempty_mask(self):                                               # :157-159
        return (self._uuid != -1) & (self._uuid != -3)

    def keys(self):                                                        # :161-166
        if self._keys is None:
            return None
        k = self._keys[self.nonempty_mask]
        return k.view(self._key_dtype).reshape(k.shape[0], self._key_size)

    def values(self):                                                      # :168-172
        if self._values is None:
            return None
        v = self._values[self.nonempty_mask]
        return v.view(self._value_dtype).reshape(v.shape[0], *self._value_shape)

    # -- kernels --------------------------------------------------------------------------
    def _kernel_get(self, key_rows, fallback_row=None):
        n = key_rows.shape[0]
        out = np.zeros((n, self._value_bytes), dtype=np.uint8)
        if fallback_row is not None:
            out[:] = fallback_row[None]                                    # closed_hashmap_impl.py:103-109
        found = np.zeros(n, dtype=np.uint8)
        self.probes += lib().ref_batch_get(self._table(), _ptr(key_rows), n, _ptr(out), _ptr(found), self.n_threads)
        return out, found.astype(bool)

    def _kernel_set(self, key_rows, value_rows):
        n = key_rows.shape[0]
        stored = np.zeros(n, dtype=np.uint8)
        lib().ref_batch_set(self._table(), _ptr(key_rows), _ptr(value_rows), n, _ptr(stored), self.n_threads)
        return stored

    # -- API ------------------------------------------------------------------------------
    def set(self, new_keys, new_values):                                   # :321-384
        new_keys, new_values = np.asarray(new_keys), np.asarray(new_values)
        assert new_keys.shape[0] == new_values.shape[0]
        if self._keys is None:
            self._allocate(new_keys, new_values)
        else:
            assert new_keys.dtype == self._key_dtype and new_keys.shape[1:] == self._key_shape
            assert new_values.dtype == self._value_dtype and new_values.shape[1:] == self._value_shape
        if new_keys.shape[0] == 0:
            return
        kr, vr = _rows(new_keys), _rows(new_values)
        _, is_found = self._kernel_get(kr)
        n_new = np.unique(kr[~is_found], axis=0).shape[0]
        if self._n_elements + n_new > int(self._rehash_threshold * self._n_buckets):
            self.rehash(int((self._n_elements + n_new) * self._rehash_factor))
        stored = self._kernel_set(kr, vr)
        self._n_elements += n_new
        return stored

    def get(self, keys, fallback_value=None):                              # :386-421
        if self._keys is None:
            raise RuntimeError("store something first")
        keys = np.asarray(keys)
        if keys.shape[0] == 0:
            return np.zeros((0, *self._value_shape), dtype=self._value_dtype), np.zeros(0, dtype=bool)
        assert keys.dtype == self._key_dtype and keys.shape[1:] == self._key_shape
        fb = None
        if fallback_value is not None:
            fb = np.broadcast_to(np.asarray(fallback_value, dtype=self._value_dtype), self._value_shape)
            fb = np.ascontiguousarray(fb).reshape(-1).view(np.uint8)
        out, found = self._kernel_get(_rows(keys), fb)
        return out.view(self._value_dtype).reshape(keys.shape[0], *self._value_shape), found

    def remove(self, keys):                                                # :423-454
        if self._keys is None:
            raise RuntimeError("store something first")
        keys = np.asarray(keys)
        if keys.shape[0] == 0:
            return np.zeros(0, dtype=bool)
        assert keys.dtype == self._key_dtype and keys.shape[1:] == self._key_shape
        uniq = np.unique(keys.reshape(keys.shape[0], -1), axis=0)          # sorted like torch.unique(dim=0)
        kr = _rows(uniq)
        removed = np.zeros(kr.shape[0], dtype=np.uint8)
        n = lib().ref_batch_remove(self._table(), _ptr(kr), kr.shape[0], _ptr(removed), self.n_threads)
        self._n_elements -= int(n)
        return removed.astype(bool)

    def rehash(self, n_buckets):                                           # :456-468
        keys, values = self.keys(), self.values()
        keys = keys.reshape(keys.shape[0], *self._key_shape)
        self.__init__(n_buckets=n_buckets, rehash_factor=self._rehash_factor,
                      rehash_threshold=self._rehash_threshold, rng=self._rng, n_threads=self.n_threads)
        self.set(keys, values)

    # -- helpers for the placement known-answer tests ---------------------------------------
    def slots_of(self, keys):
        kr = _rows(np.asarray(keys))
        out = np.zeros(kr.shape[0], dtype=np.int64)
        lib().ref_batch_find(self._table(), _ptr(kr), kr.shape[0], _ptr(out))
        return out

    def hashes_of(self, keys):
        kr = _rows(np.asarray(keys))
        h1 = np.zeros(kr.shape[0], dtype=np.int64)
        h2 = np.zeros(kr.shape[0], dtype=np.int64)
        lib().ref_batch_hash(self._table(), _ptr(kr), kr.shape[0], _ptr(h1), _ptr(h2))
        return h1, h2
