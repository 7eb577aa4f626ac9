"""Batched GPU hashmap with the Python surface of the reference's ``CudaClosedHashmap``
(reference: sparse_dok/components/cuda_closed_hashmap.py:20-477), backed by libdokhip.

What differs underneath (and why callers do not see it):

* Storage is one array of 128-byte buckets (see ``csrc/dok_packed8.h`` / ``csrc/dok_tagged.h``)
  instead of the reference's three arrays ``_uuid/_keys/_values``.  ``n_buckets`` keeps the
  reference meaning - the number of key slots asked for - and the physical table has at least
  that many slots.
* Key identity is the key row's bytes, not a 63-bit hash of it, so two keys are never confused.
* ``n_elements`` is maintained by the kernels themselves (fresh inserts are counted where the
  slot is claimed), which replaces the reference's "get, unique, count" pre-pass in ``set``.
  The rehash rule is the reference's: grow to ``int((n + n_new) * rehash_factor)`` when
  ``n + n_new > int(rehash_threshold * n_buckets)``.
* The hash-constant keyword arguments are accepted and kept for ``get_hash`` / ``get_uuid`` /
  ``test_uniformity``; slot placement uses the library's own hash.
* ``coord_dims`` (not in the reference) makes the map coordinate-keyed: key rows are int64
  coordinates inside ``coord_dims``.  They are stored as one linearised 8-byte key where that is
  possible (at most 8 dimensions, fewer than 2^63 elements) and as the coordinate rows themselves,
  on the multi-word layout, otherwise (`coord_rows_needed`).  This is how ``SparseDOKTensor``
  uses the map.
"""
import ctypes
import math

import numpy as np
import torch
from torch import Tensor

from . import _lib
from ._lib import DokTable, DOK_BUCKET_BYTES, DOK_HEADER_WORDS, DOK_MAX_DIMS, DOK_LIN_DIMS


try:
    _raw_stream = torch._C._cuda_getCurrentRawStream       # (2 us less per call than the Stream object)
except AttributeError:                                     # (older torch: the documented way)
    _raw_stream = None


def _stream_ptr(device):
    """The current HIP stream of `device`, as the library's entry points take it."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(device.index or 0))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


# A batch goes through the bulk insert (partition by table range, merge each range in LDS)
# instead of the per-row compare-and-swap kernel when it is large in absolute terms and holds at
# least this many rows per physical bucket.  The bulk path costs about 22 us per million rows
# plus 45 us per million buckets (it streams the whole table once) plus ~0.05 ms of launches;
# the per-row kernel about 66 us per million rows (MI355X, 8-byte keys, 4-byte values; measured
# 1M .. 33M rows: at 2 rows per bucket the bulk path is 1.1x to 1.4x faster, at 5 rows 1.5x to
# 1.9x, at 1.25 rows 0.8x to 0.97x).
# In a table that ends up nearly full the per-row kernel walks longer chains (about 100 us per
# million rows into a table at 85 % with tombstones), so there the bulk path pays from fewer
# rows per bucket on.
BULK_MIN_ROWS = 1 << 20
# The multi-word layout's bulk form (one compare-and-swap per new row, a deferred list, two more
# small launches) pays from a few tens of thousands of rows on.
TAGGED_FAST_MIN_ROWS = 1 << 15
BULK_MIN_ROWS_PER_BUCKET = 2.0
BULK_MIN_ROWS_PER_BUCKET_LOADED = 1.5
BULK_LOADED_FILL = 0.7
# A removal that needs no per-row flags takes the partitioned form from this many keys per physical
# bucket on (and BULK_MIN_ROWS keys): two scatters of the keys, then lookups in table order.
# Measured (MI355X): 32M of the 64M keys of a table of 13.4M buckets (2.4 keys per bucket) 1.10 ms
# against 1.62 ms per row; 20M of the 100M float16 entries of a table of 9.8M buckets at load factor
# 0.85 (2.0 per bucket) 1.20 against 1.15 ms.
BULK_REMOVE_MIN_ROWS_PER_BUCKET = 2.2


def coord_rows_needed(dims):
    """Whether coordinates inside `dims` have to be kept as int64 rows (multi-word keys) because one
    8-byte linear key cannot hold them, or the table has more dimensions than linearised tables take."""
    volume = 1
    for s in dims:
        volume *= max(int(s), 1)
    return len(dims) > DOK_LIN_DIMS or volume >= 2**63


def bulk_pays(n, n_phys, slots_per_bucket, n_upper):
    """Whether a batch of n rows into a table of n_phys buckets should take the bulk path.
    n_upper: upper bound of the slots in use before the batch; it is not lowered by removals,
    so it also counts tombstones - which is what the length of the probe chains depends on."""
    if n < BULK_MIN_ROWS:
        return False
    loaded = n_upper + n >= BULK_LOADED_FILL * n_phys * slots_per_bucket
    per_bucket = min(BULK_MIN_ROWS_PER_BUCKET, BULK_MIN_ROWS_PER_BUCKET_LOADED) if loaded else BULK_MIN_ROWS_PER_BUCKET
    return n >= per_bucket * n_phys


def _next_prime(n):
    """Smallest prime > n (deterministic Miller-Rabin, exact below 3.3e24)."""
    def is_prime(m):
        if m < 2:
            return False
        small = (2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37)
        for p in small:
            if m % p == 0:
                return m == p
        d, r = m - 1, 0
        while d % 2 == 0:
            d //= 2
            r += 1
        for a in small:
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


_SAME_SIZE_INT = {1: torch.int8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def _ordered_bits(t):
    """Floating-point rows as integers of the same width whose order is the order of the values
    and whose equality is equality of the BIT PATTERNS - the identity the table goes by: two NaNs
    of one bit pattern are one key, -0.0 and +0.0 are two (`torch.unique` on the float values has
    it the other way round).  A float's bits, read as a signed integer, already sort like the
    float when the sign is clear; with the sign set the order is reversed, which flipping the
    other bits undoes.  The map is its own inverse.  Integer and bool rows come back unchanged."""
    if not t.dtype.is_floating_point:
        return t
    bits = t.view(_SAME_SIZE_INT[t.element_size()])
    width = 8 * t.element_size()
    return bits ^ ((bits >> (width - 1)) & ((1 << (width - 1)) - 1))


def unique_rows(keys):
    """Distinct rows of `keys` by bit pattern, sorted (row-wise lexicographically) by value: what
    `keys.unique(dim=0)` gives (reference: cuda_closed_hashmap.py:438) wherever the two notions of
    equality agree, i.e. for every batch without NaNs and without both zeros in one column."""
    ordered = _ordered_bits(keys)
    if keys[0].numel() == 1:
        # one element per key: the 1-D sort gives the order of unique(dim=0) far faster
        uniq = ordered.reshape(-1).unique().reshape(-1, *keys.shape[1:])
    else:
        uniq = ordered.unique(dim=0)
    if keys.dtype.is_floating_point:
        uniq = _ordered_bits(uniq.view(keys.dtype)).view(keys.dtype)
    return uniq


def unique_rows_inverse(keys):
    """`unique_rows` together with, for every row of `keys`, the position of its key among the
    distinct rows."""
    n = keys.shape[0]
    ordered = _ordered_bits(keys).reshape(n, -1)
    uniq, inverse = ordered.unique(dim=0, return_inverse=True)
    uniq = uniq.reshape(-1, *keys.shape[1:])
    if keys.dtype.is_floating_point:
        uniq = _ordered_bits(uniq.view(keys.dtype)).view(keys.dtype)
    return uniq, inverse


def _row_fits(keys, values):
    """Whether a table can hold key and value rows of these shapes inside its 128-byte buckets."""
    kb = int(np.prod(keys.shape[1:], dtype=np.int64)) * keys.element_size()
    vb = int(np.prod(values.shape[1:], dtype=np.int64)) * values.element_size()
    return _lib.load().dok_layout_of(kb, vb, ctypes.byref(ctypes.c_int32(0))) >= 0


class _TableState:
    """Physical state of one table.  Shallow clones of a map share one instance, so a rehash or
    an insert through any of them is seen by all."""
    pass


_SHARED = ("_table", "_header", "_desc", "_n_phys", "_slots_per_bucket", "_layout", "_n_buckets",
           "_key_shape", "_key_dtype", "_value_shape", "_value_dtype", "_key_bytes", "_value_bytes",
           "_n_upper", "_n_exact", "_seed", "_pending_clear",
           "_rows", "_rows_used", "_row_shape", "_row_dtype", "_miss_counter", "_miss_seen")


def _forward(name):
    def fget(self):
        return getattr(self._st, name)

    def fset(self, value):
        setattr(self._st, name, value)
    return property(fget, fset)


class CudaClosedHashmap:
    def __init__(
        self,
        n_buckets=1024,
        device="cuda:0",
        prime1=None,
        prime2=None,
        alpha1=None,
        alpha2=None,
        beta1=None,
        beta2=None,
        key_size=None,
        key_perm=None,
        rehash_factor=2.0,
        rehash_threshold=0.75,
        coord_dims=None,
        seed=None,
        coord_rows=None,
    ):
        self._st = _TableState()
        self._empty_marker = -1
        self._removed_marker = -3
        self._n_buckets = int(n_buckets)
        self.device = torch.device(device)
        self._key_size = key_size
        self._prime1, self._prime2 = prime1, prime2
        self._alpha1, self._alpha2 = alpha1, alpha2
        self._beta1, self._beta2 = beta1, beta2
        self._rehash_factor = rehash_factor
        self._rehash_threshold = rehash_threshold
        self._key_perm = None
        if key_perm is not None:
            if not isinstance(key_perm, Tensor):
                key_perm = torch.tensor(key_perm, dtype=torch.long, device=self.device)
            self._key_perm = key_perm.to(device=self.device, dtype=torch.long)
        self._coord_dims = None if coord_dims is None else tuple(int(d) for d in coord_dims)
        if self._coord_dims is not None and len(self._coord_dims) > DOK_MAX_DIMS:
            raise NotImplementedError(f"coordinate tables of more than {DOK_MAX_DIMS} dimensions: a coordinate "
                                      "row no longer fits a 128-byte bucket")
        # key format of a coordinate table: linearised (False) or int64 rows (True); None = rows only
        # where a linear key cannot hold the coordinates
        self._coord_rows = False
        if self._coord_dims is not None:
            need = coord_rows_needed(self._coord_dims)
            assert coord_rows is None or coord_rows or not need, "these coordinates do not fit a linear key"
            self._coord_rows = need or (bool(coord_rows) and len(self._coord_dims) >= 2)
        self._seed = int(seed) if seed is not None else int(np.random.randint(1, 2**62, dtype=np.int64))

        # physical state; the table itself is allocated at the first set(), when the key and
        # value widths are known (the reference allocates _keys/_values there too)
        self._header = torch.zeros(DOK_HEADER_WORDS, device=self.device, dtype=torch.long)
        self._table = None
        self._desc = None
        self._n_phys = 0
        self._slots_per_bucket = 0
        self._layout = 0
        self._key_shape = None
        self._key_dtype = None
        self._value_shape = None
        self._value_dtype = None
        self._key_bytes = 0
        self._value_bytes = 0
        # host-side upper bound of n_elements; lets set() skip the device read-back.  _n_exact: the
        # bound IS the count (read from the table header, nothing enqueued since that could change it)
        self._n_upper = 0
        self._n_exact = True
        # True only inside set()/set_coo(), between the allocation of the table and its first
        # insert: the bucket memory is still uninitialised (a bulk build writes all of it)
        self._pending_clear = False
        # device counter that _update_existing adds to (never reset: the host keeps the last value
        # it read, which saves a fill launch per call)
        self._miss_counter = None
        self._miss_seen = 0
        # value rows kept outside the table (see _OutOfLineValuesMap); unused by this class
        self._rows = None
        self._rows_used = 0
        self._row_shape = None
        self._row_dtype = None

    # ------------------------------------------------------------------ physical table
    for _name in _SHARED:
        locals()[_name] = _forward(_name)
    del _name

    @property
    def _allocated(self):
        return self._table is not None

    def _make_desc(self, table, header, n_phys):
        d = DokTable()
        d.buckets = table.data_ptr()
        d.header = header.data_ptr()
        d.n_phys_buckets = n_phys
        d.seed = self._seed
        d.key_bytes = self._stored_key_bytes()
        d.value_bytes = self._value_bytes
        if self._coord_dims is not None:
            d.lin_ndim = len(self._coord_dims)
            for i, s in enumerate(self._coord_dims):
                d.lin_dims[i] = s
        else:
            d.lin_ndim = 0
        return d

    def _stored_key_bytes(self):
        """Bytes of a key as the table stores it: a coordinate table linearises its rows into 8
        bytes unless the coordinate space is too large for that."""
        if self._coord_dims is not None and not self._coord_rows:
            return 8
        return self._key_bytes

    def _alloc_table(self, n_buckets, clear=True):
        """New table tensors and their descriptor.  clear=False leaves the memory uninitialised:
        only for a caller that clears it (_clear_table) or builds it in bulk right away."""
        lib = _lib.load()
        kb = self._stored_key_bytes()
        slots = ctypes.c_int32(0)
        layout = lib.dok_layout_of(kb, self._value_bytes, ctypes.byref(slots))
        _lib.check(min(layout, 0), "CudaClosedHashmap")
        n_phys = int(lib.dok_phys_buckets_for(max(int(n_buckets), 1), kb, self._value_bytes))
        assert 1 <= n_phys < 2**32, "table too large"
        table = torch.empty(n_phys * DOK_BUCKET_BYTES, device=self.device, dtype=torch.uint8)
        assert table.data_ptr() % DOK_BUCKET_BYTES == 0
        header = torch.empty(DOK_HEADER_WORDS, device=self.device, dtype=torch.long)
        desc = self._make_desc(table, header, n_phys)
        if clear:
            self._clear_table(desc)
        return table, header, desc, n_phys, int(slots.value), int(layout)

    def _clear_table(self, desc):
        _lib.check(_lib.load().dok_table_clear(ctypes.byref(desc), _stream_ptr(self.device)), "clear")

    def _ensure_cleared(self):
        if self._pending_clear:
            self._pending_clear = False
            self._clear_table(self._desc)

    def _init_storage(self, keys, values):
        self._key_shape = tuple(keys.shape[1:])
        self._key_dtype = keys.dtype
        self._value_shape = tuple(values.shape[1:])
        self._value_dtype = values.dtype
        self._key_bytes = int(np.prod(self._key_shape, dtype=np.int64)) * keys.element_size()
        self._value_bytes = int(np.prod(self._value_shape, dtype=np.int64)) * values.element_size()
        if self._coord_dims is not None:
            assert keys.dtype == torch.long and self._key_shape == (len(self._coord_dims),), \
                "a coordinate-keyed map takes int64 key rows of one coordinate per dimension"
        (self._table, self._header, self._desc, self._n_phys,
         self._slots_per_bucket, self._layout) = self._alloc_table(self._n_buckets, clear=False)
        self._pending_clear = True
        self._n_upper = 0

    def _read_header(self):
        h = self._header.cpu()
        n_full = int(h[_lib.DOK_H_NFULL])
        if n_full:
            # reported once, by the first read after the batch that overflowed
            self._header[_lib.DOK_H_NFULL] = 0
            raise RuntimeError(f"hashmap is full: {n_full} rows could not be stored")
        return h

    # ------------------------------------------------------------------ reference-compatible state
    @property
    def _n_elements(self):
        """0-dim int64 device tensor, as in the reference (a view of the table header)."""
        return self._header[_lib.DOK_H_NELEM]

    @property
    def n_elements(self):
        n = int(self._read_header()[_lib.DOK_H_NELEM])
        self._n_upper = n
        self._n_exact = True
        return n

    def _touch(self):
        """Called by whatever enqueues a kernel that may change the number of entries."""
        self._n_exact = False

    def _count_now(self):
        """n_elements, without the device read-back when the host already knows it."""
        return self._n_upper if self._n_exact else self.n_elements

    @property
    def n_buckets(self):
        return self._n_buckets

    @property
    def load_factor(self):
        return self.n_elements / self.n_buckets

    @property
    def key_shape(self):
        assert self._allocated
        return torch.Size(self._key_shape)

    @property
    def value_shape(self):
        assert self._allocated
        return torch.Size(self._value_shape)

    @property
    def key_type(self):
        return self._key_dtype

    @property
    def value_type(self):
        return self._value_dtype

    def __len__(self):
        return self.n_elements

    # raw-table attributes of the reference.  The physical layout is different, so these are
    # materialised on demand from the live entries; None means "nothing stored yet", which is
    # the only thing the reference's own callers test them for.
    @property
    def _keys(self):
        return None if not self._allocated else self.keys().reshape(-1, *self._key_shape)

    @property
    def _values(self):
        return None if not self._allocated else self.values()

    @property
    def _uuid(self):
        if not self._allocated:
            return torch.full((self._n_buckets,), self._empty_marker, device=self.device, dtype=torch.long)
        return self.get_uuid(self.keys().reshape(-1, *self._key_shape))

    def uuid(self):
        return self._uuid

    @property
    def nonempty_mask(self):
        n = 0 if not self._allocated else self.n_elements
        return torch.ones(n, device=self.device, dtype=torch.bool)

    # ------------------------------------------------------------------ hash constants (compat)
    def _flat_key_size(self):
        assert self._allocated or self._key_size is not None
        if self._allocated:
            return int(np.prod(self._key_shape, dtype=np.int64))
        return int(self._key_size)

    def _draw(self, bounds):
        return torch.tensor([int(np.random.randint(int(b))) - 1 for b in bounds], device=self.device)

    @property
    def prime1(self):
        if self._prime1 is None:
            ks = self._flat_key_size()
            draws = [np.random.randint(self.n_buckets, self.n_buckets * 2) for _ in range(ks)]
            self._prime1 = torch.tensor([_next_prime(int(i)) for i in draws], device=self.device)
        return self._prime1

    @property
    def prime2(self):
        if self._prime2 is None:
            ks = self._flat_key_size()
            draws = [np.random.randint(0, 2**60, dtype="int64") for _ in range(ks)]
            self._prime2 = torch.tensor([_next_prime(int(i)) for i in draws], device=self.device)
        return self._prime2

    @property
    def alpha1(self):
        if self._alpha1 is None:
            self._alpha1 = self._draw(self.prime1.cpu())
        return self._alpha1

    @property
    def alpha2(self):
        if self._alpha2 is None:
            self._alpha2 = self._draw(self.prime1.cpu())
        return self._alpha2

    @property
    def beta1(self):
        if self._beta1 is None:
            self._beta1 = self._draw(self.prime1.cpu())
        return self._beta1

    @property
    def beta2(self):
        if self._beta2 is None:
            self._beta2 = self._draw(self.prime1.cpu())
        return self._beta2

    @property
    def key_perm(self):
        if self._key_perm is None:
            assert self._allocated
            self._key_perm = torch.arange(int(np.prod(self._key_shape, dtype=np.int64)), device=self.device)
        else:
            assert self._key_perm.shape[0] == int(np.prod(self._key_shape, dtype=np.int64))
        return self._key_perm

    @key_perm.setter
    def key_perm(self, new):
        if not isinstance(new, Tensor):
            new = torch.tensor(new, device=self.device, dtype=torch.long)
        assert new.shape == self.key_perm.shape
        self._key_perm = new.to(device=self.device, dtype=torch.long)

    def permute_keys(self, ordering):
        """Reorder the elements of every stored key (reference: :179-191).  Keys are hashed as
        whole rows here, so the entries are moved into a fresh table."""
        assert self._allocated, "hashmap is empty"
        assert len(self._key_shape) == 1, "keys are not one dimensional"
        assert len(ordering) == self._key_shape[0]
        assert len(set(ordering)) == len(ordering), "duplicates are not allowed"
        keys, values = self.items()
        ordering = list(ordering)
        if self._coord_dims is not None:
            self._coord_dims = tuple(self._coord_dims[o] for o in ordering)
        for name in ("_prime1", "_prime2", "_alpha1", "_alpha2", "_beta1", "_beta2"):
            if getattr(self, name) is not None:
                setattr(self, name, getattr(self, name)[ordering])
        (self._table, self._header, self._desc, self._n_phys,
         self._slots_per_bucket, self._layout) = self._alloc_table(self._n_buckets)
        self._n_upper = 0
        if keys.shape[0]:
            self._launch_set(self._prep_rows(keys[:, ordering], "keys"), values.contiguous())
            self._n_upper = keys.shape[0]

    @staticmethod
    def _hash_words(keys):
        n = keys.shape[0]
        keys = keys.reshape(n, -1).clone()
        if keys.dtype == torch.float:
            keys = keys.view(dtype=torch.int32).long()
            keys[keys == -2**31] = 0
        elif keys.dtype == torch.half:
            keys = keys.view(dtype=torch.int16).long()
            keys[keys == -2**15] = 0
        elif keys.dtype == torch.double:
            keys = keys.view(dtype=torch.int64)
            keys[keys == -2**63] = 0
        else:
            keys = keys.to(torch.long)
        return keys

    def get_hash(self, keys):
        """The reference's bucket hash of each key row (cuda_closed_hashmap.py:278-300)."""
        w = self._hash_words(keys)
        t = (self.alpha1[None] * w + self.beta1[None]) % self.prime1[None]
        if self._key_perm is not None:
            t = t[:, self._key_perm]
        return t.prod(dim=-1).abs() % self.n_buckets

    def get_uuid(self, keys):
        """The reference's 63-bit identity hash of each key row (cuda_closed_hashmap.py:302-319)."""
        w = self._hash_words(keys)
        return ((self.alpha2[None] * w + self.beta2[None]) % self.prime2[None]).prod(dim=-1).abs()

    def test_uniformity(self, keys):
        codes = self.get_hash(keys)
        logits = (torch.bincount(codes, minlength=self.n_buckets) + 1).log()
        logp = torch.log_softmax(logits, dim=-1)
        return (-(logp * logp.exp()).sum(dim=-1)).exp() / self.n_buckets

    # ------------------------------------------------------------------ batch preparation
    def _prep_rows(self, t, what):
        t = t.contiguous()
        if t.numel() and t.data_ptr() % 8 != 0:
            t = t.clone()
        return t

    def _check_keys(self, keys):
        assert keys.dtype == self._key_dtype, f"keys are {keys.dtype}, the map holds {self._key_dtype}"
        assert keys.device == self.device, f"keys are on {keys.device}, the map is on {self.device}"
        assert tuple(keys.shape[1:]) == self._key_shape, \
            f"key rows have shape {tuple(keys.shape[1:])}, the map holds {self._key_shape}"

    # ------------------------------------------------------------------ set / get / remove
    def _bulk_workspace(self, n):
        """Workspace tensor for a bulk insert of n rows, or None if the batch should take the
        per-row kernel."""
        if self._layout != _lib.DOK_LAYOUT_PACKED8:
            # served for values of one word, and for the first batch of a new table
            if n < TAGGED_FAST_MIN_ROWS or not (self._value_bytes <= 8 or self._pending_clear):
                return None
        elif not bulk_pays(n, self._n_phys, self._slots_per_bucket, self._n_upper):
            return None
        nbytes = int(_lib.load().dok_bulk_workspace_bytes(ctypes.byref(self._desc), n))
        if nbytes <= 0:
            return None
        ws = torch.empty(nbytes, device=self.device, dtype=torch.uint8)
        assert ws.data_ptr() % 256 == 0
        return ws

    def _launch_set(self, keys, values, coo=False):
        """Enqueue one insert of the batch.  coo=True: `keys` is the [ndim, n] coordinate matrix
        of a coordinate-keyed map instead of [n, ...] key rows."""
        lib = _lib.load()
        n = keys.shape[1] if coo else keys.shape[0]
        desc, stream = ctypes.byref(self._desc), _stream_ptr(self.device)
        self._touch()
        ws = self._bulk_workspace(n)
        if ws is not None and self._pending_clear:
            # first insert into a new table: the build writes every bucket, no clear needed
            self._pending_clear = False
            fn = lib.dok_coo_build_bulk if coo else lib.dok_map_build_bulk
            _lib.check(fn(desc, keys.data_ptr(), values.data_ptr(), n, ws.data_ptr(), ws.numel(), stream), "set")
            return
        self._ensure_cleared()
        if ws is not None:
            fn = lib.dok_coo_set_bulk if coo else lib.dok_map_set_bulk
            _lib.check(fn(desc, keys.data_ptr(), values.data_ptr(), n, ws.data_ptr(), ws.numel(), stream), "set")
        elif coo:
            _lib.check(lib.dok_coo_set(desc, keys.data_ptr(), values.data_ptr(), n, stream), "set_coo")
        else:
            _lib.check(lib.dok_map_set(desc, keys.data_ptr(), values.data_ptr(), n, None, stream), "set")

    def _physical_slots(self):
        return self._n_phys * self._slots_per_bucket

    def _growth_limit(self):
        """Entries beyond which `set` grows the table (reference: :365).  A threshold above 1
        switches growth off, as in the reference; rows that then find no slot are not lost
        silently: the `set` that overflowed raises (see _launch_checked)."""
        return int(self._rehash_threshold * self._n_buckets)

    def _launch_checked(self, launch, n):
        """Run an insert of n rows that stays under the growth limit.  If the rows might not fit
        physically (only possible with a threshold above 1), the header is read back right away
        so that an overflow raises in the call that caused it."""
        risky = self._n_upper + n > self._physical_slots()
        launch()
        self._n_upper += n
        if risky:
            self.n_elements

    def set(self, new_keys, new_values):
        """Upsert a batch (reference: cuda_closed_hashmap.py:321-384).  Returns None."""
        assert new_keys.shape[0] == new_values.shape[0], \
            f"{new_keys.shape[0]} key rows but {new_values.shape[0]} value rows"
        if not self._allocated:
            assert new_keys.device == new_values.device == self.device, \
                f"keys on {new_keys.device}, values on {new_values.device}, the map is on {self.device}"
            if type(self) is CudaClosedHashmap and self._coord_dims is None and not _row_fits(new_keys, new_values):
                # key + value rows wider than a bucket: the values move to a side array
                self.__class__ = _OutOfLineValuesMap
                return self.set(new_keys, new_values)
            self._init_storage(new_keys, new_values)
        else:
            self._check_keys(new_keys)
            assert new_values.dtype == self._value_dtype, \
                f"values are {new_values.dtype}, the map holds {self._value_dtype}"
            assert new_values.device == self.device, f"values are on {new_values.device}, the map is on {self.device}"
            assert tuple(new_values.shape[1:]) == self._value_shape, \
                f"value rows have shape {tuple(new_values.shape[1:])}, the map holds {self._value_shape}"
        n = new_keys.shape[0]
        try:
            if n:
                self._set_rows(self._prep_rows(new_keys, "keys"), self._prep_rows(new_values, "values"))
        finally:
            self._ensure_cleared()      # a new table never leaves this call uninitialised

    def _set_rows(self, keys, values):
        n = keys.shape[0]
        limit = self._growth_limit()
        if self._n_upper + n <= limit:
            # cannot cross the threshold whatever the batch holds: no read-back, no sync
            self._launch_checked(lambda: self._launch_set(keys, values), n)
            return
        self._ensure_cleared()
        n_old = self._count_now()
        if n_old + n <= limit:
            self._launch_checked(lambda: self._launch_set(keys, values), n)
            return
        if n_old + n <= int(0.9 * self._physical_slots()):
            # the batch fits physically: insert, then apply the reference's growth rule to the
            # count the kernel produced (same final size and contents as growing first)
            self._launch_set(keys, values)
            n_now = self.n_elements
            if n_now > limit:
                self.rehash(int(n_now * self._rehash_factor))
            return
        # the batch may not fit.  Rows that miss bound the distinct new keys from above; if even
        # that bound stays under the threshold nothing can grow and no sort is needed
        # (counted by a kernel that writes one number: no value rows, no flags).  On the packed
        # layout the counting kernel also overwrites the values of the keys it finds, so a batch
        # that only updates present keys - the usual case in a table this full - is done with it
        n_miss = self._update_existing(keys, values)
        if n_miss == 0:
            return                            # every key was present and holds its new value
        if n_miss < 0:
            n_miss = n - int(self.count_existing(keys).item())
        if n_old + n_miss <= limit:
            self._launch_checked(lambda: self._launch_set(keys, values), n_miss)
            if n_miss == 0:
                self._n_exact = True          # every key was present: the batch only overwrites values
            return
        # otherwise count the distinct new keys exactly, as the reference does
        _, is_found = self.get(keys)
        n_new = self._count_distinct(keys[~is_found])
        if n_old + n_new > limit:
            self.rehash(int((n_old + n_new) * self._rehash_factor))
        self._launch_checked(lambda: self._launch_set(keys, values), n_new)

    def set_coo(self, indices, values):
        """`set` for a coordinate-keyed map with the coordinates laid out as a COO tensor holds
        them: ``indices`` is [ndim, n] int64, ``values`` [n, *value_shape].  Saves the transpose
        copy that `set(indices.T, ...)` needs (reference: sparse_dok_tensor.py:66-69)."""
        assert self._coord_dims is not None, "set_coo needs a coordinate-keyed map"
        assert indices.dim() == 2 and indices.shape[0] == len(self._coord_dims)
        assert indices.shape[1] == values.shape[0]
        if not self._allocated:
            assert indices.device == values.device == self.device and indices.dtype == torch.long
            self._init_storage(indices[:, :0].T, values)
        else:
            assert indices.dtype == torch.long and indices.device == self.device
            assert values.dtype == self._value_dtype and values.device == self.device
            assert tuple(values.shape[1:]) == self._value_shape
        n = indices.shape[1]
        try:
            if n:
                self._set_coo_rows(indices, values)
        finally:
            self._ensure_cleared()      # a new table never leaves this call uninitialised

    def _set_coo_rows(self, indices, values):
        n = indices.shape[1]
        indices = self._prep_rows(indices, "indices")
        values = self._prep_rows(values, "values")

        def launch():
            self._launch_set(indices, values, coo=True)

        limit = self._growth_limit()
        if self._n_upper + n <= limit:
            self._launch_checked(launch, n)
            return
        self._ensure_cleared()
        n_old = self._count_now()
        if n_old + n <= limit:
            self._launch_checked(launch, n)
        elif n_old + n <= int(0.9 * self._physical_slots()):
            launch()
            n_now = self.n_elements
            if n_now > limit:
                self.rehash(int(n_now * self._rehash_factor))
        else:
            self.set(indices.T, values)       # the exact-count path works on key rows

    def items_coo(self):
        """(indices [ndim, n], values [n, *value_shape]) of a coordinate-keyed map, from one pass,
        in slot order (reference: SparseDOKTensor.indices()/values(), sparse_dok_tensor.py:156-169)."""
        assert self._coord_dims is not None
        if not self._allocated:
            return None, None
        lib = _lib.load()
        scratch = torch.empty(int(lib.dok_compact_scratch_bytes(ctypes.byref(self._desc))) // 8,
                              device=self.device, dtype=torch.long)
        count = torch.zeros(1, device=self.device, dtype=torch.long)
        n = self.n_elements
        indices = torch.empty(len(self._coord_dims), n, device=self.device, dtype=torch.long)
        values = torch.empty(n, *self._value_shape, device=self.device, dtype=self._value_dtype)
        if n:
            _lib.check(lib.dok_coo_compact(ctypes.byref(self._desc), indices.data_ptr(), values.data_ptr(), n,
                                           count.data_ptr(), scratch.data_ptr(), _stream_ptr(self.device)),
                       "items_coo")
        return indices, values

    def _count_distinct(self, keys):
        """Number of distinct rows of `keys` (the reference's `unique(dim=0).shape[0]`,
        cuda_closed_hashmap.py:363).  For the packed layout the rows are inserted into a scratch
        table of one-byte values and its entry count is read back - two kernels instead of a
        sort of the whole batch."""
        n = keys.shape[0]
        if n == 0:
            return 0
        if self._layout != _lib.DOK_LAYOUT_PACKED8:
            if self._coord_dims is not None:
                # rows outside the coordinate space are skipped by the insert
                dims = torch.tensor(self._coord_dims, device=keys.device, dtype=torch.long)
                keys = keys[((keys >= 0) & (keys < dims)).all(dim=1)]
                if keys.shape[0] == 0:
                    return 0
            return int(unique_rows(keys).shape[0])        # distinct by bit pattern, as the table sees them
        lib = _lib.load()
        kb = self._stored_key_bytes()
        n_phys = int(lib.dok_phys_buckets_for(2 * n, kb, 1))
        table = torch.empty(n_phys * DOK_BUCKET_BYTES, device=self.device, dtype=torch.uint8)
        header = torch.empty(DOK_HEADER_WORDS, device=self.device, dtype=torch.long)
        desc = self._make_desc(table, header, n_phys)
        desc.value_bytes = 1
        stream = _stream_ptr(self.device)
        ones = torch.zeros(n, device=self.device, dtype=torch.uint8)
        keys = self._prep_rows(keys, "keys")
        _lib.check(lib.dok_table_clear(ctypes.byref(desc), stream), "clear")
        _lib.check(lib.dok_map_set(ctypes.byref(desc), keys.data_ptr(), ones.data_ptr(), n, None, stream), "set")
        h = header.cpu()
        # out-of-range coordinate rows are skipped by the real insert as well
        return int(h[_lib.DOK_H_NELEM])

    def get(self, keys, fallback_value=None):
        """(values, is_found) for a batch of keys (reference: cuda_closed_hashmap.py:386-421)."""
        if not self._allocated:
            raise RuntimeError("store something first")
        if keys.shape[0] == 0:
            return (torch.empty(0, *self._value_shape, device=self.device, dtype=self._value_dtype),
                    torch.empty(0, device=self.device, dtype=torch.bool))
        self._check_keys(keys)
        # The fallback row.  A tensor on the map's device stays there and is read by the kernel: no
        # copy to the host, no synchronisation, and the call can be captured into a HIP graph and
        # see the row's contents at replay time (the reference passes a device array too,
        # closed_hashmap_impl.py:103-109).  Anything else becomes a few bytes passed by value.
        fb = fb_dev = None
        if isinstance(fallback_value, Tensor) and fallback_value.device == self.device:
            assert fallback_value.dtype == self._value_dtype
            fb_dev = torch.broadcast_to(fallback_value, self._value_shape).contiguous()
        elif fallback_value is not None:
            if not isinstance(fallback_value, Tensor):
                fallback_value = torch.tensor(fallback_value, dtype=self._value_dtype)
            assert fallback_value.dtype == self._value_dtype
            row = torch.empty(self._value_shape, dtype=self._value_dtype)
            row.copy_(torch.broadcast_to(fallback_value.cpu(), self._value_shape))
            fb = row.reshape(-1).view(torch.uint8).numpy().tobytes()
        keys = self._prep_rows(keys, "keys")
        n = keys.shape[0]
        values = torch.empty(n, *self._value_shape, device=self.device, dtype=self._value_dtype)
        is_found = torch.empty(n, device=self.device, dtype=torch.bool)
        lib = _lib.load()
        if fb_dev is not None:
            _lib.check(lib.dok_map_get_dev_fallback(ctypes.byref(self._desc), keys.data_ptr(), n, values.data_ptr(),
                                                    fb_dev.data_ptr(), is_found.data_ptr(),
                                                    _stream_ptr(self.device)), "get")
        else:
            _lib.check(lib.dok_map_get(ctypes.byref(self._desc), keys.data_ptr(), n, values.data_ptr(),
                                       fb, is_found.data_ptr(), _stream_ptr(self.device)), "get")
        return values, is_found

    def remove(self, keys):
        """Remove a batch of keys; returns the mask over the distinct rows of ``keys`` in sorted
        order - ``keys.unique(dim=0)``, except that rows are told apart by bit pattern like the
        table does (see `unique_rows`; reference: cuda_closed_hashmap.py:423-454)."""
        if not self._allocated:
            raise RuntimeError("store something first")
        if keys.shape[0] == 0:
            return torch.zeros(0, device=keys.device, dtype=torch.bool)
        self._check_keys(keys)
        return self._remove_rows(self._prep_rows(unique_rows(keys), "keys"), unique=True)

    def _remove_rows_no_mask(self, keys):
        """Remove a batch whose per-row outcome nobody asks for (`del map[keys]`): large batches go
        through the partitioned removal, the rest through the per-row kernel."""
        n = keys.shape[0]
        if (self._layout == _lib.DOK_LAYOUT_PACKED8 and n >= BULK_MIN_ROWS
                and n >= BULK_REMOVE_MIN_ROWS_PER_BUCKET * self._n_phys):
            lib = _lib.load()
            nbytes = int(lib.dok_bulk_workspace_bytes(ctypes.byref(self._desc), n))
            if nbytes > 0:
                ws = torch.empty(nbytes, device=self.device, dtype=torch.uint8)
                self._touch()
                _lib.check(lib.dok_map_remove_bulk(ctypes.byref(self._desc), keys.data_ptr(), n, ws.data_ptr(),
                                                   ws.numel(), _stream_ptr(self.device)), "remove")
                return
        self._remove_rows(keys)

    def _remove_rows(self, keys, unique=False):
        """Remove without the sort: mask aligned with ``keys`` (equal rows: one reports True).
        unique=True: the caller vouches that no row occurs twice (no atomic per row is needed then)."""
        n = keys.shape[0]
        is_removed = torch.empty(n, device=self.device, dtype=torch.bool)
        lib = _lib.load()
        self._touch()
        fn = lib.dok_map_remove_unique if unique else lib.dok_map_remove
        _lib.check(fn(ctypes.byref(self._desc), keys.data_ptr(), n,
                      is_removed.data_ptr(), _stream_ptr(self.device)), "remove")
        return is_removed

    def _update_existing(self, keys, values):
        """Overwrite the values of the rows of an upsert batch whose keys are present; returns the
        number of rows whose key is absent (nothing is inserted), or -1 where the layout has no
        such kernel.  The entry count cannot change."""
        if self._layout != _lib.DOK_LAYOUT_PACKED8:
            return -1
        if self._miss_counter is None:
            self._miss_counter = torch.zeros((), device=self.device, dtype=torch.long)
            self._miss_seen = 0
        _lib.check(_lib.load().dok_map_update_existing(ctypes.byref(self._desc), keys.data_ptr(), values.data_ptr(),
                                                       keys.shape[0], self._miss_counter.data_ptr(),
                                                       _stream_ptr(self.device)), "set")
        total = int(self._miss_counter.item())
        n_miss, self._miss_seen = total - self._miss_seen, total
        return n_miss

    def count_existing(self, keys):
        """How many rows of ``keys`` are present (device int64 scalar)."""
        if not self._allocated:
            raise RuntimeError("store something first")
        self._check_keys(keys)
        keys = self._prep_rows(keys, "keys")
        count = torch.zeros((), device=self.device, dtype=torch.long)
        lib = _lib.load()
        _lib.check(lib.dok_map_count_existing(ctypes.byref(self._desc), keys.data_ptr(), keys.shape[0],
                                              count.data_ptr(), _stream_ptr(self.device)), "count")
        return count

    # ------------------------------------------------------------------ read-out
    def _compact(self, want_keys, want_values):
        lib = _lib.load()
        scratch_bytes = int(lib.dok_compact_scratch_bytes(ctypes.byref(self._desc)))
        scratch = torch.empty(scratch_bytes // 8, device=self.device, dtype=torch.long)
        count = torch.zeros(1, device=self.device, dtype=torch.long)
        stream = _stream_ptr(self.device)
        # the header already holds the number of live entries: size the outputs from it
        n = self.n_elements
        keys = values = None
        if want_keys:
            keys = torch.empty(n, *self._key_shape, device=self.device, dtype=self._key_dtype)
        if want_values:
            values = torch.empty(n, *self._value_shape, device=self.device, dtype=self._value_dtype)
        if n:
            _lib.check(lib.dok_map_compact(
                ctypes.byref(self._desc),
                keys.data_ptr() if keys is not None else None,
                values.data_ptr() if values is not None else None,
                n, count.data_ptr(), scratch.data_ptr(), stream), "compact")
        return keys, values

    def keys(self):
        """Live key rows, [n, prod(key_shape)], in slot order (reference: :161-166)."""
        if not self._allocated:
            return None
        keys, _ = self._compact(True, False)
        return keys.reshape(keys.shape[0], self._flat_key_size())

    def values(self):
        """Live value rows in the same order as ``keys()`` (reference: :168-172)."""
        if not self._allocated:
            return None
        _, values = self._compact(False, True)
        return values

    def items(self):
        """(keys, values) from one pass."""
        if not self._allocated:
            return None, None
        keys, values = self._compact(True, True)
        return keys.reshape(keys.shape[0], self._flat_key_size()), values

    def set_values(self, selectors, new_values):
        """Overwrite values of live entries picked by position in ``values()`` order (:174-177)."""
        keys, values = self.items()
        values[selectors] = new_values
        self._launch_set(self._prep_rows(keys.reshape(-1, *self._key_shape), "keys"), values.contiguous())

    # ------------------------------------------------------------------ rehash / clone
    def rehash(self, n_buckets):
        """Move every entry into a fresh table of ``n_buckets`` slots (reference: :456-468)."""
        n_buckets = int(n_buckets)
        if not self._allocated:
            self._n_buckets = n_buckets
            return
        if n_buckets < self._n_upper:
            n_now = self.n_elements
            if n_buckets < n_now:
                raise ValueError(f"rehash({n_buckets}): the map holds {n_now} entries")
        lib = _lib.load()
        old = (self._table, self._header, self._desc)
        self._seed = int(np.random.randint(1, 2**62, dtype=np.int64))
        table, header, desc, n_phys, slots, layout = self._alloc_table(n_buckets, clear=False)
        if layout == _lib.DOK_LAYOUT_PACKED8:
            ws = None
            if self._n_upper >= (1 << 23) and self._n_upper >= 2.5 * n_phys:
                # (the upper bound is only a hint for picking the path; both give the same table)
                nbytes = int(lib.dok_rehash_bulk_workspace_bytes(ctypes.byref(old[2]), ctypes.byref(desc)))
                if nbytes > 0:
                    ws = torch.empty(nbytes, device=self.device, dtype=torch.uint8)
            if ws is not None:
                # writes every bucket of the new table: no clear
                _lib.check(lib.dok_map_rehash_bulk(ctypes.byref(old[2]), ctypes.byref(desc), ws.data_ptr(),
                                                   ws.numel(), _stream_ptr(self.device)), "rehash")
            else:
                self._clear_table(desc)
                _lib.check(lib.dok_map_rehash(ctypes.byref(old[2]), ctypes.byref(desc),
                                              _stream_ptr(self.device)), "rehash")
        else:
            self._clear_table(desc)
            _lib.check(lib.dok_map_rehash(ctypes.byref(old[2]), ctypes.byref(desc),
                                          _stream_ptr(self.device)), "rehash")
        self._table, self._header, self._desc, self._n_phys = table, header, desc, n_phys
        self._n_buckets = n_buckets
        # the old table tensors stay referenced by `old` until the copies above are enqueued;
        # torch's allocator orders their reuse on the same stream
        del old

    def clone(self, deepclone=False):
        """Shallow clone shares the table; deep clone copies it (reference: :193-231)."""
        new = CudaClosedHashmap(
            n_buckets=self._n_buckets, device=self.device,
            prime1=self._prime1, prime2=self._prime2, alpha1=self._alpha1, alpha2=self._alpha2,
            beta1=self._beta1, beta2=self._beta2, key_perm=self._key_perm,
            rehash_factor=self._rehash_factor, rehash_threshold=self._rehash_threshold,
            coord_dims=self._coord_dims, seed=self._seed, coord_rows=self._coord_rows or None,
        )
        new.__class__ = self.__class__
        if not deepclone:
            new._st = self._st
            return new
        for name in _SHARED:
            setattr(new, name, getattr(self, name))
        if self._rows is not None:
            new._rows = self._rows.clone()
        new._miss_counter, new._miss_seen = None, 0
        if self._allocated:
            new._table = self._table.clone()
            new._header = self._header.clone()
            new._desc = new._make_desc(new._table, new._header, new._n_phys)
        else:
            new._header = self._header.clone()
        return new

    # ------------------------------------------------------------------ probe statistics
    def probe_stats(self, keys):
        """Mean number of buckets a lookup of each of ``keys`` visits."""
        self._check_keys(keys)
        keys = self._prep_rows(keys, "keys")
        n = keys.shape[0]
        values = torch.empty(n, *self._value_shape, device=self.device, dtype=self._value_dtype)
        is_found = torch.empty(n, device=self.device, dtype=torch.bool)
        before = self._header.cpu()
        lib = _lib.load()
        _lib.check(lib.dok_map_get_stats(ctypes.byref(self._desc), keys.data_ptr(), n, values.data_ptr(),
                                         None, is_found.data_ptr(), _stream_ptr(self.device)), "get_stats")
        after = self._header.cpu()
        probes = int(after[_lib.DOK_H_NPROBE] - before[_lib.DOK_H_NPROBE])
        ops = int(after[_lib.DOK_H_NOPS] - before[_lib.DOK_H_NOPS])
        return probes / max(ops, 1)

    def __getitem__(self, keys):
        return self.get(keys)

    def __setitem__(self, keys, values):
        return self.set(keys, values)

    def __delitem__(self, keys):
        # `del hm[keys]` discards the mask, so the sort that only orders the mask is skipped
        if not self._allocated:
            raise RuntimeError("store something first")
        if keys.shape[0] == 0:
            return
        self._check_keys(keys)
        self._remove_rows_no_mask(self._prep_rows(keys, "keys"))


class _OutOfLineValuesMap(CudaClosedHashmap):
    """The map for rows that do not fit a 128-byte bucket (8 * (1 + ceil(K/8) + ceil(V/8)) > 128):
    the table maps each key to the int64 number of a row of a side array `_rows`
    [capacity, *value_shape], and the value rows live there.  A CudaClosedHashmap turns into this
    class in its first `set`, when the widths are known; everything that deals with keys only
    (remove, keys, rehash, the growth rule, the counts) is the base class working on the
    key -> row-number table.  The reference compiles its kernels for any KeySize / ValueSize
    (closed_hashmap_impl_class.cu:7); this keeps every value width usable.  Keys wider than 112
    bytes still do not fit (a slot needs the tag word, the key words and the row number).
    Rows of removed keys stay allocated until the side array is compacted, which `set` does when it
    is full and more than half of it is garbage.  This path is composed from the batched kernels
    and torch indexing; it is not tuned."""

    @property
    def value_shape(self):
        assert self._allocated
        return torch.Size(self._row_shape)

    @property
    def value_type(self):
        return self._row_dtype

    def _reserve_rows(self, n_new):
        """Room for n_new more value rows.  True if the rows of the present keys were renumbered."""
        need = self._rows_used + n_new
        if need <= self._rows.shape[0]:
            return False
        if self._rows_used > 2 * self.n_elements:
            # more than half of the rows belong to removed keys: renumber the live ones 0 .. n-1
            keys, numbers = CudaClosedHashmap.items(self)
            n = keys.shape[0]
            live = self._rows[numbers.reshape(-1)]
            self._rows = torch.empty(max(2 * (n + n_new), 16), *self._row_shape, device=self.device, dtype=self._row_dtype)
            self._rows[:n] = live
            self._rows_used = n
            if n:
                CudaClosedHashmap.set(self, keys.reshape(n, *self._key_shape),
                                      torch.arange(n, device=self.device)[:, None])
            return True
        grown = torch.empty(max(need, 2 * self._rows.shape[0]), *self._row_shape, device=self.device, dtype=self._row_dtype)
        grown[: self._rows_used] = self._rows[: self._rows_used]
        self._rows = grown
        return False

    def set(self, new_keys, new_values):
        assert new_keys.shape[0] == new_values.shape[0], \
            f"{new_keys.shape[0]} key rows but {new_values.shape[0]} value rows"
        if self._rows is None:
            assert new_keys.device == new_values.device == self.device, \
                f"keys on {new_keys.device}, values on {new_values.device}, the map is on {self.device}"
            self._row_shape = tuple(new_values.shape[1:])
            self._row_dtype = new_values.dtype
            row_bytes = max(int(np.prod(self._row_shape, dtype=np.int64)) * new_values.element_size(), 1)
            self._rows = torch.empty(max(16, min(1024, (1 << 24) // row_bytes)), *self._row_shape,
                                     device=self.device, dtype=self._row_dtype)
            self._rows_used = 0
            if new_keys.shape[0] == 0:
                # (the table is allocated by the first set even if the batch is empty, as in the reference)
                CudaClosedHashmap.set(self, new_keys, torch.empty(0, 1, device=self.device, dtype=torch.long))
        else:
            assert new_values.dtype == self._row_dtype, f"values are {new_values.dtype}, the map holds {self._row_dtype}"
            assert new_values.device == self.device, f"values are on {new_values.device}, the map is on {self.device}"
            assert tuple(new_values.shape[1:]) == self._row_shape, \
                f"value rows have shape {tuple(new_values.shape[1:])}, the map holds {self._row_shape}"
        n = new_keys.shape[0]
        if n == 0:
            return
        if self._allocated:
            self._check_keys(new_keys)
        # one row per distinct key of the batch (equal keys: one of their rows wins, whole)
        keys, inverse = unique_rows_inverse(new_keys)
        m = keys.shape[0]
        winner = torch.empty(m, device=self.device, dtype=torch.long)
        winner.scatter_(0, inverse, torch.arange(n, device=self.device))
        if self._allocated:
            numbers, found = CudaClosedHashmap.get(self, keys)
            numbers = numbers.reshape(-1)
            missing = ~found
            n_new = m - int(found.sum().item())
        else:
            numbers = torch.empty(m, device=self.device, dtype=torch.long)
            missing = torch.ones(m, device=self.device, dtype=torch.bool)
            n_new = m
        if n_new:
            if self._reserve_rows(n_new) and n_new < m:
                numbers = CudaClosedHashmap.get(self, keys)[0].reshape(-1)
            fresh = torch.arange(self._rows_used, self._rows_used + n_new, device=self.device)
            numbers = numbers.masked_scatter(missing, fresh)
            self._rows_used += n_new
            CudaClosedHashmap.set(self, keys[missing], fresh[:, None])
        self._rows.index_copy_(0, numbers, new_values[winner])

    def get(self, keys, fallback_value=None):
        if not self._allocated:
            raise RuntimeError("store something first")
        if keys.shape[0] == 0:
            return (torch.empty(0, *self._row_shape, device=self.device, dtype=self._row_dtype),
                    torch.empty(0, device=self.device, dtype=torch.bool))
        numbers, found = CudaClosedHashmap.get(self, keys)            # (row 0 for absent keys)
        values = self._rows[numbers.reshape(-1)]
        if fallback_value is None:
            fallback = torch.zeros((), device=self.device, dtype=self._row_dtype)
        elif isinstance(fallback_value, Tensor):
            assert fallback_value.dtype == self._row_dtype
            fallback = fallback_value.to(self.device)
        else:
            fallback = torch.tensor(fallback_value, dtype=self._row_dtype, device=self.device)
        fallback = torch.broadcast_to(fallback, self._row_shape)
        values = torch.where(found.reshape(-1, *([1] * len(self._row_shape))), values, fallback)
        return values, found

    def values(self):
        if not self._allocated:
            return None
        _, numbers = self._compact(False, True)
        return self._rows[numbers.reshape(-1)]

    def items(self):
        if not self._allocated:
            return None, None
        keys, numbers = CudaClosedHashmap.items(self)
        return keys, self._rows[numbers.reshape(-1)]

    def set_values(self, selectors, new_values):
        keys, values = self.items()
        values[selectors] = new_values
        self.set(keys.reshape(-1, *self._key_shape), values)
