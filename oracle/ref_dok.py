"""TEST INFRASTRUCTURE - NOT PRODUCT CODE.

CPU restatement of the reference's ``SparseDOKTensor`` hot path
(sparse_dok/components/sparse_dok_tensor.py) on top of ``RefClosedHashmap``: everything is
host memory (torch CPU tensors for the selector algebra, numpy for the table).

Restated, with the reference lines each method follows:
  __init__             :18-69     empty map of 32 buckets, or next_power_of_2(nnz) buckets and one
                                   set of (indices.T, values[:, None])
  _handle_selectors    :220-300   selector normalisation, broadcast, axis placement
  __getitem__          :302-315   stack -> [ndim, N] -> transpose -> get(fallback 0) -> view ->
                                   squeeze_ of every scalar selector position (which raises
                                   IndexError when that position is not an axis of the result,
                                   exactly as the reference does)
  __setitem__ (dense)  :317-327   broadcast the values, then set_items_dense
  set_items_dense      sparse_dok_tensor_impl.py:412-474: bootstrap insert when unallocated,
                                   count existing, rehash when n + n_sel > B*threshold to
                                   ceil((n + n_sel)*factor), scatter, n += n_sel - n_existing
  __spgetitem__        :342-350 + get_items (sparse_dok_tensor_impl.py:148-233): count the hits,
                                   new map of int(2n) buckets keyed by selector-space index, insert
                                   every hit
  __setitem__ (sparse) :321-323 + set_items_sparse (sparse_dok_tensor_impl.py:235-340): remove every
                                   addressed element, rehash to ceil((n + n_src)*factor*2), store the
                                   source's nonzero entries through the selectors, n += n_src
  indices/values/to_dense :156-209

Deliberate differences: numpy selectors are converted with torch.from_numpy (the reference's
call has an invalid signature, :235,239); a bare int selector is accepted.
Parity pins: tests/test_oracle_dok.py (dense torch/numpy indexing wherever the reference's axis
rule coincides with numpy's, hand-derived shapes where it does not).
"""
import ctypes

import numpy as np
import torch
from torch import Tensor

from .ref_hashmap import RefAccessor, RefClosedHashmap, lib, _ptr


def next_power_of_2(n):                       # util.py:125-137
    if n and not (n & (n - 1)):
        return n
    count = 0
    while n != 0:
        n >>= 1
        count += 1
    return 1 << count


def shape_to_stride(shape):                   # util.py:289-293
    if len(shape) > 0:
        return tuple(np.flip(np.cumprod(shape[1::][::-1])).tolist()) + (1,)
    return tuple()


def _accessor(t):
    a = RefAccessor()
    a.data = t.data_ptr()
    for j in range(t.dim()):
        a.sizes[j] = t.shape[j]
        a.strides[j] = t.stride(j)
    return a


class RefSparseDOKTensor:
    def __init__(self, size, indices=None, values=None, dtype=None, rng=None):
        self._size = torch.Size(size)
        self._rng = rng if rng is not None else np.random.default_rng(0)
        if dtype is None:
            self._dtype = torch.float32 if values is None else values.dtype
        else:
            self._dtype = dtype
        if indices is None:
            self._hashmap = RefClosedHashmap(n_buckets=32, rng=self._rng)                 # :45-48
        else:
            assert indices.shape[0] == self.ndim and indices.shape[1] == values.shape[0]
            self._hashmap = RefClosedHashmap(n_buckets=next_power_of_2(values.shape[0]), rng=self._rng)  # :59-62
            self._hashmap.set(indices.T.contiguous().numpy(),
                              values.to(self._dtype)[:, None].contiguous().numpy())         # :66-69

    @property
    def shape(self):
        return self._size

    @property
    def ndim(self):
        return len(self._size)

    @property
    def dtype(self):
        return self._dtype

    def _nnz(self):
        return self._hashmap.n_elements

    def indices(self):                                                                      # :156-162
        k = self._hashmap.keys()
        if k is None:
            return torch.empty(self.ndim, 0, dtype=torch.long)
        return torch.from_numpy(np.ascontiguousarray(k)).T

    def values(self):                                                                       # :164-169
        v = self._hashmap.values()
        if v is None:
            return torch.empty(0, dtype=self._dtype)
        return torch.from_numpy(np.ascontiguousarray(v)).flatten()

    def to_dense(self):                                                                     # :195-209
        return torch.sparse_coo_tensor(self.indices(), self.values(), size=tuple(self.shape)).to_dense()

    # ---- selectors (:220-300) -----------------------------------------------------------
    def _handle_selectors(self, selectors):
        if isinstance(selectors, (Tensor, slice, np.ndarray, list, int)):
            selectors = (selectors,)
        sel = []
        for s in selectors:
            if isinstance(s, np.ndarray):
                s = torch.from_numpy(s)
            if isinstance(s, Tensor) and s.dtype == torch.bool:
                sel += list(s.nonzero(as_tuple=True))                                       # :226-228
            elif isinstance(s, Tensor) and s.dtype in (torch.int64, torch.int32, torch.int16):
                sel.append(s.long())                                                        # :230-232
            elif isinstance(s, int):
                sel.append(torch.tensor(s, dtype=torch.long))                               # :242-243
            elif isinstance(s, slice):
                sel.append(s)
            elif isinstance(s, (tuple, list)):
                sel.append(torch.tensor(s, dtype=torch.long))                               # :248-250
            else:
                raise ValueError
        sel = sel + [slice(None)] * (self.ndim - len(sel))                                  # :255
        scalar_idx = [i for i in range(len(sel)) if isinstance(sel[i], Tensor) and sel[i].ndim == 0]

        slices = [s for s in sel if isinstance(s, slice)]
        if len(sel) != len(slices):
            bshape = torch.broadcast_shapes(*[s.shape for s in sel if isinstance(s, Tensor)])
        else:
            bshape = tuple()
        sel_ndim = len(bshape) + len(slices)
        for i in range(len(sel)):
            if isinstance(sel[i], Tensor):
                sel[i] = torch.broadcast_to(sel[i], bshape)
        first = None
        for i, s in enumerate(sel):
            if isinstance(s, Tensor):
                first = i
                break

        idx = 0
        met = False
        for i in range(len(sel)):
            if isinstance(sel[i], Tensor):
                newaxis = [None] * sel_ndim
                for j in range(first, first + len(bshape)):
                    newaxis[j] = slice(None)
                sel[i] = sel[i][tuple(newaxis)]
                if not met:
                    idx += len(bshape)
                    met = True
            else:
                start, stop = sel[i].start, sel[i].stop
                start = 0 if start is None else start
                stop = self.shape[i] if stop is None else stop
                stop = max(min(stop, self.shape[i]), start)                                 # :287-290
                newaxis = [None] * sel_ndim
                newaxis[idx] = slice(None)
                sel[i] = torch.arange(start, stop)[tuple(newaxis)]
                idx += 1
        sel = torch.broadcast_tensors(*sel)                                                 # :299
        return sel, scalar_idx

    # ---- getitem (:302-315) -------------------------------------------------------------
    def __getitem__(self, selectors):
        sel, scalar_idx = self._handle_selectors(selectors)
        stacked = torch.stack(sel, dim=0)
        out_shape = stacked.shape[1:]
        flat = stacked.reshape(self.ndim, -1)
        if self._hashmap._values is None:
            values = torch.zeros(flat.shape[1:], dtype=self._dtype)
        else:
            v, _ = self._hashmap.get(flat.T.contiguous().numpy(), fallback_value=0)
            values = torch.from_numpy(np.ascontiguousarray(v))
        values = values.view(out_shape)
        for i in reversed(scalar_idx):
            values.squeeze_(i)
        return values

    # ---- setitem, dense source (:317-327 and sparse_dok_tensor_impl.py:412-474) -----------
    def __setitem__(self, selectors, values):
        sel, _ = self._handle_selectors(selectors)
        bshape = sel[0].shape
        if isinstance(values, RefSparseDOKTensor) or (isinstance(values, Tensor) and values.is_sparse):
            assert tuple(values.shape) == tuple(bshape)
            return self._set_items_sparse(values, sel)
        if not isinstance(values, Tensor):
            # the reference ignores non-tensor values here; its README documents scalar
            # assignment, which is what is restated
            values = torch.tensor(values, dtype=self._dtype)
        values = torch.broadcast_to(values.to(self._dtype), bshape)
        self._set_items_dense(values, sel)

    def _set_items_dense(self, src, sel):
        hm = self._hashmap
        n_sel = int(np.prod(src.shape))
        if n_sel == 0:
            return
        if hm._keys is None:                                                                # :413-416
            first_key = torch.stack([s.reshape(-1)[0] for s in sel], dim=0)[None]
            first_val = src.reshape(-1)[:1][None].contiguous()
            hm.set(first_key.numpy(), first_val.numpy())
        ndim, sel_ndim = len(sel), sel[0].dim()
        esizes = np.array(list(src.shape) + [0] * (8 - sel_ndim), dtype=np.int64)
        estrides = np.array(list(shape_to_stride(tuple(src.shape))) + [0] * (8 - sel_ndim), dtype=np.int64)
        acc = (RefAccessor * ndim)(*[_accessor(s) for s in sel])
        vacc = _accessor(src)
        n_existing = lib().ref_dok_count_items(hm._table(), acc, ndim, sel_ndim, _ptr(esizes), _ptr(estrides),
                                               n_sel, 1)                                    # :448-460
        if hm.n_elements + n_sel > hm.n_buckets * hm._rehash_threshold:                     # :461-462
            hm.rehash(int(np.ceil((hm.n_elements + n_sel) * hm._rehash_factor)))
        lib().ref_dok_set_items_dense(hm._table(), acc, ctypes.byref(vacc), ndim, sel_ndim,
                                      _ptr(esizes), _ptr(estrides), n_sel, 1)               # :464-473
        hm._n_elements += n_sel - int(n_existing)                                           # :474

    def _index_space(self, sel):
        ndim, sel_ndim = len(sel), sel[0].dim()
        shape = tuple(sel[0].shape)
        esizes = np.array(list(shape) + [0] * (8 - sel_ndim), dtype=np.int64)
        estrides = np.array(list(shape_to_stride(shape)) + [0] * (8 - sel_ndim), dtype=np.int64)
        acc = (RefAccessor * ndim)(*[_accessor(s) for s in sel])
        return ndim, sel_ndim, esizes, estrides, acc, int(np.prod(shape))

    # ---- sparse-valued getitem (:342-350, get_items sparse_dok_tensor_impl.py:148-233) ------
    def __spgetitem__(self, selectors):
        sel, _ = self._handle_selectors(selectors)
        bshape = tuple(sel[0].shape)
        out = RefSparseDOKTensor(bshape, dtype=self._dtype, rng=self._rng)
        hm = self._hashmap
        if hm._values is None:
            return out
        ndim, sel_ndim, esizes, estrides, acc, n_sel = self._index_space(sel)
        n = lib().ref_dok_count_items(hm._table(), acc, ndim, sel_ndim, _ptr(esizes), _ptr(estrides), n_sel, 1)
        oh = RefClosedHashmap(n_buckets=int(n * 2.0), rng=self._rng)
        if n:
            oh._allocate(np.zeros((1, sel_ndim), dtype=np.int64), np.zeros((1, 1), dtype=hm._value_dtype))
            lib().ref_dok_get_items(hm._table(), oh._table(), acc, ndim, sel_ndim, _ptr(esizes), _ptr(estrides), n_sel)
            oh._n_elements += int(n)
        out._hashmap = oh
        return out

    # ---- setitem, sparse source (:321-323, set_items_sparse sparse_dok_tensor_impl.py:235-340) ----
    def _set_items_sparse(self, src, sel):
        hm = self._hashmap
        if isinstance(src, RefSparseDOKTensor):
            src_indices, src_values = src.indices().contiguous(), src.values().contiguous()
        else:
            src = src.coalesce() if not src.is_coalesced() else src
            src_indices, src_values = src.indices().contiguous(), src.values().contiguous()
        src_values = src_values.to(self._dtype)
        if hm._keys is None:
            first_key = torch.stack([s.reshape(-1)[0] for s in sel], dim=0)[None]
            hm.set(first_key.numpy(), np.zeros((1, 1), dtype=src_values.numpy().dtype))
        ndim, sel_ndim, esizes, estrides, acc, n_sel = self._index_space(sel)
        n_removed = lib().ref_dok_zero_items(hm._table(), acc, ndim, sel_ndim, _ptr(esizes), _ptr(estrides), n_sel)
        hm._n_elements -= int(n_removed)
        n_src = int(src_values.shape[0])
        hm.rehash(int(np.ceil((hm.n_elements + n_src) * hm._rehash_factor * 2)))
        acc = (RefAccessor * ndim)(*[_accessor(s) for s in sel])
        si, sv = src_indices.numpy(), src_values.numpy()
        lib().ref_dok_set_items_sparse_v1(hm._table(), acc, ndim, sel_ndim, _ptr(si), _ptr(sv), n_src,
                                          int(src_values.dtype.is_floating_point))
        hm._n_elements += n_src
