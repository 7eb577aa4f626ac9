"""Dictionary-of-keys sparse tensor with the Python surface of the reference's
``SparseDOKTensor`` (reference: sparse_dok/components/sparse_dok_tensor.py:17-561).

The tensor is a size plus a coordinate-keyed ``CudaClosedHashmap`` whose key rows are int64
coordinates and whose values have shape ``(1,)``.  The hot methods run as single fused HIP
kernels of libdokhip:

* ``__getitem__``  : selector gather -> linearise -> table lookup -> dense write
                     (the reference stacks and transposes the selectors first, :302-315)
* ``__setitem__``  : selector gather -> linearise -> upsert (dense source, :317-327 and
                     sparse_dok_tensor_impl.py:412-474)
* ``to_dense``     : one scan of the table scattering into a zero tensor (:195-209)
* ``indices/values``: one compaction pass (:156-169)

Selector handling follows the reference's ``_handle_selectors`` (:220-300), including its axis
placement rule (the broadcast axes of all tensor selectors sit at the position of the first
tensor selector; every slice keeps an axis of its own, in order) and its squeeze of axes named
by scalar selectors.  Where the reference raises by accident (a bare ``int`` selector, numpy
selectors, a scalar selector behind a slice) the intended result is returned instead; a slice
step other than 1, which the reference silently ignores, raises ``ValueError``.
"""
import ctypes
import weakref

import numpy as np
import torch
from torch import Tensor

from . import _lib
from ._lib import DokIndex, DokView, DOK_MAX_DIMS, DOK_LIN_DIMS
from .closed_hashmap import CudaClosedHashmap, _stream_ptr, coord_rows_needed
from .util import str2dtype, next_power_of_2, shape_to_stride

_INT_DTYPES = {torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8}

# The storage of a tensor is a coordinate-keyed map over its size.  Where one 8-byte key can hold a
# linearised coordinate (at most 8 dimensions, fewer than 2^63 elements) the map stores that; a
# larger tensor keeps the int64[ndim] coordinate vectors themselves as multi-word keys (the
# reference's own key format, sparse_dok_tensor.py:45-69).  Every indexing method runs as the same
# fused kernels on either (the library picks them from the table descriptor).  One tag word, ndim
# key words and the value word have to fit a 128-byte bucket, hence DOK_MAX_DIMS dimensions at most.


def _make_storage(size, n_buckets, device, rehash_factor=2.0, rehash_threshold=0.75):
    """An empty map keyed the way a tensor of this size needs it."""
    if len(size) > DOK_MAX_DIMS:
        raise NotImplementedError(f"tensors of more than {DOK_MAX_DIMS} dimensions: a coordinate row "
                                  "no longer fits a 128-byte bucket")
    return CudaClosedHashmap(n_buckets=n_buckets, device=device, coord_dims=tuple(int(s) for s in size),
                             rehash_factor=rehash_factor, rehash_threshold=rehash_threshold)


# `nonzero` of a boolean mask needs a device-to-host synchronisation (its result's shape). Code
# that indexes with the same mask tensor again and again pays that every time, so the index
# tensors of the last few masks are kept, keyed by the mask OBJECT (a weak reference, never an
# address that could be reused) and its version counter, which every in-place write bumps.
_MASK_CACHE = {}
_MASK_CACHE_SIZE = 8


def _mask_indices(mask, device):
    key = id(mask)
    hit = _MASK_CACHE.get(key)
    if hit is not None and hit[0]() is mask and hit[1] == mask._version and hit[2] == device:
        return hit[3]
    idx = mask.to(device).nonzero(as_tuple=True)
    if len(_MASK_CACHE) >= _MASK_CACHE_SIZE:
        _MASK_CACHE.pop(next(iter(_MASK_CACHE)))
    _MASK_CACHE[key] = (weakref.ref(mask), mask._version, device, idx)
    return idx


class _Plan(object):
    """A filled dok_index_t and what goes with it.  Plans are kept per tensor, keyed by the
    STRUCTURE of the indexing expression (kinds of the selectors, slice bounds, shapes and strides of
    the index tensors, identity and version of masks): a later expression of the same structure
    only refreshes the integer bases and the data pointers (`patches`) instead of normalising the
    selectors, laying out the result and filling the descriptor again - which is most of the host
    time of a small indexing call."""
    __slots__ = ("ix", "ref", "views", "out_shape", "final_shape", "scalar_positions", "patches", "masks")


_PLAN_CACHE_SIZE = 32

class SparseDOKTensor(object):
    def __init__(self, size, indices=None, values=None, device=None, dtype=None, storage=None):
        assert isinstance(size, (list, tuple))
        self._plans = {}
        self._size = torch.Size(size)
        # view dimension i addresses dimension _perm[i] of the storage (identity unless the tensor
        # was made by permute/transpose, which share the storage)
        self._perm = tuple(range(len(size)))

        if storage is None:
            self.device = torch.device("cuda:0") if device is None else torch.device(device)
        else:
            assert isinstance(storage, CudaClosedHashmap)
            self.device = storage.device

        if storage is not None and storage._allocated:
            assert len(storage.key_shape) == 1 and storage.key_shape[0] == self.ndim
            self._dtype = storage.value_type
        elif dtype is None:
            self._dtype = torch.float32 if values is None else values.dtype
        else:
            self._dtype = str2dtype(dtype)

        if storage is not None:
            self._hashmap = self._adopt_storage(storage)
        else:
            n_buckets = 32 if indices is None else next_power_of_2(values.shape[0])
            self._hashmap = _make_storage(self._size, n_buckets, self.device)
        if indices is not None:
            assert values is not None
            assert len(indices.shape) == 2
            assert len(values.shape) == 1
            assert indices.shape[1] == values.shape[0]
            assert indices.shape[0] == self.ndim
            self._store_coo(indices.to(self.device), values.to(device=self.device, dtype=self.dtype)[:, None])

    def _store_coo(self, indices, vals):
        """Upsert entries given as [ndim, n] coordinates (this view's dimension order must be the
        storage's) and [n, 1] values; coordinates outside the size are skipped."""
        hm = self._hashmap
        if hm._coord_dims == tuple(self._size):
            hm.set_coo(indices, vals)
        else:
            hm.set(indices.T, vals)

    def _adopt_storage(self, storage):
        """Use `storage` directly if it is keyed the way this tensor needs (coordinates inside this
        size); otherwise move its entries into such a map."""
        if storage._coord_dims == tuple(self._size):
            return storage
        new = _make_storage(self._size, storage.n_buckets, storage.device,
                            storage._rehash_factor, storage._rehash_threshold)
        if storage._allocated:
            keys, values = storage.items()
            if keys.shape[0]:
                new.set(keys.reshape(-1, self.ndim).long(), values)
                new._header[_lib.DOK_H_NOOB] = 0      # entries outside this size are dropped
        return new

    def _ensure_widths(self):
        """Fix the key / value widths of an unallocated map without storing anything."""
        if not self._hashmap._allocated:
            self._hashmap.set(torch.empty(0, self.ndim, device=self.device, dtype=torch.long),
                              torch.empty(0, 1, device=self.device, dtype=self.dtype))

    def _is_permuted(self):
        return self._perm != tuple(range(self.ndim))

    def _to_storage_order(self, per_view_dim):
        """Reorder a per-view-dimension list into the storage's dimension order."""
        out = [None] * self.ndim
        for i, item in enumerate(per_view_dim):
            out[self._perm[i]] = item
        return out

    # ------------------------------------------------------------------ constructors
    @classmethod
    def from_sparse_coo(cls, tensor):
        assert isinstance(tensor, Tensor)
        assert tensor.layout == torch.sparse_coo
        tensor = tensor.coalesce()
        return cls(size=tuple(tensor.shape), indices=tensor._indices(), values=tensor._values(),
                   device=tensor.device)

    @classmethod
    def from_dense(cls, tensor):
        assert isinstance(tensor, Tensor)
        assert tensor.layout == torch.strided
        return cls.from_sparse_coo(tensor.to_sparse())

    @classmethod
    def from_storage(cls, storage, size=None):
        assert isinstance(storage, CudaClosedHashmap)
        assert storage.value_shape == (1,)
        assert len(storage.key_shape) == 1
        ndims = storage.key_shape[0]
        if size is None:
            if storage._coord_dims is not None:
                size = storage._coord_dims
            else:
                size = tuple((storage.keys().max(dim=0).values + 1).cpu().tolist())
        else:
            assert len(size) == ndims
            assert all(i >= 0 for i in size)
        return cls(size=tuple(size), storage=storage)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = {} if kwargs is None else kwargs
        args = [a.to_sparse_coo() if isinstance(a, cls) else a for a in args]
        kwargs = {k: (a.to_sparse_coo() if isinstance(a, cls) else a) for k, a in kwargs.items()}
        return func(*args, **kwargs)

    # ------------------------------------------------------------------ simple properties
    @property
    def is_sparse(self):
        return True

    def _is_coalesced(self):
        return False

    def is_coalesced(self):
        return False

    def size(self):
        return self._size

    @property
    def shape(self):
        return self._size

    @property
    def ndim(self):
        return len(self._size)

    @property
    def dtype(self):
        return self._dtype

    def _stride(self, dim=None):
        stride = shape_to_stride(self.shape)
        return stride if dim is None else stride[dim]

    def storage(self):
        return self._hashmap

    def _nnz(self):
        return self._hashmap.n_elements

    @property
    def sparsity(self):
        volume = 1
        for n in self.shape:
            volume *= int(n)                      # (Python integers: the volume may exceed 64 bits)
        return 1 - self._nnz() / float(volume) if volume else 0.0

    def clone(self, deepclone=True):
        new = SparseDOKTensor(size=tuple(self._size), device=self.device, dtype=self.dtype)
        new._hashmap = self._hashmap.clone(deepclone=deepclone)
        new._perm = self._perm
        new._plans = {}
        return new

    # ------------------------------------------------------------------ read-out
    def indices(self):
        return self._items_coo_view()[0]

    def _items_coo_view(self):
        """(indices [ndim, nnz] in this view's dimension order, values [nnz, 1]) from one pass."""
        idx, values = self._hashmap.items_coo()
        if idx is None:
            return (torch.empty(self.ndim, 0, device=self.device, dtype=torch.long),
                    torch.empty(0, 1, device=self.device, dtype=self.dtype))
        if self._is_permuted():
            idx = idx[list(self._perm)].contiguous()
        return idx, values

    def values(self):
        values = self._hashmap.values()
        if values is None:
            return torch.empty(0, device=self.device, dtype=self.dtype)
        return values.flatten()

    def _indices(self):
        return self._hashmap._keys

    def _values(self):
        return self._hashmap._values

    def set_values(self, selectors, new_values):
        self._hashmap.set_values(selectors=selectors, new_values=new_values[:, None])

    def to_sparse_coo(self):
        idx, values = self._items_coo_view()
        return torch.sparse_coo_tensor(indices=idx, values=values.flatten(), size=tuple(self.shape),
                                       device=self.device)

    @property
    def _as_sparse_coo_tensor(self):
        return self.to_sparse_coo()

    def to_sparse_csr(self):
        return self.to_sparse_coo().to_sparse_csr()

    def to_dense(self):
        hm = self._hashmap
        storage_shape = self._to_storage_order(list(self.shape))
        dense = torch.zeros(tuple(storage_shape), device=self.device, dtype=self.dtype)
        if hm._allocated and dense.numel():
            lib = _lib.load()
            _lib.check(lib.dok_to_dense(ctypes.byref(hm._desc), dense.data_ptr(), _stream_ptr(self.device)),
                       "to_dense")
        return dense.permute(*self._perm).contiguous() if self._is_permuted() else dense

    def resize(self, *new_size):
        new_size = tuple(new_size) + (self.ndim - len(new_size)) * (-1,)
        assert len(new_size) == self.ndim
        new_size = torch.Size([self.shape[i] if new_size[i] == -1 else new_size[i] for i in range(self.ndim)])
        if new_size != self._size:
            self._rekey(new_size, lambda idx: idx)
        return self

    def _rekey(self, new_size, fn):
        """Rebuild the storage for `new_size`, mapping the [ndim, nnz] indices through fn."""
        old = self._hashmap
        new = _make_storage(new_size, old.n_buckets, self.device, old._rehash_factor, old._rehash_threshold)
        idx = values = None
        if old._allocated:
            keys, values = old.items()
            if keys.shape[0]:
                idx = fn(keys.T[list(self._perm)] if self._is_permuted() else keys.T)
        self._hashmap = new
        self._size = torch.Size(new_size)
        self._perm = tuple(range(len(new_size)))
        self._plans = {}
        if idx is not None:
            self._store_coo(idx.contiguous(), values)
            new._header[_lib.DOK_H_NOOB] = 0          # entries outside the new size are dropped

    # ------------------------------------------------------------------ selectors
    def _normalise_slice(self, sl, dim):
        if sl.step not in (None, 1):
            raise ValueError("only slices with step 1 are supported")
        size = self.shape[dim]
        start = 0 if sl.start is None else int(sl.start)
        stop = size if sl.stop is None else int(sl.stop)
        if start < 0:
            start = max(start + size, 0)
        if stop < 0:
            stop = stop + size
        stop = max(min(stop, size), start)
        return start, stop

    def _normalise(self, selectors):
        """One entry per tensor dimension: an int64 device tensor, a Python int, or a
        (start, stop) pair for a slice."""
        if not isinstance(selectors, tuple):
            selectors = (selectors,)
        flat = []
        for sel in selectors:
            if isinstance(sel, np.ndarray):
                sel = torch.from_numpy(sel)
            if isinstance(sel, Tensor) and sel.dtype == torch.bool:
                flat.extend(_mask_indices(sel, self.device))
            elif isinstance(sel, Tensor) and sel.dtype in _INT_DTYPES:
                flat.append(sel.to(self.device).long())
            elif isinstance(sel, (bool, np.bool_)):
                raise ValueError("boolean scalars are not valid selectors")
            elif isinstance(sel, (int, np.integer)):
                flat.append(int(sel))
            elif isinstance(sel, slice):
                flat.append(sel)
            elif isinstance(sel, (tuple, list)):
                flat.append(torch.tensor(sel, device=self.device, dtype=torch.long))
            else:
                raise ValueError(f"unsupported selector {type(sel)}")
        if len(flat) > self.ndim:
            raise IndexError(f"too many indices for tensor of dimension {self.ndim}")
        flat += [slice(None)] * (self.ndim - len(flat))
        return [self._normalise_slice(s, i) if isinstance(s, slice) else s for i, s in enumerate(flat)]

    @staticmethod
    def _broadcast_shape(shapes):
        out = []
        for shape in shapes:
            shape = tuple(shape)
            if len(shape) > len(out):
                out = [1] * (len(shape) - len(out)) + out
            off = len(out) - len(shape)
            for k, n in enumerate(shape):
                if out[off + k] == 1:
                    out[off + k] = n
                elif n != 1 and n != out[off + k]:
                    raise RuntimeError(f"selector shapes {shapes} do not broadcast")
        return tuple(out)

    def _layout(self, flat):
        """Where every selector lands in the result (reference rule, :255-296): the broadcast
        axes of all tensor selectors (integers count as 0-dim tensors) sit together at the
        position of the first of them; every slice keeps an axis of its own, in order.
        Returns (bshape, first axis of the broadcast block, {dim: axis} for slices, out_shape,
        scalar positions)."""
        is_t = [not isinstance(s, tuple) for s in flat]
        scalar_positions = [i for i, s in enumerate(flat)
                            if isinstance(s, int) or (isinstance(s, Tensor) and s.ndim == 0)]
        bshape = self._broadcast_shape([() if isinstance(s, int) else s.shape
                                        for s, t in zip(flat, is_t) if t]) if any(is_t) else tuple()
        first = is_t.index(True) if any(is_t) else None
        out_shape, slice_axis = [], {}
        for i, sel in enumerate(flat):
            if is_t[i]:
                if i == first:
                    out_shape.extend(bshape)
            else:
                slice_axis[i] = len(out_shape)
                out_shape.append(sel[1] - sel[0])
        return bshape, first, slice_axis, tuple(out_shape), scalar_positions

    def _handle_selectors(self, selectors, return_slice_as_tensor=True):
        """Turn an indexing expression into one int64 selector per tensor dimension, all
        broadcast (as views) to the shape of the result, plus the positions of the scalar
        selectors.  Reference: sparse_dok_tensor.py:220-300."""
        flat = self._normalise(selectors)
        bshape, first, slice_axis, out_shape, scalar_positions = self._layout(flat)
        out_ndim = len(out_shape)
        out = []
        for i, sel in enumerate(flat):
            if isinstance(sel, tuple):
                if return_slice_as_tensor:
                    view_shape = [1] * out_ndim
                    view_shape[slice_axis[i]] = sel[1] - sel[0]
                    out.append(torch.arange(sel[0], sel[1], device=self.device).reshape(view_shape))
                else:
                    out.append(slice(sel[0], sel[1]))
            else:
                if isinstance(sel, int):
                    sel = torch.tensor(sel, device=self.device, dtype=torch.long)
                view_shape = [1] * out_ndim
                view_shape[first:first + len(bshape)] = bshape
                out.append(torch.broadcast_to(sel, bshape).reshape(view_shape))
        if return_slice_as_tensor:
            out = list(torch.broadcast_tensors(*out))
        return out, scalar_positions

    def _fill_index(self, ix, storage_dim, data_ptr, base, strides):
        view = ix.sel[storage_dim]
        view.data = data_ptr
        view.base = base
        for j, st in enumerate(strides):
            view.strides[j] = st

    def _max_axes(self):
        """Most axes an indexing expression's result may have on this tensor's storage."""
        return DOK_MAX_DIMS if self._hashmap._coord_rows else DOK_LIN_DIMS

    def _index_desc(self, selectors):
        """dok_index_t of materialised selectors (the result of _handle_selectors)."""
        out_shape = tuple(selectors[0].shape)
        if len(out_shape) > self._max_axes():
            raise NotImplementedError(f"indexing expressions with more than {self._max_axes()} axes")
        ix = DokIndex()
        ix.ndim = self.ndim
        ix.sel_ndim = len(out_shape)
        for j, s in enumerate(out_shape):
            ix.shape[j] = s
        keep = []
        for d, sel in enumerate(selectors):
            assert sel.dtype == torch.long and sel.device == self.device
            self._fill_index(ix, self._perm[d], sel.data_ptr(), 0, sel.stride())
            keep.append(sel)
        return ix, out_shape

    def _plan_key(self, selectors):
        """Hashable structure of an indexing expression, or None when it holds selectors that are
        converted on the way (lists, numpy arrays, tensors of another dtype or on another device)."""
        key = []
        for sel in selectors:
            t = type(sel)
            if t is int:
                key.append(0)
            elif t is slice:
                key.append((sel.start, sel.stop, sel.step))
            elif t is Tensor:
                if sel.device != self.device:
                    return None
                if sel.dtype is torch.bool:
                    key.append((id(sel), sel._version, None))
                elif sel.dtype is torch.long:
                    key.append((sel.shape, sel.stride()))
                else:
                    return None
            else:
                return None
        return tuple(key)

    def _plan(self, selectors):
        """dok_index_t straight from the expression: integers and slices become affine
        selectors that need no device tensor (no arange kernel, no host-to-device copy of a
        scalar); only real index tensors are passed by pointer.  Returns (plan, tensors to keep alive
        until the launch)."""
        if not isinstance(selectors, tuple):
            selectors = (selectors,)
        key = self._plan_key(selectors)
        plan = self._plans.get(key) if key is not None else None
        if plan is not None:
            keep = []
            views = plan.views
            for code, pos, sd in plan.patches:
                sel = selectors[pos]
                if code == 0:
                    views[sd].base = sel
                elif code == 1:
                    views[sd].data = sel.data_ptr()
                else:
                    if plan.masks[pos]() is not sel:          # another tensor at a recycled address
                        plan = None
                        break
                    idx = _mask_indices(sel, self.device)
                    for m, d in enumerate(sd):
                        views[d].data = idx[m].data_ptr()
                    keep.append(idx)
            if plan is not None:
                return plan, keep
        flat = self._normalise(selectors)
        bshape, first, slice_axis, out_shape, scalar_positions = self._layout(flat)
        if len(out_shape) > self._max_axes():
            raise NotImplementedError(f"indexing expressions with more than {self._max_axes()} axes")
        ix = DokIndex()
        ix.ndim = self.ndim
        ix.sel_ndim = len(out_shape)
        for j, s in enumerate(out_shape):
            ix.shape[j] = s
        keep = []
        zeros = [0] * len(out_shape)
        for d, sel in enumerate(flat):
            strides = list(zeros)
            if isinstance(sel, tuple):
                strides[slice_axis[d]] = 1
                self._fill_index(ix, self._perm[d], None, sel[0], strides)
            elif isinstance(sel, int):
                self._fill_index(ix, self._perm[d], None, sel, strides)
            else:
                view = torch.broadcast_to(sel, bshape)
                strides[first:first + len(bshape)] = view.stride()
                self._fill_index(ix, self._perm[d], view.data_ptr(), 0, strides)
                keep.append(view)
        plan = _Plan()
        plan.ix, plan.ref = ix, ctypes.byref(ix)
        plan.views = [ix.sel[d] for d in range(self.ndim)]
        plan.out_shape, plan.scalar_positions = out_shape, scalar_positions
        # the reference squeezes the output axis numbered like each scalar selector's position
        final = list(out_shape)
        for i in reversed(scalar_positions):
            if i < len(final) and final[i] == 1:
                del final[i]
        plan.final_shape = tuple(final)
        if key is not None:
            # which tensor dimension(s) every selector of the expression feeds (a mask of k
            # dimensions stands for k of them)
            plan.patches, plan.masks, d = [], {}, 0
            for pos, sel in enumerate(selectors):
                if type(sel) is int:
                    plan.patches.append((0, pos, self._perm[d]))
                    d += 1
                elif type(sel) is slice:
                    d += 1
                elif sel.dtype is torch.bool:
                    plan.patches.append((2, pos, tuple(self._perm[d + m] for m in range(sel.ndim))))
                    plan.masks[pos] = weakref.ref(sel)
                    d += sel.ndim
                else:
                    plan.patches.append((1, pos, self._perm[d]))
                    d += 1
            if len(self._plans) >= _PLAN_CACHE_SIZE:
                self._plans.pop(next(iter(self._plans)))
            self._plans[key] = plan
        return plan, keep

    # ------------------------------------------------------------------ indexing
    def __getitem__(self, selectors):
        plan, keep = self._plan(selectors)
        hm = self._hashmap
        if not hm._allocated:
            return torch.zeros(plan.final_shape, device=self.device, dtype=self._dtype)
        values = torch.empty(plan.final_shape, device=self.device, dtype=self._dtype)
        if values.numel():
            rc = _lib.load().dok_getitem_dense(ctypes.byref(hm._desc), plan.ref, values.data_ptr(), _stream_ptr(self.device))
            if rc:
                _lib.check(rc, "__getitem__")
        return values

    def __setitem__(self, selectors, values):
        if isinstance(values, SparseDOKTensor) or (isinstance(values, Tensor) and values.is_sparse):
            mats, _ = self._handle_selectors(selectors)
            out_shape = tuple(mats[0].shape)
            assert tuple(values.shape) == out_shape, \
                f"expecting the value shape to be {out_shape}, got {tuple(values.shape)} instead"
            return self._set_items_sparse(values, mats)
        plan, keep = self._plan(selectors)
        if not isinstance(values, Tensor):
            values = torch.tensor(values, device=self.device, dtype=self.dtype)
        values = torch.broadcast_to(values.to(device=self.device, dtype=self.dtype), plan.out_shape)
        self._set_items_dense(values, plan.ix, selectors)

    def _set_items_dense(self, src, ix, expr):
        """Reference: SparseDOKTensorImplCuda.set_items_dense (sparse_dok_tensor_impl.py:412-474).
        One device read-back per call (after the kernel: entry count and error counters); the
        reference's count kernel + `.item()` before the scatter is replaced by the in-kernel count."""
        n_sel = int(np.prod(src.shape, dtype=np.int64))
        if n_sel == 0:
            return
        hm = self._hashmap
        if not hm._allocated:
            # The reference stores the first element before anything else (sparse_dok_tensor_impl.py:
            # 413-416), which its growth rule then counts; the kernel below writes it again.
            mats, _ = self._handle_selectors(expr)
            first_key = torch.stack([s.reshape(-1)[0] for s in self._to_storage_order(mats)], dim=0)[None]
            hm.set(first_key, src.reshape(-1)[:1, None].contiguous())
            hm._header[_lib.DOK_H_NOOB] = 0       # an out-of-range first key is counted by the kernel below
        view = DokView()
        view.data = src.data_ptr()
        for j, st in enumerate(src.stride()):
            view.strides[j] = st
        # growth rule of the reference: decided on the number of selector elements
        limit = hm.n_buckets * hm._rehash_threshold
        if hm._n_upper + n_sel > limit:
            n_now = hm.n_elements
            if n_now + n_sel > limit:
                hm.rehash(int(np.ceil((n_now + n_sel) * hm._rehash_factor)))
        lib = _lib.load()
        hm._touch()
        ws = hm._bulk_workspace(n_sel) if hm._coord_rows else None
        if ws is not None:
            _lib.check(lib.dok_setitem_dense_bulk(ctypes.byref(hm._desc), ctypes.byref(ix), ctypes.byref(view),
                                                  ws.data_ptr(), ws.numel(), _stream_ptr(self.device)), "__setitem__")
        else:
            _lib.check(lib.dok_setitem_dense(ctypes.byref(hm._desc), ctypes.byref(ix), ctypes.byref(view),
                                             _stream_ptr(self.device)), "__setitem__")
        header = hm._read_header()
        hm._n_upper, hm._n_exact = int(header[_lib.DOK_H_NELEM]), True
        n_oob = int(header[_lib.DOK_H_NOOB])
        if n_oob:
            hm._header[_lib.DOK_H_NOOB] = 0
            raise IndexError(f"{n_oob} coordinates fall outside the tensor of size {tuple(self.shape)}")

    def __spgetitem__(self, selectors):
        """Sparse-valued gather: a SparseDOKTensor over the index space holding the addressed
        entries (reference: :342-350 and get_items, sparse_dok_tensor_impl.py:148-233)."""
        selectors, _ = self._handle_selectors(selectors)
        out_shape = tuple(selectors[0].shape)
        if len(out_shape) == 0:
            raise NotImplementedError("sparse-valued indexing needs at least one result axis")
        out = SparseDOKTensor(size=out_shape, device=self.device, dtype=self.dtype)
        hm = self._hashmap
        if not hm._allocated:
            return out
        if coord_rows_needed(out_shape):
            # an index space of more than 8 axes (its offsets cannot key the result's table): look
            # the coordinate rows up, keep the hits, key them by their index vector
            n = 0
            if selectors[0].numel():
                rows = torch.stack(self._to_storage_order(list(selectors)), dim=-1).reshape(-1, self.ndim)
                values, found = hm.get(rows)
                at = found.nonzero().flatten()
                n = int(at.shape[0])
            out._hashmap = _make_storage(out_shape, int(n * 2.0), self.device)
            out._ensure_widths()
            if n:
                out._store_coo(torch.stack(torch.unravel_index(at, out_shape)), values[at])
            return out
        ix, out_shape = self._index_desc(selectors)
        lib = _lib.load()
        stream = _stream_ptr(self.device)
        n = 0
        if selectors[0].numel():
            count = torch.zeros(1, device=self.device, dtype=torch.long)
            _lib.check(lib.dok_count_items(ctypes.byref(hm._desc), ctypes.byref(ix), count.data_ptr(), stream),
                       "count_items")
            n = int(count.item())
        om = CudaClosedHashmap(n_buckets=int(n * 2.0), device=self.device, coord_dims=out_shape)
        om.set(torch.zeros(0, len(out_shape), device=self.device, dtype=torch.long),
               torch.zeros(0, 1, device=self.device, dtype=self.dtype))          # fixes widths, allocates
        if n:
            _lib.check(lib.dok_getitem_sparse(ctypes.byref(hm._desc), ctypes.byref(ix), ctypes.byref(om._desc),
                                              stream), "__spgetitem__")
        om._n_upper, om._n_exact = n, False
        out._hashmap = om
        return out

    def _set_items_sparse(self, src, selectors):
        """Reference: set_items_sparse (sparse_dok_tensor_impl.py:235-340): clear every addressed
        element, grow, then store the source's nonzero entries through the selectors."""
        if isinstance(src, SparseDOKTensor):
            # coordinates in the order of the source's (possibly permuted) view
            src_indices, vals = src._items_coo_view()
            src_values = vals.flatten()
        else:
            if src.layout != torch.sparse_coo:
                src = src.to_sparse_coo()
            src = src.coalesce()
            src_indices, src_values = src.indices().contiguous(), src.values()
        src_indices = src_indices.to(self.device)
        src_values = src_values.to(device=self.device, dtype=self.dtype).contiguous()
        hm = self._hashmap
        if not hm._allocated:
            # (reference: sparse_dok_tensor_impl.py:237-240)
            first_key = torch.stack([s.reshape(-1)[0] for s in self._to_storage_order(selectors)], dim=0)[None]
            hm.set(first_key, torch.zeros(1, 1, device=self.device, dtype=self.dtype))
            hm._header[_lib.DOK_H_NOOB] = 0
        ix, _ = self._index_desc(selectors)
        lib = _lib.load()
        stream = _stream_ptr(self.device)
        hm._touch()
        if selectors[0].numel():
            _lib.check(lib.dok_zero_items(ctypes.byref(hm._desc), ctypes.byref(ix), stream), "zero_items")
        n_src = int(src_values.shape[0])
        n_now = hm.n_elements
        hm.rehash(int(np.ceil((n_now + n_src) * hm._rehash_factor * 2)))
        if n_src:
            bits = 8 * src_values.element_size()
            mask = (1 << bits) - 1
            if src_values.dtype.is_floating_point:
                mask >>= 1                                   # minus zero counts as zero
            _lib.check(lib.dok_setitem_sparse(ctypes.byref(hm._desc), ctypes.byref(ix), src_indices.data_ptr(),
                                              src_values.data_ptr(), n_src, mask, stream), "__setitem__")
        hm._n_upper, hm._n_exact = n_now + n_src, False

    def count_items(self, selectors):
        """Number of addressed elements that are stored (reference: count_items,
        sparse_dok_tensor_impl.py:56-108)."""
        selectors, _ = self._handle_selectors(selectors)
        count = torch.zeros(1, device=self.device, dtype=torch.long)
        hm = self._hashmap
        if hm._allocated and selectors[0].numel():
            ix, _ = self._index_desc(selectors)
            lib = _lib.load()
            _lib.check(lib.dok_count_items(ctypes.byref(hm._desc), ctypes.byref(ix), count.data_ptr(),
                                           _stream_ptr(self.device)), "count_items")
        return count

    def zero_items(self, selectors):
        """Remove every addressed element (reference: zero_items, sparse_dok_tensor_impl.py:110-146)."""
        selectors, _ = self._handle_selectors(selectors)
        hm = self._hashmap
        if hm._allocated and selectors[0].numel():
            ix, _ = self._index_desc(selectors)
            lib = _lib.load()
            hm._touch()
            _lib.check(lib.dok_zero_items(ctypes.byref(hm._desc), ctypes.byref(ix), _stream_ptr(self.device)),
                       "zero_items")

    # ------------------------------------------------------------------ torch.sparse pass-throughs
    def sum(self, dim=None, keepdim=False):
        coo = self.to_sparse_coo()
        if dim is None:
            return torch.sparse.sum(coo)
        out = torch.sparse.sum(coo, dim=dim)
        return out

    def norm(self, dim=None, p=2, keepdim=False):
        coo = self.to_sparse_coo().coalesce()
        v = coo.values()
        powered = v.bool().to(v.dtype) if p == 0 else v.abs() if p == 1 else v.square() if p == 2 else v.abs().pow(p)
        t = torch.sparse_coo_tensor(coo.indices(), powered, size=tuple(self.shape), device=self.device)
        y = torch.sparse.sum(t) if dim is None else torch.sparse.sum(t, dim=dim)
        y = y.to_dense() if y.is_sparse else y
        if keepdim and dim is not None:
            for d in sorted([dim] if isinstance(dim, int) else list(dim)):
                y = y.unsqueeze(d)
        return y.sqrt() if p == 2 else y.pow(1.0 / p) if p not in (0, 1) else y

    def normalize(self, dim=-1, p=2, eps=1e-12):
        """Stored magnitudes divided by the p-norm of their slice along `dim`, as a sparse COO
        tensor (reference: sparse_dok_tensor.py:405-411 through functions.py:123-161, which takes
        the softmax of log |v|^p over the stored entries - signs are not kept - and the 1/p-th
        power of the result; entries with |v|^p below eps count as eps)."""
        coo = self.to_sparse_coo().coalesce()
        v = coo.values()
        powered = v.bool().to(v.dtype) if p == 0 else v.abs() if p == 1 else v.square() if p == 2 else v.abs().pow(p)
        logs = powered.clamp_min(eps).log()
        t = torch.sparse_coo_tensor(coo.indices(), logs, size=tuple(self.shape), device=self.device)
        y = torch.sparse.softmax(t, dim=dim % self.ndim)
        return y.sqrt() if p == 2 else y.pow(1.0 / p)

    def normalize_(self, dim=-1, p=2, eps=1e-12):
        """The reference's in-place variant works on the temporary COO copy it makes of the tensor
        (sparse_dok_tensor.py:413-419), so the DOK tensor keeps its values and the normalised COO
        tensor is what the caller gets; the same here."""
        return self.normalize(dim=dim, p=p, eps=eps)

    def softmax(self, dim=-1):
        return torch.sparse.softmax(self.to_sparse_coo().coalesce(), dim=dim % self.ndim)

    def log_softmax(self, dim=-1):
        return torch.sparse.log_softmax(self.to_sparse_coo().coalesce(), dim=dim % self.ndim)

    def index_select(self, dim, index):
        return self.to_sparse_coo().index_select(dim=dim, index=index)

    def select(self, dim, index):
        return self.to_sparse_coo().select(dim=dim, index=index)

    # ------------------------------------------------------------------ views and re-layout
    def permute_(self, *ordering):
        """Reorder the dimensions in place; nothing is moved (reference: :439-443).  The order is
        given as separate arguments, as in the reference, or as one sequence, as torch takes it."""
        if len(ordering) == 1 and isinstance(ordering[0], (list, tuple)):
            ordering = ordering[0]
        ordering = [int(o) % self.ndim for o in ordering]
        assert sorted(ordering) == list(range(self.ndim))
        self._perm = tuple(self._perm[o] for o in ordering)
        self._size = torch.Size(self._size[o] for o in ordering)
        self._plans = {}
        return self

    def permute(self, *ordering):
        """A view with reordered dimensions that shares this tensor's storage: writes through
        either are seen by both (reference: :445-450)."""
        return self.clone(deepclone=False).permute_(*ordering)

    def transpose_(self, dim0, dim1):
        assert dim0 != dim1
        order = list(range(self.ndim))
        dim0, dim1 = dim0 % self.ndim, dim1 % self.ndim
        order[dim0], order[dim1] = dim1, dim0
        return self.permute_(*order)

    def transpose(self, dim0, dim1):
        assert dim0 != dim1
        order = list(range(self.ndim))
        dim0, dim1 = dim0 % self.ndim, dim1 % self.ndim
        order[dim0], order[dim1] = dim1, dim0
        return self.permute(*order)

    def t(self):
        assert self.ndim == 2, "tensor isn't 2 dimensional, try x.transpose(dim1, dim2)"
        return self.transpose(0, 1)

    @property
    def T(self):
        return self.t()

    def flatten(self):
        stride = torch.tensor(self._stride(), device=self.device, dtype=torch.long)[:, None]
        flat = (self.indices() * stride).sum(dim=0, keepdim=True)
        return SparseDOKTensor(size=[int(np.prod(self.shape))], indices=flat, values=self.values(),
                               device=self.device)

    def reshape(self, *new_shape):
        assert np.prod(new_shape) == np.prod(self.shape)
        flat = self.flatten()
        if len(new_shape) == 1:
            return flat
        idx = flat.indices()
        strides = torch.tensor(shape_to_stride(new_shape), device=self.device, dtype=torch.long)[:, None]
        sizes = torch.tensor(new_shape, device=self.device, dtype=torch.long)[:, None]
        new_idx = torch.div(idx.expand(len(new_shape), -1), strides, rounding_mode="floor") % sizes
        return SparseDOKTensor(size=tuple(new_shape), indices=new_idx, values=flat.values(), device=self.device)

    # ------------------------------------------------------------------ unary ops on the stored values
    def _map_values(self, fn):
        keys, values = self._hashmap.items()
        new = SparseDOKTensor(size=tuple(self._size), device=self.device, dtype=self.dtype)
        new._hashmap = _make_storage(self._size, self._hashmap.n_buckets, self.device,
                                     self._hashmap._rehash_factor, self._hashmap._rehash_threshold)
        if keys is not None and keys.shape[0]:
            if self._is_permuted():
                keys = keys[:, list(self._perm)].contiguous()
            new._hashmap.set(keys, fn(values))
        return new

    def abs(self):
        return self._map_values(torch.abs)

    def _float_only(self):
        assert self.dtype in {torch.half, torch.float, torch.double}

    def sqrt(self):
        self._float_only()
        return self._map_values(torch.sqrt)

    def ceil(self):
        self._float_only()
        return self._map_values(torch.ceil)

    def floor(self):
        self._float_only()
        return self._map_values(torch.floor)

    def round(self, decimals=0):
        self._float_only()
        return self._map_values(lambda v: torch.round(v, decimals=decimals or 0))

    def __repr__(self):
        return (f"SparseDOKTensor(indices={self.indices()},\n"
                f"                values={self.values()},\n"
                f"                size={self.size()}, nnz={self._nnz()}, sparsity={round(self.sparsity, 6)})")
