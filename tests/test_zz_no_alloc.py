"""GPU test of dok_map_compact_static, the read-out that uses the library's own scratch memory
(no buffer from the caller, no allocation): its output must equal dok_map_compact's, bit for bit
and in the same order, on two calls in a row, the second on a smaller table."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _compact_both(lib, hm, dev):
    from doksparse_amd.closed_hashmap import _stream_ptr
    n = hm.n_elements
    desc = ctypes.byref(hm._desc)
    stream = _stream_ptr(dev)
    out = []
    for static in (False, True):
        # outputs pre-filled with a pattern, so that rows a call fails to write show up
        keys = torch.full((n + 3, *hm._key_shape), 0x5A, device=dev, dtype=hm._key_dtype)
        vals = torch.full((n + 3, *hm._value_shape), 0x5A, device=dev, dtype=hm._value_dtype)
        count = torch.full((1,), -1, device=dev, dtype=torch.long)
        if static:
            rc = lib.dok_map_compact_static(desc, keys.data_ptr(), vals.data_ptr(), n + 3, count.data_ptr(), stream)
        else:
            nbytes = int(lib.dok_compact_scratch_bytes(desc))
            scratch = torch.empty(nbytes // 8, device=dev, dtype=torch.long)
            rc = lib.dok_map_compact(desc, keys.data_ptr(), vals.data_ptr(), n + 3, count.data_ptr(),
                                     scratch.data_ptr(), stream)
        assert rc == 0
        torch.cuda.synchronize()
        out.append((keys.cpu().numpy(), vals.cpu().numpy(), int(count.item())))
    return n, out


@pytest.mark.parametrize("kshape,kdtype,vshape,vdtype", [
    ((1,), torch.int64, (1,), torch.float32),          # packed layout
    ((3,), torch.float32, (5,), torch.int64),          # tagged layout
])
def test_static_compact_matches_compact_on_two_calls(cuda, kshape, kdtype, vshape, vdtype):
    from doksparse_amd import CudaClosedHashmap, _lib
    lib = _lib.load()
    assert lib.dok_static_scratch_bytes() == (8 << 20) + 256
    g = torch.Generator().manual_seed(77)
    # the second table is smaller: fewer chunks of the shared scratch are used than the first
    # call left written
    for n, cap in ((300_000, 1 << 20), (5_000, 1 << 14)):
        if kdtype == torch.int64:
            keys = torch.randint(0, 2**62, (n, *kshape), generator=g, dtype=torch.int64)
        else:
            keys = torch.rand((n, *kshape), generator=g, dtype=kdtype)
        if vdtype == torch.int64:
            vals = torch.randint(-2**62, 2**62, (n, *vshape), generator=g, dtype=torch.int64)
        else:
            vals = torch.randn((n, *vshape), generator=g, dtype=vdtype)
        hm = CudaClosedHashmap(n_buckets=cap, device=cuda)
        hm.set(keys.to(cuda), vals.to(cuda))
        hm.remove(keys[: n // 7].to(cuda))                    # tombstones in the table as well
        n_live, (a, b) = _compact_both(lib, hm, cuda)
        assert a[2] == b[2] == n_live
        assert np.array_equal(a[0].view(np.uint8), b[0].view(np.uint8))
        assert np.array_equal(a[1].view(np.uint8), b[1].view(np.uint8))
        # and both are the map: every live key, once
        live = np.unique(keys[n // 7:].numpy().reshape(n - n // 7, -1).view(np.uint8)
                         .reshape(n - n // 7, -1), axis=0)
        got = np.unique(b[0][:n_live].reshape(n_live, -1).view(np.uint8).reshape(n_live, -1), axis=0)
        assert np.array_equal(live, got)


def test_static_compact_refuses_a_table_beyond_its_scratch(cuda):
    from doksparse_amd import CudaClosedHashmap, _lib
    lib = _lib.load()
    hm = CudaClosedHashmap(n_buckets=1024, device=cuda)
    hm.set(torch.arange(10, device=cuda)[:, None], torch.ones(10, 1, device=cuda))
    # the descriptor claims more buckets than the scratch has chunk counters for; the call
    # must return before it launches anything on the (much smaller) real table
    big = _lib.DokTable()
    ctypes.memmove(ctypes.byref(big), ctypes.byref(hm._desc), ctypes.sizeof(big))
    big.n_phys_buckets = (1 << 28) + 256 * 32
    count = torch.zeros(1, device=cuda, dtype=torch.long)
    rc = lib.dok_map_compact_static(ctypes.byref(big), None, None, 0, count.data_ptr(), None)
    assert rc == _lib.DOK_ETOOLARGE
    with pytest.raises(ValueError):
        _lib.check(rc, "compact")
    torch.cuda.synchronize()
    assert hm.n_elements == 10


def test_static_compact_allocates_no_device_memory(cuda):
    """What the entry point is for: with the outputs allocated beforehand, calls of
    dok_map_compact_static leave the device's free memory as it was (no hipMalloc, no hipFree, no
    growth of torch's pool), while giving the right rows."""
    from doksparse_amd import CudaClosedHashmap, _lib
    from doksparse_amd.closed_hashmap import _stream_ptr
    lib = _lib.load()
    n = 200_000
    g = torch.Generator().manual_seed(78)
    keys = torch.unique(torch.randint(0, 2**62, (n,), generator=g))[:, None].to(cuda)
    n = keys.shape[0]
    hm = CudaClosedHashmap(n_buckets=1 << 19, device=cuda)
    hm.set(keys, torch.arange(n, device=cuda, dtype=torch.float32)[:, None])
    assert hm.n_elements == n
    desc, stream = ctypes.byref(hm._desc), _stream_ptr(cuda)
    out_k = torch.zeros(n, 1, device=cuda, dtype=torch.long)
    out_v = torch.zeros(n, 1, device=cuda, dtype=torch.float32)
    count = torch.zeros(1, device=cuda, dtype=torch.long)
    # warm-up: resolves the scratch symbol on this device and loads the kernels
    assert lib.dok_map_compact_static(desc, out_k.data_ptr(), out_v.data_ptr(), n, count.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(cuda)
    reserved_before = torch.cuda.memory_reserved(cuda)
    for _ in range(3):
        out_k.zero_(); out_v.zero_(); count.zero_()          # (in place: no allocation)
        assert lib.dok_map_compact_static(desc, out_k.data_ptr(), out_v.data_ptr(), n, count.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(cuda)
    assert free_after == free_before and torch.cuda.memory_reserved(cuda) == reserved_before
    assert int(count.item()) == n
    assert torch.equal(torch.sort(out_k[:, 0]).values, torch.sort(keys[:, 0]).values)
