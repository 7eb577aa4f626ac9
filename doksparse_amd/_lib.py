"""ctypes binding of ``libdokhip.so`` (the C ABI declared in ``include/dokhip.h``).

The shared library is built in-tree by ``doksparse_amd/build.py`` (``hipcc`` for gfx950).
There is no CPU fallback: if the library is missing, loading raises.
"""
import ctypes
import os
from ctypes import c_int32, c_int64, c_uint64, c_void_p, c_char_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
# DOKHIP_LIB points at another build of the same ABI (e.g. a tuning variant)
LIB_PATH = os.environ.get("DOKHIP_LIB") or os.path.join(_HERE, "libdokhip.so")

DOK_OK = 0
DOK_EINVAL = -1
DOK_EUNSUPPORTED = -2
DOK_ELAUNCH = -3
DOK_ETOOLARGE = -4

DOK_BUCKET_BYTES = 128
DOK_MAX_DIMS = 14          # most dimensions of a coordinate table / an index space
DOK_LIN_DIMS = 8           # ... of a table of linearised coordinates and of its index spaces
DOK_HEADER_WORDS = 16
DOK_H_NELEM = 0
DOK_H_NFULL = 1
DOK_H_NPROBE = 2
DOK_H_NOOB = 3
DOK_H_NOPS = 4

DOK_LAYOUT_PACKED8 = 1
DOK_LAYOUT_TAGGED = 2


class DokTable(ctypes.Structure):
    _fields_ = [
        ("buckets", c_void_p),
        ("header", c_void_p),
        ("n_phys_buckets", c_int64),
        ("seed", c_uint64),
        ("key_bytes", c_int32),
        ("value_bytes", c_int32),
        ("lin_ndim", c_int32),
        ("reserved_", c_int32),
        ("lin_dims", c_int64 * DOK_MAX_DIMS),
    ]


class DokView(ctypes.Structure):
    _fields_ = [
        ("data", c_void_p),
        ("base", c_int64),
        ("strides", c_int64 * DOK_MAX_DIMS),
    ]


class DokIndex(ctypes.Structure):
    _fields_ = [
        ("ndim", c_int32),
        ("sel_ndim", c_int32),
        ("shape", c_int64 * DOK_MAX_DIMS),
        ("sel", DokView * DOK_MAX_DIMS),
    ]


# name -> (restype, argtypes); every symbol include/dokhip.h declares
SIGNATURES = {
    "dok_layout_of": (c_int32, [c_int32, c_int32, POINTER(c_int32)]),
    "dok_phys_buckets_for": (c_int64, [c_int64, c_int32, c_int32]),
    "dok_last_hip_error": (c_char_p, []),
    "dok_table_clear": (c_int32, [POINTER(DokTable), c_void_p]),
    "dok_map_get": (c_int32, [POINTER(DokTable), c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "dok_map_get_dev_fallback": (c_int32, [POINTER(DokTable), c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "dok_map_get_stats": (c_int32, [POINTER(DokTable), c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "dok_map_set": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "dok_bulk_workspace_bytes": (c_int64, [POINTER(DokTable), c_int64]),
    "dok_map_set_bulk": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "dok_coo_set_bulk": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "dok_map_build_bulk": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "dok_coo_build_bulk": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "dok_map_remove": (c_int32, [POINTER(DokTable), c_void_p, c_int64, c_void_p, c_void_p]),
    "dok_map_remove_unique": (c_int32, [POINTER(DokTable), c_void_p, c_int64, c_void_p, c_void_p]),
    "dok_map_remove_bulk": (c_int32, [POINTER(DokTable), c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "dok_map_count_existing": (c_int32, [POINTER(DokTable), c_void_p, c_int64, c_void_p, c_void_p]),
    "dok_map_update_existing": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "dok_compact_scratch_bytes": (c_int64, [POINTER(DokTable)]),
    "dok_map_compact": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "dok_static_scratch_bytes": (c_int64, []),
    "dok_map_compact_static": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "dok_coo_set": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p]),
    "dok_coo_compact": (c_int32, [POINTER(DokTable), c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "dok_map_rehash": (c_int32, [POINTER(DokTable), POINTER(DokTable), c_void_p]),
    "dok_rehash_bulk_workspace_bytes": (c_int64, [POINTER(DokTable), POINTER(DokTable)]),
    "dok_map_rehash_bulk": (c_int32, [POINTER(DokTable), POINTER(DokTable), c_void_p, c_int64, c_void_p]),
    "dok_getitem_dense": (c_int32, [POINTER(DokTable), POINTER(DokIndex), c_void_p, c_void_p]),
    "dok_setitem_dense": (c_int32, [POINTER(DokTable), POINTER(DokIndex), POINTER(DokView), c_void_p]),
    "dok_setitem_dense_bulk": (c_int32, [POINTER(DokTable), POINTER(DokIndex), POINTER(DokView), c_void_p, c_int64, c_void_p]),
    "dok_count_items": (c_int32, [POINTER(DokTable), POINTER(DokIndex), c_void_p, c_void_p]),
    "dok_zero_items": (c_int32, [POINTER(DokTable), POINTER(DokIndex), c_void_p]),
    "dok_getitem_sparse": (c_int32, [POINTER(DokTable), POINTER(DokIndex), POINTER(DokTable), c_void_p]),
    "dok_setitem_sparse": (c_int32, [POINTER(DokTable), POINTER(DokIndex), c_void_p, c_void_p, c_int64,
                                     c_uint64, c_void_p]),
    "dok_to_dense": (c_int32, [POINTER(DokTable), c_void_p, c_void_p]),
    "dok_line_gather": (c_int32, [POINTER(DokTable), c_int64, c_uint64, c_void_p, c_void_p]),
    "dok_line_gather_granule": (c_int32, [POINTER(DokTable), c_int64, c_uint64, c_int32, c_void_p, c_void_p]),
}

_lib = None


def load():
    """Load the library once and attach the signatures.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m doksparse_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no CPU fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


class DokError(RuntimeError):
    pass


def check(rc, what):
    """Turn a negative return code into an exception of the kind the reference raises."""
    if rc == DOK_OK:
        return
    if rc == DOK_EINVAL:
        raise AssertionError(f"{what}: invalid argument")
    if rc == DOK_EUNSUPPORTED:
        raise NotImplementedError(f"{what}: not supported by the table layouts (a key/value row too wide for a "
                                  "128-byte bucket, or a linearised coordinate space of 2^63 or more elements)")
    if rc == DOK_ETOOLARGE:
        raise ValueError(f"{what}: the table is larger than the library's own scratch memory serves; "
                         "use the variant that takes a scratch buffer")
    if rc == DOK_ELAUNCH:
        msg = load().dok_last_hip_error().decode()
        raise DokError(f"{what}: HIP launch failed: {msg}")
    raise DokError(f"{what}: error {rc}")
