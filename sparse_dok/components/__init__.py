"""``from sparse_dok.components import ...`` of the reference (sparse_dok/components/__init__.py:1-2)."""
from doksparse_amd import CudaClosedHashmap, SparseDOKTensor

__all__ = ["CudaClosedHashmap", "SparseDOKTensor"]
