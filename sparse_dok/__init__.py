"""Import surface of the reference package: ``from sparse_dok import CudaClosedHashmap,
SparseDOKTensor`` keeps working unchanged (reference: sparse_dok/__init__.py:1-2).  The classes
are those of ``doksparse_amd``; nothing else lives here."""
from doksparse_amd import CudaClosedHashmap, SparseDOKTensor

sparse_dok_tensor = SparseDOKTensor

__all__ = ["CudaClosedHashmap", "SparseDOKTensor", "sparse_dok_tensor"]
