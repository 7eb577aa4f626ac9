"""MI355X-native batched hashmap and DOK sparse-tensor indexing (drop-in for the matching
classes of DeMoriarty/DOKSparse's ``sparse_dok`` package)."""
from .closed_hashmap import CudaClosedHashmap
from .sparse_dok_tensor import SparseDOKTensor

sparse_dok_tensor = SparseDOKTensor

__all__ = ["CudaClosedHashmap", "SparseDOKTensor", "sparse_dok_tensor"]
