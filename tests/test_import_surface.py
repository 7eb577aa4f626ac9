"""The reference's import surface resolves to this package's classes.  No kernel is launched."""
from doksparse_amd import CudaClosedHashmap, SparseDOKTensor


def test_reference_import_surface():
    """`from sparse_dok import ...` of the reference (sparse_dok/__init__.py:1-2) resolves to the
    classes of this package."""
    import sparse_dok
    import sparse_dok.components as comp
    assert sparse_dok.CudaClosedHashmap is CudaClosedHashmap
    assert sparse_dok.SparseDOKTensor is SparseDOKTensor
    assert sparse_dok.sparse_dok_tensor is SparseDOKTensor
    assert comp.CudaClosedHashmap is CudaClosedHashmap and comp.SparseDOKTensor is SparseDOKTensor
