"""RoDe row-decomposition SpMM / SDDMM for AMD MI355X (gfx950).

Public surface (same names as the reference's ``RoDe_SDDMM/rode_sddmm.py``):
``RoDeCSR``, ``rode_sddmm``, ``torch_sddmm_reference``, ``compare_results``;
plus ``rode_spmm`` for the SpMM host API, which the reference exposes in C++
only (``RoDe_SpMM/RoDeSpmm.h``).
"""
from .rode_sddmm import RoDeCSR, compare_results, rode_sddmm, torch_sddmm_reference  # noqa: F401
from .rode_spmm import rode_spmm  # noqa: F401
from .autograd import csr_row_softmax, sparse_attention  # noqa: F401

__all__ = ["RoDeCSR", "rode_sddmm", "rode_spmm", "csr_row_softmax", "sparse_attention",
           "torch_sddmm_reference", "compare_results"]
