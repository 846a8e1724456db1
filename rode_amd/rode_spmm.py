"""SpMM op on a ``RoDeCSR``.  The reference offers SpMM only as a C++ host API
(``RoDe_SpMM/RoDeSpmm.h:4-8``); this wraps the same entry point for tensors."""
import torch

from . import rode_sddmm_hip


def rode_spmm(sparse_matrix, dense, out=None, values=None):
    """C = S @ dense.  ``dense`` is (n, width) float32 or float16 with ``width`` a
    multiple of 4 (8 for float16; multiples of 32 are the fast path); returns an
    (m, width) float32 tensor.  ``values`` (optional)
    replaces the values of S for this call.  Differentiable with respect to dense
    and values when ``out`` is not given."""
    if dense.dim() != 2 or dense.shape[0] != sparse_matrix.n:
        raise ValueError(f"dense shape must be ({sparse_matrix.n}, width), got {tuple(dense.shape)}")
    vec = 8 if dense.dtype == torch.float16 else 4
    if dense.shape[1] == 0 or dense.shape[1] % vec != 0:
        raise ValueError(f"dense width must be a positive multiple of {vec}, got {dense.shape[1]}")
    assert dense.is_cuda and dense.device == sparse_matrix.device, (
        f"dense must be on {sparse_matrix.device}, got {dense.device}")
    assert dense.dtype in (torch.float32, torch.float16), f"dense must be float32 or float16, got {dense.dtype}"
    seg = sparse_matrix.config
    assert seg["k_block"] == 32 and seg["vec_len"] == 4, "the kernels need k_block=32, vec_len=4"
    vals = sparse_matrix.values if values is None else values
    if out is None and torch.is_grad_enabled() and (dense.requires_grad or vals.requires_grad):
        from .autograd import SpmmFunction
        return SpmmFunction.apply(sparse_matrix, vals, dense)
    if values is not None:
        sparse_matrix = sparse_matrix.with_values(values)
    return rode_sddmm_hip.spmm_forward(
        sparse_matrix.block_indices, sparse_matrix.residue_indices, sparse_matrix.st_offsets,
        sparse_matrix.m1, sparse_matrix.m2, sparse_matrix.row_offsets, sparse_matrix.column_indices,
        sparse_matrix.values, sparse_matrix.m, sparse_matrix.n, dense.contiguous(), out, plan=sparse_matrix.plan,
        seg_length=sparse_matrix.config["seg_length"], checked_lists=True,
        plans=sparse_matrix.call_plans(dense.shape[1], 4),
        every_row_stored=out is None and sparse_matrix.spmm_stores_every_row())
