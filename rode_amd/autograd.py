"""Gradients of SDDMM and SpMM, CSR row softmax, and the sparse-attention chain
SDDMM -> softmax -> SpMM on one decomposed pattern.

The reference's op is forward-only (``RoDe_SDDMM/rode_sddmm.py:194-248``).  Every
gradient is again one of the two kernels on the same pattern or on its transpose:

    out = v (.) (L R^T)|pattern :  dL = (g (.) v) R          (SpMM, same pattern)
                                   dR = (g (.) v)^T L        (SpMM, transposed pattern)
                                   dv = g (.) (L R^T)|pattern (SDDMM)
    C   = A B                   :  dB = A^T dC               (SpMM, transposed pattern)
                                   dv = (dC B^T)|pattern      (SDDMM with unit values)
"""
import ctypes

import torch

from . import _lib, rode_sddmm_hip


def _sddmm(csr, values, lhs, rhs):
    return rode_sddmm_hip.sddmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                        csr.row_offsets, csr.column_indices, values.contiguous(), csr.m, csr.n,
                                        lhs.contiguous(), rhs.contiguous(), lhs.shape[1], plan=csr.plan, seg_length=csr.config["seg_length"])


def _spmm(csr, values, dense):
    return rode_sddmm_hip.spmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                       csr.row_offsets, csr.column_indices, values.contiguous(), csr.m, csr.n,
                                       dense.contiguous(), plan=csr.plan, seg_length=csr.config["seg_length"],
                                       every_row_stored=csr.spmm_stores_every_row())


class SddmmFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, csr, values, lhs, rhs):
        ctx.csr = csr
        ctx.save_for_backward(values, lhs, rhs)
        return _sddmm(csr, values.detach().float(), lhs.detach(), rhs.detach())

    @staticmethod
    def backward(ctx, g):
        csr = ctx.csr
        values, lhs, rhs = ctx.saved_tensors
        g = g.contiguous().float()
        gv = g * values.float()
        d_values = d_lhs = d_rhs = None
        if ctx.needs_input_grad[2]:
            d_lhs = _spmm(csr, gv, rhs.float()).to(lhs.dtype)
        if ctx.needs_input_grad[3]:
            csr_t, perm = csr.transpose(with_values=False)
            d_rhs = _spmm(csr_t, rode_sddmm_hip.permute(gv, perm), lhs.float()).to(rhs.dtype)
        if ctx.needs_input_grad[1]:
            d_values = _sddmm(csr, g, lhs, rhs).to(values.dtype)
        return None, d_values, d_lhs, d_rhs


class SpmmFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, csr, values, dense):
        ctx.csr = csr
        ctx.save_for_backward(values, dense)
        return _spmm(csr, values.detach().float(), dense.detach())

    @staticmethod
    def backward(ctx, g):
        csr = ctx.csr
        values, dense = ctx.saved_tensors
        g = g.contiguous().float()
        d_values = d_dense = None
        if ctx.needs_input_grad[2]:
            csr_t, perm = csr.transpose(with_values=False)
            d_dense = _spmm(csr_t, rode_sddmm_hip.permute(values.float().contiguous(), perm), g).to(dense.dtype)
        if ctx.needs_input_grad[1]:
            if g.shape[1] % 4 != 0 or g.shape[1] > 512:
                raise NotImplementedError("the gradient with respect to the sparse values is an SDDMM over the dense "
                                          "width, which must be a multiple of 4 up to 512")
            d_values = _sddmm(csr, torch.ones_like(values, dtype=torch.float32), g, dense.float()).to(values.dtype)
        return None, d_values, d_dense


def _softmax_call(fn_name, row_offsets, a, b, scale):
    lib = _lib.load()
    out = torch.empty_like(a)
    if a.numel() == 0:  # a pattern without nonzeros
        return out
    m = row_offsets.numel() - 1
    with rode_sddmm_hip._on_device(a.device):
        s = rode_sddmm_hip._stream_handle(a.device)
        if b is None:
            code = lib.rode_hip_csr_softmax_f32(m, row_offsets.data_ptr(), a.data_ptr(), out.data_ptr(), scale, s)
        else:
            code = lib.rode_hip_csr_softmax_backward_f32(m, row_offsets.data_ptr(), a.data_ptr(), b.data_ptr(),
                                                         out.data_ptr(), scale, s)
    _lib.check(code, fn_name)
    return out


class CsrSoftmaxFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, csr, scores, scale):
        p = _softmax_call("rode_hip_csr_softmax_f32", csr.row_offsets, scores.detach().contiguous().float(), None,
                          float(scale))
        ctx.csr, ctx.scale = csr, float(scale)
        ctx.save_for_backward(p)
        return p

    @staticmethod
    def backward(ctx, g):
        (p,) = ctx.saved_tensors
        ds = _softmax_call("rode_hip_csr_softmax_backward_f32", ctx.csr.row_offsets, p, g.contiguous().float(),
                           ctx.scale)
        return None, ds, None


def csr_row_softmax(sparse_matrix, scores, scale=1.0):
    """softmax(scale * scores) over every row of the pattern; (nnz,) float32."""
    if scores.shape != sparse_matrix.values.shape:
        raise ValueError(f"scores shape must be {tuple(sparse_matrix.values.shape)}, got {tuple(scores.shape)}")
    assert scores.is_cuda and scores.device == sparse_matrix.device, f"scores must be on {sparse_matrix.device}"
    return CsrSoftmaxFunction.apply(sparse_matrix, scores, scale)


# Rows longer than this many nonzeros keep the one wavefront that the fused kernel gives a
# row busy for too long; such patterns go through the three separate kernels, whose row
# decomposition balances them.
FUSED_MAX_ROW = 16384


def _attention_call(csr, values, q, k, v, scale, keep):
    """q: (m, d) or (heads, m, d), k and v alike; returns out of q's shape (float32) and
    what the gradient needs: with keep == "probs" the probabilities, (nnz,) or (heads, nnz),
    and None; with keep == "scores" the scaled scores in their place and the
    (maximum, 1 / sum) pair of every row, (m, 2) or (heads, m, 2) - cheaper to write, and
    p = exp(score - maximum) / sum; with keep == None two Nones."""
    lib = _lib.load()
    heads = q.shape[0] if q.dim() == 3 else 1
    m, d = q.shape[-2:]
    nnz = values.numel()
    lead = q.shape[:-2]
    probs = torch.empty(lead + (nnz,), dtype=torch.float32, device=q.device) if keep else None
    stats = torch.empty(lead + (m, 2), dtype=torch.float32, device=q.device) if keep == "scores" else None
    if nnz == 0:  # no nonzeros: nothing attends to anything
        return torch.zeros(lead + (m, d), dtype=torch.float32, device=q.device), probs, stats
    out = torch.empty(lead + (m, d), dtype=torch.float32, device=q.device)
    plans = csr.call_plans()  # (the attention kernels use a group plan and ignore the other kinds)
    with rode_sddmm_hip._on_device(q.device):
        code = lib.rode_hip_attention_forward_batched(
            _lib.DENSE_CODE["f16" if q.dtype == torch.float16 else "f32"], heads, m, csr.n, nnz, d,
            csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(), values.data_ptr(), q.data_ptr(), k.data_ptr(),
            v.data_ptr(), float(scale), out.data_ptr(), probs.data_ptr() if keep else None,
            stats.data_ptr() if stats is not None else None, ctypes.byref(plans),
            rode_sddmm_hip._stream_handle(q.device))
    _lib.check(code, "rode_hip_attention_forward_batched")
    return out, probs, stats


def _attention_backward_call(csr, csr_t, t_slot, probs, stats, g, out, q, k, v, scale):
    """(dq, dk, dv) in float32 through the two gradient kernels: the row pass over the
    pattern, the column pass over the transposed pattern; every head in the same two launches.
    probs, stats: what ``_attention_call`` kept (stats None: probs holds probabilities)."""
    lib = _lib.load()
    heads = q.shape[0] if q.dim() == 3 else 1
    m, d = q.shape[-2:]
    n = k.shape[-2]
    nnz = csr.nnz
    kind = _lib.DENSE_CODE["f16" if q.dtype == torch.float16 else "f32"]
    dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    dk = torch.empty(k.shape, dtype=torch.float32, device=q.device)
    dv = torch.empty(v.shape, dtype=torch.float32, device=q.device)
    pairs = torch.empty(2 * probs.numel(), dtype=torch.float32, device=q.device)
    plans, plans_t = csr.call_plans(), csr_t.call_plans()
    with rode_sddmm_hip._on_device(q.device):
        s = rode_sddmm_hip._stream_handle(q.device)
        _lib.check(lib.rode_hip_attention_backward_rows(
            kind, heads, m, n, nnz, d, csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(), csr.values.data_ptr(),
            probs.data_ptr(), stats.data_ptr() if stats is not None else None, g.data_ptr(), out.data_ptr(), k.data_ptr(),
            v.data_ptr(), float(scale), t_slot.data_ptr(),
            dq.data_ptr(), pairs.data_ptr(), ctypes.byref(plans), s), "rode_hip_attention_backward_rows")
        _lib.check(lib.rode_hip_attention_backward_cols(
            kind, heads, m, n, nnz, d, csr_t.row_offsets.data_ptr(), csr_t.column_indices.data_ptr(), pairs.data_ptr(),
            g.data_ptr(), q.data_ptr(), dk.data_ptr(), dv.data_ptr(), ctypes.byref(plans_t), s),
            "rode_hip_attention_backward_cols")
    return dq, dk, dv


# True / False / "auto": whether the gradient of the fused attention runs as the two gradient
# kernels or as the chain of separate kernels.  "auto": the two kernels unless a column of the
# pattern has more than FUSED_MAX_ROW nonzeros (one wavefront per column, as per row in the
# forward pass).
FUSED_BACKWARD = "auto"


class FusedAttentionFunction(torch.autograd.Function):
    """Forward: one kernel (``rode_hip_attention_forward_batched``), which leaves the scaled
    scores and every row's (maximum, 1 / sum) for the gradient.  Backward: two kernels on
    those and the output (``rode_hip_attention_backward_rows`` / ``_cols``), or the kernels of
    the chain - the probabilities from the scores (row softmax), dP = (dOut v^T)|pattern
    (SDDMM), the softmax gradient, dq and dk as SpMM on the pattern and its transpose,
    dv = P^T dOut."""

    @staticmethod
    def forward(ctx, csr, q, k, v, scale):
        need = any(ctx.needs_input_grad[1:4])
        values = csr.values
        q, k, v = q.detach().contiguous(), k.detach().contiguous(), v.detach().contiguous()
        out, scores, stats = _attention_call(csr, values, q, k, v, scale, "scores" if need else None)
        ctx.csr, ctx.scale = csr, float(scale)
        if need:
            ctx.save_for_backward(scores, stats, q, k, v, out)
        return out

    @staticmethod
    def backward(ctx, g):
        csr, scale = ctx.csr, ctx.scale
        scores, stats, q, k, v, out = ctx.saved_tensors
        g = g.contiguous().float()
        dq = dk = dv = None
        if scores.numel() == 0:  # no nonzeros: the output does not depend on anything
            zeros = lambda t, need: torch.zeros_like(t) if need else None
            return (None, zeros(q, ctx.needs_input_grad[1]), zeros(k, ctx.needs_input_grad[2]),
                    zeros(v, ctx.needs_input_grad[3]), None)
        csr_t = perm = None
        fused = FUSED_BACKWARD
        if fused or ctx.needs_input_grad[2] or ctx.needs_input_grad[3]:
            csr_t, perm = csr.transpose(with_values=False)
        if fused == "auto":
            fused = csr_t.max_row_length <= FUSED_MAX_ROW
        if fused:
            dq, dk, dv = _attention_backward_call(csr, csr_t, csr.transposed_slots(), scores, stats, g, out, q, k, v, scale)
            return (None, dq.to(q.dtype) if ctx.needs_input_grad[1] else None,
                    dk.to(k.dtype) if ctx.needs_input_grad[2] else None,
                    dv.to(v.dtype) if ctx.needs_input_grad[3] else None, None)
        need = ctx.needs_input_grad
        # the chain works on probabilities: the row softmax of the kept scores (the same
        # exp(score - maximum) / sum the forward kernel used)
        flat = scores.reshape(-1, scores.shape[-1])
        probs = torch.stack([_softmax_call("rode_hip_csr_softmax_f32", csr.row_offsets, flat[h], None, 1.0)
                             for h in range(flat.shape[0])]).reshape(scores.shape)
        if q.dim() == 3:  # the chain of separate kernels takes one head at a time
            per_head = [FusedAttentionFunction._chained_backward(csr, csr_t, perm, scale, need, probs[h], g[h], q[h], k[h], v[h])
                        for h in range(q.shape[0])]
            dq, dk, dv = (torch.stack(t) if t[0] is not None else None for t in zip(*per_head))
        else:
            dq, dk, dv = FusedAttentionFunction._chained_backward(csr, csr_t, perm, scale, need, probs, g, q, k, v)
        return None, dq, dk, dv, None

    @staticmethod
    def _chained_backward(csr, csr_t, perm, scale, need, probs, g, q, k, v):
        dq = dk = dv = None
        if need[3]:
            dv = _spmm(csr_t, rode_sddmm_hip.permute(probs, perm), g).to(v.dtype)
        if need[1] or need[2]:
            dp = _sddmm(csr, csr.ones(), g, v.float())  # (g is float32: both operands of an SDDMM share a type)
            ds = _softmax_call("rode_hip_csr_softmax_backward_f32", csr.row_offsets, probs, dp, scale)
            ds.mul_(csr.values)  # scores are values (.) (q k^T)
            # float16 operands are gathered as they are (the sums are float32 either way)
            if need[1]:
                dq = _spmm(csr, ds, k).to(q.dtype)
            if need[2]:
                dk = _spmm(csr_t, rode_sddmm_hip.permute(ds, perm), q).to(k.dtype)
        return dq, dk, dv


def sparse_attention(mask, q, k, v, scale=None, fused="auto"):
    """softmax(scale * mask (.) (q k^T)) v on the sparsity pattern of ``mask`` (a
    ``RoDeCSR``; its values multiply the scores, use 1 for a pure mask).  q is (m, d),
    k is (n, d) with d in {32, 64, 128}; v is (n, dv) with dv a multiple of 32.  One
    row decomposition serves all three kernels; differentiable in q, k and v.  With a
    leading dimension - q (heads, m, d), k and v (heads, n, d) - every head uses the one
    mask, and the fused kernels take all heads in one launch.

    ``fused``: "auto" runs the forward pass as one kernel when it applies (dv == d, q, k
    and v of one dtype, float32 mask values, no row longer than ``FUSED_MAX_ROW``) and as
    SDDMM -> softmax -> SpMM otherwise; True insists on the one kernel (``ValueError`` when
    it does not apply), False on the three."""
    from .rode_sddmm import rode_sddmm
    from .rode_spmm import rode_spmm
    if scale is None:
        scale = q.shape[-1] ** -0.5
    if fused not in (True, False, "auto"):
        raise ValueError(f'fused must be True, False or "auto", got {fused!r}')
    if q.dim() not in (2, 3) or k.dim() != q.dim() or v.dim() != q.dim():
        raise ValueError("q, k and v must all be 2-D, or all 3-D with the heads first")
    if q.dim() == 3 and not (q.shape[0] == k.shape[0] == v.shape[0]):
        raise ValueError(f"q, k and v must have the same number of heads, got {q.shape[0]}, {k.shape[0]}, {v.shape[0]}")
    if fused:
        why = None
        if q.shape[-1] not in (32, 64, 128) or k.shape[-1] != q.shape[-1] or v.shape[-1] != q.shape[-1]:
            why = "q, k and v must have the same width, 32, 64 or 128"
        elif not (q.dtype == k.dtype == v.dtype and q.dtype in (torch.float32, torch.float16)):
            why = "q, k and v must share one dtype, float32 or float16"
        elif mask.values.dtype != torch.float32:
            why = "the mask values must be float32"
        elif q.shape[-2] != mask.m or k.shape[-2] != mask.n or v.shape[-2] != mask.n:
            why = f"q must have {mask.m} rows, k and v {mask.n}"
        elif not (q.is_cuda and q.device == mask.device and k.device == q.device and v.device == q.device):
            why = f"q, k and v must be on {mask.device}"
        elif fused == "auto" and mask.max_row_length > FUSED_MAX_ROW:
            why = "rows too long"
        if why is None:
            if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
                return FusedAttentionFunction.apply(mask, q, k, v, scale)
            # nothing to differentiate: the kernel keeps nothing for a gradient
            return _attention_call(mask, mask.values, q.contiguous(), k.contiguous(), v.contiguous(), scale, None)[0]
        if fused is True:
            raise ValueError(f"the fused attention kernel does not apply: {why}")
    if q.dim() == 3:  # the three kernels take one head at a time
        return torch.stack([sparse_attention(mask, q[h], k[h], v[h], scale, False) for h in range(q.shape[0])])
    scores = rode_sddmm(mask, q, k)
    probs = csr_row_softmax(mask, scores, scale)
    return rode_spmm(mask, v, values=probs)
