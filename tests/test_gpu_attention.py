"""The chain around the op that benchmark configuration 5 describes: SDDMM scores ->
(row softmax) -> SpMM on one decomposed pattern, plus gradients.  None of this exists
in the reference (forward-only SDDMM), so the oracles are the CPU oracle for the two
products and dense fp64 PyTorch (autograd) for softmax and gradients."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dense(rp, col, val, m, n, dtype=torch.float64):
    from gpu_common import DEV
    from helpers import row_of_index
    A = torch.zeros(m, n, dtype=dtype, device=DEV)
    A[torch.from_numpy(row_of_index(rp)).to(DEV), torch.from_numpy(col.astype(np.int64)).to(DEV)] = \
        torch.from_numpy(val).to(DEV, dtype)
    return A


@pytest.mark.parametrize("half", [False, True])
def test_sddmm_then_spmm_pipeline(half):
    """S = mask (.) (Q K^T), O = S V with the decomposition computed once
    (configuration 5 at 1/4 size; fp16 operands accumulate in fp32)."""
    import oracle
    from gpu_common import DEV, TOL_F16, TOL_F32, make_csr, round_half
    from helpers import spmm_row_l1_error
    from rode_amd import rode_sddmm, rode_spmm, workloads
    m, n, rp, col, val = workloads.config("c5_attention", 1 / 4)
    d = 64
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((m, d)).astype(np.float32) for _ in range(3))
    dt = torch.float16 if half else torch.float32
    mask = make_csr(rp, col, val, m, n, d)
    scores = rode_sddmm(mask, torch.from_numpy(q).to(DEV, dt), torch.from_numpy(k).to(DEV, dt))
    out = rode_spmm(mask.with_values(scores), torch.from_numpy(v).to(DEV, dt)).cpu().numpy()
    assert mask.with_values(scores).block_indices.data_ptr() == mask.block_indices.data_ptr()
    if half:
        q, k, v = round_half(q), round_half(k), round_half(v)
    s64 = oracle.sddmm_f64(rp, col, val, q, k)
    # the second product starts from the fp32 scores the first one delivered
    ref = oracle.spmm_f64(rp, col, scores.cpu().numpy(), v)
    assert spmm_row_l1_error(out, ref) <= (TOL_F16 if half else TOL_F32)
    # end to end against fp64 all the way: errors of both stages, still inside the bound
    ref_all = oracle.spmm_d(rp, col, s64, v.astype(np.float64))
    assert spmm_row_l1_error(out, ref_all) <= (TOL_F16 if half else TOL_F32)


def test_transpose():
    from gpu_common import make_csr
    from helpers import random_csr
    rng = np.random.default_rng(1)
    m, n = 300, 411
    rp, col, val = random_csr(rng, m, n, 30, long_rows=2, long_len=400)
    csr = make_csr(rp, col, val, m, n, 32)
    csr_t, perm = csr.transpose()
    assert (csr_t.m, csr_t.n, csr_t.nnz) == (n, m, csr.nnz)
    A = _dense(rp, col, val, m, n)
    At = _dense(csr_t.row_offsets.cpu().numpy(), csr_t.column_indices.cpu().numpy(), csr_t.values.cpu().numpy(), n, m)
    assert torch.equal(At, A.t())
    assert torch.equal(csr_t.values, csr.values[perm])
    again, _ = csr.transpose()
    assert again.block_indices.data_ptr() == csr_t.block_indices.data_ptr()  # cached
    # a copy with other values made BEFORE the first transpose shares the cache with its source
    fresh = make_csr(rp, col, val, m, n, 32)
    copy = fresh.with_values(fresh.values * 2)
    t1, _ = copy.transpose()
    t2, _ = fresh.transpose()
    assert t1.block_indices.data_ptr() == t2.block_indices.data_ptr()
    assert torch.equal(t1.values, 2 * t2.values)


def test_row_softmax_forward_backward():
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import csr_row_softmax
    rng = np.random.default_rng(2)
    m, n = 500, 3000
    rp, col, val = random_csr(rng, m, n, 60, long_rows=3, long_len=2500, empty_frac=0.1)
    csr = make_csr(rp, col, val, m, n, 32)
    s = torch.from_numpy(rng.standard_normal(len(val)).astype(np.float32) * 4).to(DEV).requires_grad_()
    w = torch.from_numpy(rng.standard_normal(len(val)).astype(np.float32)).to(DEV)
    p = csr_row_softmax(csr, s, 0.7)
    (p * w).sum().backward()
    # dense fp64 reference with -inf outside the pattern
    rows = torch.from_numpy(np.repeat(np.arange(m), np.diff(rp))).to(DEV)
    cols = torch.from_numpy(col.astype(np.int64)).to(DEV)
    sd = s.detach().double().requires_grad_()
    dense = torch.full((m, n), float("-inf"), dtype=torch.float64, device=DEV).index_put((rows, cols), 0.7 * sd)
    nonempty = torch.from_numpy(np.diff(rp) > 0).to(DEV)
    pd = torch.softmax(dense[nonempty], dim=1)
    full = torch.zeros(m, n, dtype=torch.float64, device=DEV).index_put((torch.nonzero(nonempty)[:, 0],), pd)
    pref = full[rows, cols]
    (pref * w.double()).sum().backward()
    assert (p.detach().double() - pref.detach()).abs().max().item() < 1e-6
    sums = torch.zeros(m, dtype=torch.float64, device=DEV).index_add(0, rows, p.detach().double())
    assert (sums[nonempty] - 1).abs().max().item() < 1e-5
    assert (s.grad.double() - sd.grad).abs().max().item() < 1e-5


def test_row_softmax_in_place():
    """The C ABI allows out == in and ds == dp."""
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(6)
    m, n = 400, 2000
    rp, col, val = random_csr(rng, m, n, 70, long_rows=3, long_len=1900, empty_frac=0.1)
    csr = make_csr(rp, col, val, m, n, 32)
    s = torch.from_numpy(rng.standard_normal(len(val)).astype(np.float32) * 3).to(DEV)
    g = torch.from_numpy(rng.standard_normal(len(val)).astype(np.float32)).to(DEV)
    p = torch.empty_like(s)
    rp_d = csr.row_offsets.data_ptr()
    _lib.check(lib.rode_hip_csr_softmax_f32(m, rp_d, s.data_ptr(), p.data_ptr(), 0.5, None), "softmax")
    inplace = s.clone()
    _lib.check(lib.rode_hip_csr_softmax_f32(m, rp_d, inplace.data_ptr(), inplace.data_ptr(), 0.5, None), "softmax")
    ds = torch.empty_like(s)
    _lib.check(lib.rode_hip_csr_softmax_backward_f32(m, rp_d, p.data_ptr(), g.data_ptr(), ds.data_ptr(), 0.5, None), "bwd")
    g_inplace = g.clone()
    _lib.check(lib.rode_hip_csr_softmax_backward_f32(m, rp_d, p.data_ptr(), g_inplace.data_ptr(), g_inplace.data_ptr(),
                                                     0.5, None), "bwd")
    torch.cuda.synchronize()
    assert torch.equal(inplace, p) and torch.equal(g_inplace, ds)


@pytest.mark.parametrize("k", [32, 64, 128, 40])
def test_sddmm_and_spmm_gradients(k):
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import rode_sddmm, rode_spmm
    rng = np.random.default_rng(k)
    m, n = 260, 333
    rp, col, val = random_csr(rng, m, n, 25, long_rows=2, long_len=300)
    csr = make_csr(rp, col, val, m, n, k)
    rows = torch.from_numpy(np.repeat(np.arange(m), np.diff(rp))).to(DEV)
    cols = torch.from_numpy(col.astype(np.int64)).to(DEV)
    mk = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(DEV)
    lhs, rhs, w = mk(m, k).requires_grad_(), mk(n, k).requires_grad_(), mk(len(val))
    vals = csr.values.clone().requires_grad_()
    out = rode_sddmm(csr, lhs, rhs, values=vals)
    (out * w).sum().backward()
    l64, r64, v64 = (t.detach().double().requires_grad_() for t in (lhs, rhs, vals))
    ref = v64 * (l64 @ r64.t())[rows, cols]
    (ref * w.double()).sum().backward()
    for got, want in ((out, ref), (lhs.grad, l64.grad), (rhs.grad, r64.grad), (vals.grad, v64.grad)):
        scale = want.abs().max().item() + 1e-12
        assert (got.detach().double() - want.detach()).abs().max().item() <= 2e-5 * scale
    # SpMM: C = A B
    dense, wc = mk(n, k).requires_grad_(), mk(m, k)
    vals2 = csr.values.clone().requires_grad_()
    C = rode_spmm(csr, dense, values=vals2)
    (C * wc).sum().backward()
    d64, v64 = dense.detach().double().requires_grad_(), vals2.detach().double().requires_grad_()
    A = torch.zeros(m, n, dtype=torch.float64, device=DEV).index_put((rows, cols), v64)
    Cref = A @ d64
    (Cref * wc.double()).sum().backward()
    for got, want in ((C, Cref), (dense.grad, d64.grad), (vals2.grad, v64.grad)):
        scale = want.abs().max().item() + 1e-12
        assert (got.detach().double() - want.detach()).abs().max().item() <= 2e-5 * scale
    # without requires_grad the plain path is taken and nothing is recorded
    assert not rode_sddmm(csr, lhs.detach(), rhs.detach()).requires_grad


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("half", [False, True])
def test_sparse_attention_against_dense(half, fused):
    from gpu_common import DEV, make_csr
    from rode_amd import sparse_attention, workloads
    m, n, rp, col, val = workloads.config("c5_attention", 1 / 16)
    d = 64
    rng = np.random.default_rng(8)
    dt = torch.float16 if half else torch.float32
    mk = lambda r: torch.from_numpy(rng.standard_normal((r, d)).astype(np.float32)).to(DEV, dt)
    q, k, v = mk(m).requires_grad_(), mk(n).requires_grad_(), mk(n).requires_grad_()
    w = torch.from_numpy(rng.standard_normal((m, d)).astype(np.float32)).to(DEV)
    mask = make_csr(rp, col, val, m, n, d)
    out = sparse_attention(mask, q, k, v, fused=fused)
    (out * w).sum().backward()
    q64, k64, v64 = (t.detach().double().requires_grad_() for t in (q, k, v))
    allowed = _dense(rp, col, val, m, n) != 0
    scores = (q64 @ k64.t()) * d ** -0.5
    ref = torch.softmax(scores.masked_fill(~allowed, float("-inf")), dim=1) @ v64
    (ref * w.double()).sum().backward()
    tol = 3e-3 if half else 2e-5
    for got, want in ((out, ref), (q.grad, q64.grad), (k.grad, k64.grad), (v.grad, v64.grad)):
        scale = want.abs().max().item()
        assert (got.detach().double() - want.detach()).abs().max().item() <= tol * scale


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("half", [False, True])
def test_fused_attention_kernel_against_the_three_kernels(d, half):
    """rode_hip_attention_forward against fp64 on the host and against SDDMM -> softmax ->
    SpMM of this library: weighted mask values, rows without nonzeros, rows of 1, 63, 64,
    65 and 700 nonzeros (one step, a full step, a step and one slot, many steps), scores
    large enough that the running maximum matters."""
    from gpu_common import DEV, make_csr
    from rode_amd import csr_row_softmax, rode_sddmm, sparse_attention
    from rode_amd.autograd import _attention_call
    rng = np.random.default_rng(100 + d)
    m, n = 300, 2000
    lens = rng.integers(0, 90, m)
    lens[:9] = [0, 1, 63, 64, 65, 700, 0, 128, 1500 if d == 64 else 40]  # 1500: longer than the scores kept in LDS
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum(lens)
    col = np.concatenate([np.sort(rng.choice(n, l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(0.5, 1.5, len(col)).astype(np.float32)
    dt = torch.float16 if half else torch.float32
    mk = lambda r, s: torch.from_numpy((s * rng.standard_normal((r, d))).astype(np.float32)).to(DEV, dt)
    q, k, v = mk(m, 1.5), mk(n, 1.5), mk(n, 1.0)
    mask = make_csr(rp, col, val, m, n, d)
    scale = 0.37
    out, probs, none = _attention_call(mask, mask.values, q, k, v, scale, "probs")
    assert none is None
    out_only, none, none2 = _attention_call(mask, mask.values, q, k, v, scale, None)
    assert none is None and none2 is None and torch.equal(out, out_only)
    # the other form of what a gradient needs: scaled scores and (maximum, 1 / sum) per row
    out_s, scores, stats = _attention_call(mask, mask.values, q, k, v, scale, "scores")
    assert torch.equal(out, out_s) and stats.shape == (m, 2)
    row_of = torch.repeat_interleave(torch.arange(m, device=DEV), torch.from_numpy(np.diff(rp)).to(DEV))
    from_scores = torch.exp(scores - stats[row_of, 0]) * stats[row_of, 1]
    assert (from_scores - probs).abs().max().item() <= 2e-6
    # fp64 on the host
    q64, k64, v64 = (t.double().cpu().numpy() for t in (q, k, v))
    rows = np.repeat(np.arange(m), lens)
    sc = scale * val.astype(np.float64) * np.einsum("ij,ij->i", q64[rows], k64[col])
    ref_out = np.zeros((m, d))
    ref_p = np.zeros(len(col))
    for r in range(m):
        a, b = rp[r], rp[r + 1]
        if b > a:
            e = np.exp(sc[a:b] - sc[a:b].max())
            ref_p[a:b] = e / e.sum()
            ref_out[r] = ref_p[a:b] @ v64[col[a:b]]
    # tolerance: scores reach +-30 here, an fp32 dot product of 128 such terms is off by ~1e-5,
    # and a probability near 1/2 moves by as much; fp16 operands are compared after rounding
    tol = 2e-3 if half else 5e-5
    assert np.abs(probs.cpu().numpy() - ref_p).max() <= tol
    assert np.abs(out.cpu().numpy() - ref_out).max() <= tol * max(1.0, np.abs(ref_out).max())
    assert not out[0].any() and not out[6].any()  # rows without nonzeros
    # the three kernels
    chain_p = csr_row_softmax(mask, rode_sddmm(mask, q, k), scale)
    assert (chain_p - probs).abs().max().item() <= tol
    chain = sparse_attention(mask, q, k, v, scale=scale, fused=False)
    assert (chain - out).abs().max().item() <= tol * max(1.0, chain.abs().max().item())


def test_fused_attention_without_nonzeros():
    from gpu_common import DEV, make_csr
    from rode_amd import sparse_attention
    m, n, d = 10, 12, 32
    rp = np.zeros(m + 1, dtype=np.int32)
    mask = make_csr(rp, np.zeros(0, dtype=np.int32), np.zeros(0, dtype=np.float32), m, n, d)
    z = lambda r: torch.ones(r, d, device=DEV)
    for fused in (True, False):
        out = sparse_attention(mask, z(m), z(n), z(n), fused=fused)
        assert out.shape == (m, d) and not out.any()


def test_fused_attention_dispatch():
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import autograd, sparse_attention
    rng = np.random.default_rng(5)
    m, n, d = 64, 96, 32
    rp, col, val = random_csr(rng, m, n, 20)
    mask = make_csr(rp, col, val, m, n, d)
    mk = lambda r, w: torch.from_numpy(rng.standard_normal((r, w)).astype(np.float32)).to(DEV)
    q, k = mk(m, d), mk(n, d)
    with pytest.raises(ValueError, match="same width"):
        sparse_attention(mask, q, k, mk(n, 64), fused=True)
    with pytest.raises(ValueError, match="dtype"):
        sparse_attention(mask, q, k.half(), mk(n, d), fused=True)
    with pytest.raises(ValueError, match="fused must be"):
        sparse_attention(mask, q, k, mk(n, d), fused="yes")
    # other widths of v, and patterns with very long rows, take the three kernels by themselves
    assert sparse_attention(mask, q, k, mk(n, 64)).shape == (m, 64)
    v = mk(n, d)
    limit = autograd.FUSED_MAX_ROW
    try:
        autograd.FUSED_MAX_ROW = 1
        a = sparse_attention(mask, q, k, v)
    finally:
        autograd.FUSED_MAX_ROW = limit
    b = sparse_attention(mask, q, k, v)
    assert (a - b).abs().max().item() <= 2e-5 * max(1.0, b.abs().max().item())


@pytest.mark.parametrize("half", [False, True])
def test_heads_in_one_launch_match_the_loop_over_heads(half):
    """q, k, v with a leading heads dimension over one mask: the fused kernels take all heads
    in one launch (blockIdx.y); outputs and all three gradients equal those of one call per
    head, bit for bit (the same kernels on the same operands), group plan and rows outside
    groups both present."""
    from gpu_common import DEV, make_csr
    from rode_amd import rode_sddmm_hip, sparse_attention
    from test_gpu_group import _window_matrix
    rng = np.random.default_rng(5)
    m, d, heads = 10000, 64, 3
    n = m + 300
    rp, col, val = _window_matrix(rng, m, n, 160, 8)
    mask = make_csr(rp, col, rng.uniform(0.5, 1.5, len(col)).astype(np.float32), m, n, d, locality=True)
    assert isinstance(mask.plan, rode_sddmm_hip.GroupPlan) and mask.plan.counts[1] >= 2048 and mask.plan.counts[2] > 0
    dt = torch.float16 if half else torch.float32
    mk = lambda r: torch.from_numpy(rng.standard_normal((heads, r, d)).astype(np.float32)).to(DEV, dt)
    q, k, v = mk(m).requires_grad_(), mk(n).requires_grad_(), mk(n).requires_grad_()
    w = mk(m).float()
    out = sparse_attention(mask, q, k, v, fused=True)
    assert out.shape == (heads, m, d)
    (out * w).sum().backward()
    batched = (out.detach().clone(), q.grad.clone(), k.grad.clone(), v.grad.clone())
    for h in range(heads):
        qh, kh, vh = (t[h].detach().clone().requires_grad_() for t in (q, k, v))
        oh = sparse_attention(mask, qh, kh, vh, fused=True)
        (oh * w[h]).sum().backward()
        for got, want in zip(batched, (oh.detach(), qh.grad, kh.grad, vh.grad)):
            assert torch.equal(got[h], want)
    # the three separate kernels take the heads one at a time
    chain = sparse_attention(mask, q.detach(), k.detach(), v.detach(), fused=False)
    tol = 3e-3 if half else 5e-5
    assert (chain - batched[0]).abs().max().item() <= tol * max(1.0, chain.abs().max().item())
    with pytest.raises(ValueError, match="heads"):
        sparse_attention(mask, q, k[:2], v, fused=True)


@pytest.mark.gpu
def test_row_statistics_need_the_per_nonzero_array():
    """The forward entry point writes scores and row statistics together or not at all, and
    wants the statistics 8-byte aligned: both misuses are refused before anything is launched."""
    import ctypes
    from gpu_common import DEV
    from rode_amd import _lib
    lib = _lib.load()
    m = n = 64
    rp = torch.arange(0, 2 * m + 1, 2, dtype=torch.int32, device=DEV)
    col = (torch.arange(2 * m, device=DEV) % n).int()
    val = torch.ones(2 * m, device=DEV)
    q = torch.randn(m, 32, device=DEV)
    out, kept, stats = torch.empty(m, 32, device=DEV), torch.empty(2 * m, device=DEV), torch.empty(m * 2 + 1, device=DEV)
    s = torch.cuda.current_stream(DEV).cuda_stream

    def call(kept_ptr, stats_ptr):
        return lib.rode_hip_attention_forward_batched(_lib.DENSE_CODE["f32"], 1, m, n, 2 * m, 32, rp.data_ptr(), col.data_ptr(),
                                                      val.data_ptr(), q.data_ptr(), q.data_ptr(), q.data_ptr(), 1.0,
                                                      out.data_ptr(), kept_ptr, stats_ptr, None, s)
    assert call(None, stats.data_ptr()) != 0
    assert call(kept.data_ptr(), stats.data_ptr() + 4) != 0
    assert call(kept.data_ptr(), stats.data_ptr()) == 0
    torch.cuda.synchronize()
    assert torch.isfinite(stats[: 2 * m]).all() and (stats[1 : 2 * m : 2] > 0).all()
