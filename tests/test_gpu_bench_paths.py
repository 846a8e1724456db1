"""The paths the benchmark measures, under the parity bar of the other GPU tests.

``bench.py`` builds every matrix with the segment length picked from the row lengths
(``config="auto"``) and the plan picked from the pattern (``locality="auto"``), at full size.
Each case here builds the matrix the same way, checks that the decomposition and the plan are
the ones the benchmark table states for that configuration, runs SpMM and SDDMM (and the
fused attention forward on the attention mask) through the Python op / C ABI, and compares a
fixed sample of rows with the fp64 oracle: fp32 operands within 1e-4 of the row's L1 norm,
fp16 operands (fp32 accumulation) within 2e-3, SDDMM additionally per element against the
magnitude of the summed terms and by the rule of the reference's tests
(RoDe_SDDMM/test.cu:221-237) against the reference's fp32 loop (RoDe_SDDMM/main.cu:65-91).
"""
import functools

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

# workload -> (segment length auto_config picks, plan kind locality="auto" keeps)
EXPECTED = {
    "c1_uniform": (128, None),
    "c2_lognormal": (128, None),
    "c3_banded": (512, "window"),
    "c4_powerlaw": (512, "hub"),
    "c5_attention": (1024, "group"),
}

# the rows of the benchmark table: (workload, K, fp16 operands)
CASES = [
    ("c1_uniform", 32, False),
    ("c2_lognormal", 32, False), ("c2_lognormal", 128, False),
    ("c3_banded", 32, False), ("c3_banded", 128, False),
    ("c4_powerlaw", 32, False), ("c4_powerlaw", 64, False), ("c4_powerlaw", 128, False), ("c4_powerlaw", 128, True),
    ("c5_attention", 64, False), ("c5_attention", 64, True),
]


@functools.lru_cache(maxsize=1)  # cases of one workload follow each other; one matrix at a time stays resident
def _bench_matrix(workload):
    from gpu_common import DEV, t
    from rode_amd import RoDeCSR, workloads
    m, n, rp, col, val = workloads.config(workload)
    # exactly what bench.py does with its default flags (--seg 0, no --no-plan)
    csr = RoDeCSR(t(rp), t(col), t(val), DEV, m, n, 128, config="auto", locality="auto")
    return m, n, rp, col, val, csr


def _with_k(csr, k):
    """The same decomposition and plan for another dense width (only the shape checks of
    the ops read ``k``; with config="auto" the decomposition does not depend on it)."""
    from rode_amd import RoDeCSR
    other = object.__new__(RoDeCSR)
    other.__dict__.update(csr.__dict__)
    other.k = k
    return other


def _plan_kind(csr):
    from rode_amd import rode_sddmm_hip
    if csr.plan is None:
        return None
    return {rode_sddmm_hip.WindowPlan: "window", rode_sddmm_hip.HubPlan: "hub", rode_sddmm_hip.GroupPlan: "group"}[type(csr.plan)]


def _sample(rp):
    from test_gpu_sddmm import sample_rows, sub_csr
    rows = sample_rows(rp, np.random.default_rng(12))
    sub_rp, idx = sub_csr(rp, rows)
    return rows, sub_rp, idx


@pytest.mark.parametrize("workload,k,half", CASES, ids=[f"{w}-k{k}-{'f16' if h else 'f32'}" for w, k, h in CASES])
def test_benchmarked_path_against_oracle(workload, k, half):
    import oracle
    from gpu_common import DEV, TOL_F16, TOL_F32, check_csr_decomposition, round_half
    from helpers import reference_error_count, sddmm_row_l1_errors, spmm_row_l1_error
    from rode_amd import rode_sddmm, rode_spmm
    m, n, rp, col, val, base = _bench_matrix(workload)
    seg, kind = EXPECTED[workload]
    assert base.config["seg_length"] == seg, f"auto_config picked {base.config['seg_length']}, the table states {seg}"
    assert _plan_kind(base) == kind, f"locality='auto' kept {_plan_kind(base)}, the table states {kind}"
    if k == 32 or not half:  # (once per workload is enough; cheap against the rest)
        check_csr_decomposition(base, rp)
    csr = _with_k(base, k)
    tol = TOL_F16 if half else TOL_F32
    dt = torch.float16 if half else torch.float32
    g = torch.Generator(device=DEV).manual_seed(300 + k)
    B = torch.randn(n, k, device=DEV, generator=g).to(dt)  # SpMM operand and SDDMM rhs, as in the benchmark
    L = torch.randn(m, k, device=DEV, generator=g).to(dt)
    rows, sub_rp, idx = _sample(rp)
    d_rows, d_idx = torch.from_numpy(rows).to(DEV), torch.from_numpy(idx).to(DEV)
    Bh = B.float().cpu().numpy()  # (fp16 operands: the oracle gets the rounded values)
    Lh = L[d_rows].float().cpu().numpy()

    C = rode_spmm(csr, B)
    refC, scaleC = oracle.spmm_f64(sub_rp, col[idx], val[idx], Bh, with_abs=True)
    gotC = C[d_rows].cpu().numpy()
    err_spmm = spmm_row_l1_error(gotC, refC)
    assert err_spmm <= tol, f"SpMM row-L1 error {err_spmm}"
    assert (np.abs(gotC - refC) / np.maximum(scaleC, 1e-30)).max() <= (2e-3 if half else 2e-6)
    del C

    out = rode_sddmm(csr, L, B)
    ref, scale = oracle.sddmm_f64(sub_rp, col[idx], val[idx], Lh, Bh, with_abs=True)
    got = out[d_idx].cpu().numpy()
    assert np.max(np.abs(got - ref) / np.maximum(scale, 1e-30)) <= (2e-3 if half else 2e-6)
    err, cond = sddmm_row_l1_errors(got, ref, scale, sub_rp)
    assert err[cond <= 100].max(initial=0.0) <= tol
    if not half:
        ref32 = oracle.sddmm_f32(sub_rp, col[idx], val[idx], Lh, Bh)
        assert reference_error_count(got, ref32) == 0
    print(f"{workload} K={k} {'f16' if half else 'f32'} SEG={seg} plan={kind}: {len(rows)} rows / {len(idx)} nnz sampled, "
          f"SpMM {err_spmm:.2e}, SDDMM {err[cond <= 100].max(initial=0.0):.2e} ({int((cond > 100).sum())} rows with condition > 100)")


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_benchmarked_attention_forward_against_host_softmax(half):
    """Configuration 5 at full size through ``sparse_attention(fused=True)`` (4096 kept groups:
    one wave per group) against SDDMM, row softmax and SpMM in fp64 on the host, on sampled rows."""
    import oracle
    from gpu_common import DEV
    from rode_amd import sparse_attention
    m, n, rp, col, val, base = _bench_matrix("c5_attention")
    assert _plan_kind(base) == "group" and base.plan.counts[1] >= 2048
    d = 64
    csr = _with_k(base, d)
    dt = torch.float16 if half else torch.float32
    g = torch.Generator(device=DEV).manual_seed(500)
    q, k, v = (torch.randn(r, d, device=DEV, generator=g).to(dt) for r in (m, n, n))
    out = sparse_attention(csr, q, k, v, fused=True)
    rows, sub_rp, idx = _sample(rp)
    d_rows = torch.from_numpy(rows).to(DEV)
    qh, kh, vh = q[d_rows].float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy()
    sc = oracle.sddmm_f64(sub_rp, col[idx], val[idx], qh, kh) * d ** -0.5
    starts = sub_rp[:-1].astype(np.int64)
    lens = np.diff(sub_rp)
    assert (lens > 0).all()
    mx = np.repeat(np.maximum.reduceat(sc, starts), lens)
    e = np.exp(sc - mx)
    p = e / np.repeat(np.add.reduceat(e, starts), lens)
    ref = oracle.spmm_d(sub_rp, col[idx], p, vh)
    got = out[d_rows].cpu().numpy()
    tol = 2e-3 if half else 2e-5
    assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_benchmarked_attention_training_step_against_dense_autograd(half):
    """Configuration 5 at full size, forward and gradient kernels as ``bench.py --chain --fused
    scores --train`` runs them (group kernels on the mask and on its transpose), against dense
    fp64 autograd on the GPU; a random weight per output element makes every gradient matter."""
    from gpu_common import DEV
    from rode_amd import rode_sddmm_hip, sparse_attention
    m, n, rp, col, val, base = _bench_matrix("c5_attention")
    assert _plan_kind(base) == "group" and base.plan.counts[1] >= 2048
    d = 64
    csr = _with_k(base, d)
    csr_t, _ = csr.transpose(with_values=False)
    assert isinstance(csr_t.plan, rode_sddmm_hip.GroupPlan) and csr_t.plan.counts[1] >= 1024
    dt = torch.float16 if half else torch.float32
    g = torch.Generator(device=DEV).manual_seed(501)
    q, k, v = (torch.randn(r, d, device=DEV, generator=g).to(dt).requires_grad_() for r in (m, n, n))
    w = torch.randn(m, d, device=DEV, generator=g)
    (sparse_attention(csr, q, k, v, fused=True) * w).sum().backward()
    q64, k64, v64 = (x.detach().double().requires_grad_() for x in (q, k, v))
    rows = torch.repeat_interleave(torch.arange(m, device=DEV), torch.from_numpy(np.diff(rp)).to(DEV))
    cols = torch.from_numpy(col).to(DEV).long()
    scores = torch.full((m, n), float("-inf"), dtype=torch.float64, device=DEV)
    weight = torch.zeros((m, n), dtype=torch.float64, device=DEV)
    weight[rows, cols] = torch.from_numpy(val).to(DEV).double()
    logits = (q64 @ k64.t()) * weight * d ** -0.5
    scores = torch.where(weight != 0, logits, scores)
    ((torch.softmax(scores, dim=1) @ v64) * w.double()).sum().backward()
    tol = 3e-3 if half else 2e-5
    for got, want in ((q.grad, q64.grad), (k.grad, k64.grad), (v.grad, v64.grad)):
        assert (got.double() - want).abs().max().item() <= tol * want.abs().max().item()
    del scores, weight, logits
    torch.cuda.empty_cache()


def test_auto_config_longest_segment_length_runs():
    """A matrix for which ``auto_config`` returns its largest segment length, 2048 (enough
    segments, 90th percentile of the rows with block segments above 1024), through both ops."""
    import oracle
    from gpu_common import DEV, TOL_F32, check_csr_decomposition, t
    from helpers import sddmm_row_l1_errors, spmm_row_l1_error
    from rode_amd import RoDeCSR, rode_sddmm, rode_spmm
    rng = np.random.default_rng(31)
    m, n, k = 12000, 6000, 64
    lens = rng.choice([5, 40, 700, 1500, 2100, 3000], size=m, p=[.1, .1, .2, .3, .2, .1])
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    csr = RoDeCSR(t(rp), t(col), t(val), DEV, m, n, k, config="auto", locality="auto")
    assert csr.config["seg_length"] == 2048
    check_csr_decomposition(csr, rp)
    B = rng.standard_normal((n, k)).astype(np.float32)
    L = rng.standard_normal((m, k)).astype(np.float32)
    C = rode_spmm(csr, t(B).to(DEV)).cpu().numpy()
    assert spmm_row_l1_error(C, oracle.spmm_f64(rp, col, val, B)) <= TOL_F32
    out = rode_sddmm(csr, t(L).to(DEV), t(B).to(DEV)).cpu().numpy()
    ref, scale = oracle.sddmm_f64(rp, col, val, L, B, with_abs=True)
    assert np.max(np.abs(out - ref) / np.maximum(scale, 1e-30)) <= 2e-6
    err, cond = sddmm_row_l1_errors(out, ref, scale, rp)
    assert err[cond <= 100].max() <= TOL_F32
