"""GPU parity tests of the locality plan and the window kernels (chunks of the residue
list whose dense rows fit an LDS window): the planned entry points against the fp64 oracle
and against the same call without a plan, through the Python op (ctypes over the C ABI)."""
import numpy as np
import pytest
import torch

import oracle
from gpu_common import DEV, TOL_F16, TOL_F32, round_half, t
from rode_amd import RoDeCSR, rode_sddmm, rode_spmm, workloads

pytestmark = pytest.mark.gpu


def banded(rows, cols, per_row, band, seed, far=0, long_every=0, long_len=0, empty_every=0):
    """Rows with `per_row` distinct columns inside a band around the diagonal, `far` more
    anywhere (outside the window), every `long_every`-th row `long_len` columns long (it gets
    block segments and a tail), every `empty_every`-th row empty."""
    rng = np.random.default_rng(seed)
    cols_of = []
    for r in range(rows):
        if empty_every and r % empty_every == empty_every - 1:
            cols_of.append(np.empty(0, dtype=np.int64))
            continue
        want = long_len if long_every and r % long_every == 0 else per_row
        centre = int(r * (cols - 1) / max(rows - 1, 1))
        lo, hi = max(0, centre - band // 2), min(cols, centre + band // 2)
        pick = rng.choice(np.arange(lo, hi), size=min(want, hi - lo), replace=False)
        if far:
            pick = np.concatenate([pick, rng.integers(0, cols, far)])
        cols_of.append(np.unique(pick))
    lens = np.array([len(c) for c in cols_of])
    row_ptr = np.zeros(rows + 1, dtype=np.int32)
    row_ptr[1:] = np.cumsum(lens)
    col = np.concatenate(cols_of).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(np.float32)
    return row_ptr, col, val


def both(row_ptr, col, val, m, n, k):
    planned = RoDeCSR(t(row_ptr), t(col), t(val), DEV, m, n, k, locality=True)
    plain = RoDeCSR(t(row_ptr), t(col), t(val), DEV, m, n, k, locality=False)
    return planned, plain


def check_products(row_ptr, col, val, m, n, k, half=False, expect_plan=True):
    planned, plain = both(row_ptr, col, val, m, n, k)
    assert (planned.plan is not None) == expect_plan
    assert plain.plan is None
    rng = np.random.default_rng(17)
    B = rng.standard_normal((n, k)).astype(np.float32)
    L = rng.standard_normal((m, k)).astype(np.float32)
    dt = torch.float16 if half else torch.float32
    Bd, Ld = t(B).to(DEV, dt), t(L).to(DEV, dt)
    if half:
        B, L = round_half(B), round_half(L)
    tol = TOL_F16 if half else TOL_F32
    c64 = oracle.spmm_f64(row_ptr, col, val, B)
    l1 = np.maximum(np.abs(c64).sum(axis=1), 1e-30)
    o64, scale = oracle.sddmm_f64(row_ptr, col, val, L, B, with_abs=True)
    for csr in (planned, plain):
        C = rode_spmm(csr, Bd).cpu().numpy()
        assert np.max(np.abs(C - c64).max(axis=1) / l1) <= tol
        out = rode_sddmm(csr, Ld, Bd).cpu().numpy()
        # per element against the magnitude of the summed terms (strict for any row)
        assert np.max(np.abs(out - o64) / np.maximum(scale, 1e-30)) <= (2e-3 if half else 2e-6)
    return planned


def test_plan_of_a_banded_matrix_has_a_window_on_every_chunk():
    m, n, rp, col, val = workloads.config("c3_banded", 0.01)
    csr = RoDeCSR(t(rp), t(col), t(val), DEV, m, n, 128, locality=True)
    assert csr.m1 == 0 and csr.plan is not None
    d = csr.plan.descriptors()
    assert len(d) == (csr.m2 + 127) // 128 == csr.plan.counts[0] == csr.plan.counts[1]
    assert (d[:, 1] > 0).all() and (d[:, 1] <= 512).all()
    assert (d[:, 3] == 0).all()                            # every nonzero inside its chunk's window
    assert int(d[:, 2].sum()) == int(rp[-1])               # the residue list holds every nonzero here
    rows = np.arange(len(d)) * 128
    assert (d[:, 0] <= rows + 128).all() and (d[:, 0] + d[:, 1] >= rows - 128).all()  # windows follow the diagonal
    assert (d[:, 0] >= 0).all() and (d[:, 0] + d[:, 1] <= n).all()


def test_plan_of_scattered_columns_has_no_window():
    m, n, rp, col, val = workloads.config("c2_lognormal", 0.1)
    assert RoDeCSR(t(rp), t(col), t(val), DEV, m, n, 128, locality=True).plan is None
    # "auto" also drops a plan that covers too few chunks to be worth two more launches
    m, n, rp, col, val = workloads.config("c3_banded", 0.01)
    assert RoDeCSR(t(rp), t(col), t(val), DEV, m, n, 128).plan is None


@pytest.mark.parametrize("k,half", [(128, False), (64, False), (256, False), (200, False), (36, False), (128, True),
                                    (72, True), (32, False)])
def test_banded_matrix_planned_against_oracle(k, half):
    # 36 and 200: partial last tile; 32 fp32 / 64 fp16 and narrower: one tile, the plan is ignored by the kernels
    m, n, rp, col, val = workloads.config("c3_banded", 0.004)
    check_products(rp, col, val, m, n, k, half)


def test_rows_with_segments_tails_far_columns_and_empty_rows():
    # long rows (block segments + tails in the residue list, summed whole by the block kernel
    # under the whole-lists promise when there are many segments), columns outside the window,
    # empty rows with an unaligned start, a last chunk that is not full
    m = n = 3000
    rp, col, val = banded(m, n, 21, 200, seed=5, far=2, long_every=97, long_len=150, empty_every=13)
    csr = check_products(rp, col, val, m, n, 128)
    d = csr.plan.descriptors()
    win = d[d[:, 1] > 0]
    assert len(win) > 0 and (win[:, 3] > 0).any()           # some slots are outside their window
    check_products(rp, col, val, m, n, 64, half=False)
    check_products(rp, col, val, m, n, 128, half=True)


def test_window_clipped_at_the_matrix_edges_and_rectangular_operand():
    m, n = 2000, 700  # the band runs from column 0 to column n - 1
    rp, col, val = banded(m, n, 17, 300, seed=9)
    check_products(rp, col, val, m, n, 128)


def test_non_finite_dense_rows_stay_in_the_rows_that_reference_them():
    m = n = 1500
    rp, col, val = banded(m, n, 15, 120, seed=3, far=1)
    planned, plain = both(rp, col, val, m, n, 128)
    assert planned.plan is not None
    B = torch.randn(n, 128, device=DEV)
    bad = [0, 7, 640, n - 1]
    B[bad] = float("inf")
    touched = np.zeros(m, dtype=bool)
    rows = np.repeat(np.arange(m), np.diff(rp))
    touched[rows[np.isin(col, bad)]] = True
    for csr in (planned, plain):
        C = rode_spmm(csr, B).cpu().numpy()
        assert np.isfinite(C[~touched]).all()
        assert (~np.isfinite(C[touched])).any(axis=1).all()


def test_values_replaced_per_call_and_gradients_use_the_plan():
    m = n = 2048
    rp, col, val = banded(m, n, 19, 160, seed=11)
    planned, plain = both(rp, col, val, m, n, 64)
    assert planned.plan is not None and planned.with_values(planned.values * 2).plan is planned.plan
    L = torch.randn(m, 64, device=DEV, requires_grad=True)
    R = torch.randn(n, 64, device=DEV, requires_grad=True)
    outs = []
    for csr in (planned, plain):
        L.grad = R.grad = None
        s = rode_sddmm(csr, L, R)
        C = rode_spmm(csr, R, values=s)
        C.square().sum().backward()
        outs.append((s.detach().clone(), C.detach().clone(), L.grad.clone(), R.grad.clone()))
    for a, b in zip(*outs):
        assert torch.allclose(a, b, rtol=2e-4, atol=2e-4 * float(b.abs().max()))


def test_full_size_banded_configuration_planned():
    # configuration 3 at full size, K = 128: linearity and a row sample against the oracle
    m, n, rp, col, val = workloads.config("c3_banded", 1.0)
    csr = RoDeCSR(t(rp), t(col), t(val), DEV, m, n, 128)
    assert csr.plan is not None and csr.plan.counts[0] == csr.plan.counts[1]
    rng = np.random.default_rng(23)
    B = rng.standard_normal((n, 128)).astype(np.float32)
    L = rng.standard_normal((m, 128)).astype(np.float32)
    Bd, Ld = t(B).to(DEV), t(L).to(DEV)
    C = rode_spmm(csr, Bd)
    out = rode_sddmm(csr, Ld, Bd)
    sample = np.unique(np.concatenate([np.arange(0, 300), rng.integers(0, m, 400), np.arange(m - 300, m)]))
    idx = np.concatenate([np.arange(rp[r], rp[r + 1]) for r in sample])
    srp = np.zeros(len(sample) + 1, dtype=np.int32)
    srp[1:] = np.cumsum(rp[sample + 1] - rp[sample])
    c64 = oracle.spmm_f64(srp, col[idx], val[idx], B)
    l1 = np.maximum(np.abs(c64).sum(axis=1), 1e-30)
    assert np.max(np.abs(C[sample].cpu().numpy() - c64).max(axis=1) / l1) <= TOL_F32
    o64, scale = oracle.sddmm_f64(srp, col[idx], val[idx], L[sample], B, with_abs=True)
    assert np.max(np.abs(out.cpu().numpy()[idx] - o64) / np.maximum(scale, 1e-30)) <= 2e-6
    # linearity in the dense operand (exact property at any size)
    C2 = rode_spmm(csr, 2 * Bd)
    assert torch.equal(C2, 2 * C)
