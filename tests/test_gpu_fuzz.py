"""Randomised shapes, densities, segment lengths and widths against the CPU oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(24))
def test_random_problem(seed):
    import oracle
    from gpu_common import TOL_F16, TOL_F32, check_csr_decomposition, make_csr, round_half, run_sddmm, run_spmm
    from helpers import random_csr, sddmm_row_l1_errors, spmm_row_l1_error
    rng = np.random.default_rng(9000 + seed)
    m = int(rng.integers(1, 3000))
    n = int(rng.integers(1, 3000))
    mean = int(rng.integers(1, min(n, 120) + 1))
    nlong = int(rng.integers(0, 4))
    seg = int(rng.choice([32, 64, 96, 128, 480, 512, 1024, 4096]))
    k = int(rng.choice([32, 64, 128, 128, 32, 16, 96, 200, 256]))
    half = bool(rng.integers(0, 2)) and k % 8 == 0
    rp, col, val = random_csr(rng, m, n, mean, long_rows=nlong, long_len=max(2, min(n, 2500)),
                              empty_frac=float(rng.choice([0.0, 0.1, 0.5])))
    if seed % 5 == 0:  # every entry of some rows explicitly zero, as padding does
        val[rng.random(len(val)) < 0.2] = 0.0
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    csr = make_csr(rp, col, val, m, n, k, seg)
    check_csr_decomposition(csr, rp)
    tol = TOL_F16 if half else TOL_F32
    lh, rh = (round_half(lhs), round_half(rhs)) if half else (lhs, rhs)

    out = run_sddmm(csr, lhs, rhs, half)
    ref, scale = oracle.sddmm_f64(rp, col, val, lh, rh, with_abs=True)
    err, cond = sddmm_row_l1_errors(out, ref, scale, rp)
    assert float(err[cond <= 100].max(initial=0.0)) <= tol, (seed, m, n, seg, k, half)
    strict = np.abs(out - ref) / np.maximum(scale, 1e-30)
    assert strict.max(initial=0.0) <= (2e-3 if half else 2e-6), (seed, m, n, seg, k, half)

    C = run_spmm(csr, rhs, half)
    assert spmm_row_l1_error(C, oracle.spmm_f64(rp, col, val, rh)) <= tol, (seed, m, n, seg, k, half)
