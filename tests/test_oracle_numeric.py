"""Pins the numeric half of the oracle.  oracle.sddmm_f32 restates the
reference's own CPU check (RoDe_SDDMM/main.cu:65-91); oracle.spmm_* is the
textbook CSR product (the reference has no CPU SpMM).  Checked against fp64
numpy einsum / scipy.sparse (library routines), closed-form special cases and a
pure-Python brute force on tiny inputs."""
import numpy as np
import pytest

import oracle
from helpers import random_csr, sddmm_numpy64, spmm_scipy64


@pytest.mark.parametrize("k", [32, 64, 128, 20])
def test_sddmm_against_numpy(k):
    rng = np.random.default_rng(k)
    m, n = 300, 257
    rp, col, val = random_csr(rng, m, n, 30, long_rows=3, long_len=250)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    ref = sddmm_numpy64(rp, col, val, lhs, rhs)
    got64, scale = oracle.sddmm_f64(rp, col, val, lhs, rhs, with_abs=True)
    np.testing.assert_allclose(got64, ref, rtol=1e-12, atol=1e-12)
    got32 = oracle.sddmm_f32(rp, col, val, lhs, rhs)
    assert np.all(np.abs(got32 - ref) <= 4e-7 * k * scale + 1e-30)  # fp32 left-to-right summation bound
    np.testing.assert_array_equal(oracle.sddmm_f32(rp, col, val, lhs, rhs, threads=4), got32)


def test_sddmm_special_cases():
    rng = np.random.default_rng(0)
    m, n, k = 64, 50, 32
    rp, col, val = random_csr(rng, m, n, 10)
    ones_l, ones_r = np.ones((m, k), np.float32), np.ones((n, k), np.float32)
    np.testing.assert_array_equal(oracle.sddmm_f32(rp, col, val, ones_l, ones_r), (val * np.float32(k)))
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    assert not oracle.sddmm_f32(rp, col, np.zeros_like(val), lhs, rhs).any()
    # one-hot lhs rows pick one rhs entry: out = val * rhs[col, j]
    j = 5
    onehot = np.zeros((m, k), np.float32); onehot[:, j] = 1
    np.testing.assert_array_equal(oracle.sddmm_f32(rp, col, val, onehot, rhs), val * rhs[col, j])
    # operands are not interchangeable: lhs is indexed by row, rhs by column
    sq_rp, sq_col, sq_val = random_csr(rng, 40, 40, 6)
    a = rng.standard_normal((40, k)).astype(np.float32)
    b = rng.standard_normal((40, k)).astype(np.float32)
    assert not np.allclose(oracle.sddmm_f32(sq_rp, sq_col, sq_val, a, b), oracle.sddmm_f32(sq_rp, sq_col, sq_val, b, a))


def test_sddmm_brute_force_tiny():
    rp = np.array([0, 2, 2, 5], np.int32)
    col = np.array([1, 3, 0, 2, 3], np.int32)
    val = np.array([0.5, -2.0, 1.0, 3.0, -1.0], np.float32)
    lhs = np.arange(12, dtype=np.float32).reshape(3, 4) / 4
    rhs = (np.arange(16, dtype=np.float32).reshape(4, 4) - 7) / 8
    want = []
    for r in range(3):
        for idx in range(rp[r], rp[r + 1]):
            want.append(float(val[idx]) * sum(float(lhs[r, t]) * float(rhs[col[idx], t]) for t in range(4)))
    np.testing.assert_allclose(oracle.sddmm_f32(rp, col, val, lhs, rhs), want, rtol=1e-6)


@pytest.mark.parametrize("n", [32, 64, 128, 48])
def test_spmm_against_scipy(n):
    rng = np.random.default_rng(n)
    m, k = 300, 211
    rp, col, val = random_csr(rng, m, k, 25, long_rows=3, long_len=200)
    B = rng.standard_normal((k, n)).astype(np.float32)
    ref = spmm_scipy64(rp, col, val, B, m, k)
    got64, scale = oracle.spmm_f64(rp, col, val, B, with_abs=True)
    np.testing.assert_allclose(got64, ref, rtol=1e-12, atol=1e-12)
    got32 = oracle.spmm_f32(rp, col, val, B)
    assert np.all(np.abs(got32 - ref) <= 4e-7 * 300 * scale + 1e-30)
    np.testing.assert_array_equal(oracle.spmm_f32(rp, col, val, B, threads=4), got32)


def test_spmm_special_cases():
    rng = np.random.default_rng(1)
    m, k, n = 80, 80, 32
    rp, col, val = random_csr(rng, m, k, 12, empty_frac=0.3)
    # B = 1 -> row sums in every column
    got = oracle.spmm_f64(rp, col, val, np.ones((k, n), np.float32))
    sums = np.array([val[rp[r]:rp[r + 1]].astype(np.float64).sum() for r in range(m)])
    np.testing.assert_allclose(got, np.repeat(sums[:, None], n, 1), rtol=1e-12, atol=1e-15)
    # identity pattern -> C = diag(val) * B
    B = rng.standard_normal((k, n)).astype(np.float32)
    d = rng.uniform(-1, 1, k).astype(np.float32)
    got = oracle.spmm_f32(np.arange(k + 1, dtype=np.int32), np.arange(k, dtype=np.int32), d, B)
    np.testing.assert_array_equal(got, d[:, None] * B)
    # empty rows are written as zeros; linearity in B
    C = oracle.spmm_f64(rp, col, val, B)
    assert not C[np.diff(rp) == 0].any()
    B2 = rng.standard_normal((k, n)).astype(np.float32)
    lin = oracle.spmm_f64(rp, col, val, B) + oracle.spmm_f64(rp, col, val, B2)
    both = oracle.spmm_f64(rp, col, val, (B.astype(np.float64) + B2).astype(np.float32))
    np.testing.assert_allclose(both, lin, rtol=1e-5, atol=1e-5)
    # transposed operand would fail: a permutation pattern moves rows of B, not columns
    perm = rng.permutation(k).astype(np.int32)
    got = oracle.spmm_f32(np.arange(k + 1, dtype=np.int32), perm, np.ones(k, np.float32), B)
    np.testing.assert_array_equal(got, B[perm])


def test_spmm_double_against_scipy():
    import scipy.sparse as sp
    rng = np.random.default_rng(3)
    m, k, n = 200, 150, 64
    rp, col, val = random_csr(rng, m, k, 20, long_rows=2, long_len=140)
    val64 = rng.uniform(-1, 1, len(val))
    B = rng.standard_normal((k, n))
    ref = sp.csr_matrix((val64, col, rp), shape=(m, k)) @ B
    np.testing.assert_allclose(oracle.spmm_d(rp, col, val64, B), ref, rtol=1e-13, atol=1e-13)
