"""SpMM parity on the GPU, through the Python op and the C ABI.  The reference has
no SpMM test or CPU SpMM; the oracle is the textbook CSR product in fp64
(oracle.spmm_f64, pinned by scipy.sparse), judged with the row-L1-normalised
bound: 1e-4 for fp32 B, 2e-3 for fp16 B with fp32 accumulation."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _check(csr, rp, col, val, B, half=False):
    import oracle
    from gpu_common import TOL_F16, TOL_F32, check_csr_decomposition, round_half, run_spmm
    from helpers import spmm_row_l1_error
    check_csr_decomposition(csr, rp)
    C = run_spmm(csr, B, half)
    assert C.shape == (csr.m, B.shape[1]) and C.dtype == np.float32
    if half:
        B = round_half(B)
    ref64, scale = oracle.spmm_f64(rp, col, val, B, with_abs=True)
    err = spmm_row_l1_error(C, ref64)
    assert err <= (TOL_F16 if half else TOL_F32), f"row-L1 error {err}"
    if not half:
        strict = np.abs(C - ref64) / np.maximum(scale, 1e-30)
        assert strict.max(initial=0.0) <= 2e-6, f"per-element error {strict.max()}"
    return err


@pytest.mark.parametrize("n", [32, 64, 128, 96, 256])
@pytest.mark.parametrize("seg", [32, 512])
def test_unpadded_rows(n, seg):
    from gpu_common import make_csr
    from helpers import random_csr
    rng = np.random.default_rng(100 * n + seg)
    m, k = 1500, 1333
    rp, col, val = random_csr(rng, m, k, 37, long_rows=6, long_len=1300, empty_frac=0.15)
    B = rng.standard_normal((k, n)).astype(np.float32)
    _check(make_csr(rp, col, val, m, k, 32, seg), rp, col, val, B)


@pytest.mark.parametrize("n", [4, 8, 20, 36, 72, 100, 160, 200, 264])
def test_any_width(n):
    """Widths beyond the reference's multiples of 32: any multiple of 4 (the partial last
    tile is guarded; the columns next to it must stay untouched)."""
    import oracle
    from gpu_common import DEV, make_csr
    from helpers import random_csr, spmm_row_l1_error
    from rode_amd import rode_spmm
    rng = np.random.default_rng(n)
    m, k = 600, 650
    rp, col, val = random_csr(rng, m, k, 35, long_rows=4, long_len=600, empty_frac=0.1)
    B = rng.standard_normal((k, n)).astype(np.float32)
    csr = make_csr(rp, col, val, m, k, 32)
    _check(csr, rp, col, val, B)
    if n % 8 == 0:
        _check(csr, rp, col, val, B, half=True)
    assert rode_spmm(csr, torch.from_numpy(B).to(DEV)).shape == (m, n)
    # an fp64 run of the same width (vector of 2)
    from rode_amd import rode_sddmm_hip
    C64 = rode_sddmm_hip.spmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                      csr.row_offsets, csr.column_indices, csr.values.double(), m, k,
                                      torch.from_numpy(B).to(DEV).double()).cpu().numpy()
    ref = oracle.spmm_f64(rp, col, val, B)
    assert spmm_row_l1_error(C64, ref) <= 1e-12


def test_edge_tile_does_not_write_past_the_row():
    """C is (m, n) with n = 36: the second 32-wide tile has 4 live columns.  A canary row
    appended after C and the next row's first columns must be unchanged / correct."""
    import oracle
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(77)
    m, k, n = 300, 320, 36
    rp, col, val = random_csr(rng, m, k, 40, long_rows=3, long_len=300)
    B = rng.standard_normal((k, n)).astype(np.float32)
    csr = make_csr(rp, col, val, m, k, 32)
    buf = torch.zeros((m + 1) * n, device=DEV)
    buf[m * n:] = 123.0
    out = buf[: m * n].view(m, n)
    rode_sddmm_hip.spmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                csr.row_offsets, csr.column_indices, csr.values, m, k, torch.from_numpy(B).to(DEV),
                                out=out)
    assert (buf[m * n:] == 123.0).all()
    ref = oracle.spmm_f64(rp, col, val, B)
    assert np.abs(out.cpu().numpy() - ref).max() <= 1e-4 * np.abs(ref).sum(axis=1).max()


def test_padded_reference_matrices():
    """The reference generators' matrices (rows padded to 4 with explicit zeros)."""
    from gpu_common import make_csr
    from rode_amd import workloads
    for m, k, per_row, n in [(63, 67, 10, 32), (1023, 1031, 65, 128), (31, 4097, 200, 64), (1000, 1, 1, 32),
                             (1, 1000, 100, 128), (2048, 2048, 128, 64), (1024, 1024, 512, 32)]:
        rp, col, val = workloads.reference_csr(m, k, per_row, poisson=True)
        B = workloads.reference_dense(k, n, 456)
        _check(make_csr(rp, col, val, m, k, 32, 512), rp, col, val, B)


@pytest.mark.parametrize("n", [32, 64, 128])
def test_fp16_dense(n):
    from gpu_common import make_csr
    from helpers import random_csr
    rng = np.random.default_rng(n)
    m, k = 900, 1200
    rp, col, val = random_csr(rng, m, k, 50, long_rows=4, long_len=1100)
    B = rng.standard_normal((k, n)).astype(np.float32)
    for seg in (32, 512):
        _check(make_csr(rp, col, val, m, k, 32, seg), rp, col, val, B, half=True)


@pytest.mark.parametrize("n", [32, 64, 128, 96])
def test_fp64(n):
    """The double overloads (RoDeSpmm.h:10-14): fp64 values, B and C; bound 1e-12 of the row's L1 norm."""
    import oracle
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(n)
    m, k = 1100, 900
    rp, col, val = random_csr(rng, m, k, 41, long_rows=5, long_len=850, empty_frac=0.1)
    val64 = rng.uniform(-1, 1, len(val))
    B = rng.standard_normal((k, n))
    for seg in (32, 512):
        csr = make_csr(rp, col, val, m, k, 32, seg)
        C = rode_sddmm_hip.spmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                        csr.row_offsets, csr.column_indices, torch.from_numpy(val64).to(DEV), m, k,
                                        torch.from_numpy(B).to(DEV)).cpu().numpy()
        assert C.dtype == np.float64
        ref = oracle.spmm_d(rp, col, val64, B)
        l1 = np.abs(ref).sum(axis=1)
        assert (np.abs(C - ref).max(axis=1) <= 1e-12 * np.maximum(l1, 1e-300) + 1e-300).all()
        assert not C[np.diff(rp) == 0].any()
    with pytest.raises(RuntimeError, match="float64"):
        rode_sddmm_hip.spmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                    csr.row_offsets, csr.column_indices, csr.values, m, k, torch.from_numpy(B).to(DEV))


def test_fp64_cxx_overloads():
    """RoDeSpmm_n32(double) / RoDeSpmm_n128(double) through their mangled names."""
    import oracle
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    rng = np.random.default_rng(21)
    m, k = 700, 640
    rp, col, val = random_csr(rng, m, k, 45, long_rows=3, long_len=600)
    val64 = rng.uniform(-1, 1, len(val))
    csr = make_csr(rp, col, val, m, k, 32, 512)
    dv = torch.from_numpy(val64).to(DEV)
    for mangled, width in [("_Z12RoDeSpmm_n32iiiiPKdPKiS2_S2_S2_S2_S0_PdP12ihipStream_tS5_", 32),
                           ("_Z13RoDeSpmm_n128iiiiPKdPKiS2_S2_S2_S2_S0_PdP12ihipStream_tS5_", 64)]:
        fn = getattr(lib, mangled)
        fn.restype = None
        fn.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p] * 10
        B = rng.standard_normal((k, width))
        dB = torch.from_numpy(B).to(DEV)
        C = torch.zeros(m, width, dtype=torch.float64, device=DEV)
        torch.cuda.synchronize()
        fn(csr.m1, csr.m2, k, width, dv.data_ptr(), csr.column_indices.data_ptr(), csr.row_offsets.data_ptr(),
           csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(), dB.data_ptr(),
           C.data_ptr(), None, None)
        torch.cuda.synchronize()
        np.testing.assert_allclose(C.cpu().numpy(), oracle.spmm_d(rp, col, val64, B), rtol=1e-11, atol=1e-11)


def test_special_cases_and_edges():
    from gpu_common import DEV, make_csr, run_spmm
    from helpers import random_csr
    from rode_amd import rode_spmm
    rng = np.random.default_rng(4)
    m, k, n = 800, 700, 64
    rp, col, val = random_csr(rng, m, k, 45, long_rows=3, long_len=650, empty_frac=0.2)
    csr = make_csr(rp, col, val, m, k, 32, 512)
    # B = 1 -> every column holds the row sums
    C = run_spmm(csr, np.ones((k, n), np.float32))
    sums = np.array([val[rp[r]:rp[r + 1]].astype(np.float64).sum() for r in range(m)])
    assert np.abs(C - sums[:, None]).max() < 1e-4 and (C == C[:, :1]).all()
    assert not C[np.diff(rp) == 0].any()
    # permutation pattern with unit values moves rows of B exactly
    perm = rng.permutation(k).astype(np.int32)
    B = rng.standard_normal((k, n)).astype(np.float32)
    pcsr = make_csr(np.arange(k + 1, dtype=np.int32), perm, np.ones(k, np.float32), k, k, 32, 512)
    np.testing.assert_array_equal(run_spmm(pcsr, B), B[perm])
    # a non-finite B row must only reach the rows that reference it (the head slots
    # of an unaligned segment belong to the previous row and are skipped, not multiplied by 0)
    B[0, :] = np.inf
    bad = int(col[rp[17]])
    B[bad, 5] = np.nan
    C = run_spmm(csr, B)
    touches = np.array([np.isin([0, bad], col[rp[r]:rp[r + 1]]).any() for r in range(m)])
    assert np.isfinite(C[~touches]).all() and (~np.isfinite(C[touches])).any(axis=1).all()
    # accumulate-in-place semantics of the reference kernels: rows with >= 32 aligned
    # slots add to C, shorter rows overwrite, empty rows are left alone
    B = rng.standard_normal((k, n)).astype(np.float32)
    base = run_spmm(csr, B)
    pre = torch.full((m, n), 2.0, device=DEV)
    got = rode_spmm(csr, torch.from_numpy(B).to(DEV), out=pre).cpu().numpy()
    aligned = np.diff(rp) + rp[:-1] % 4
    adds = aligned >= 32
    # an empty row whose offset is a multiple of 4 is in no list; one at another offset is a zero-slot residue
    keeps = (np.diff(rp) == 0) & (rp[:-1] % 4 == 0)
    np.testing.assert_allclose(got[adds], base[adds] + 2.0, rtol=1e-5, atol=1e-5)
    np.testing.assert_array_equal(got[~adds & ~keeps], base[~adds & ~keeps])
    assert (got[keeps] == 2.0).all()
    # empty matrix
    empty = make_csr(np.zeros(6, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), 5, 7, 32)
    assert not rode_spmm(empty, torch.ones(7, 32, device=DEV)).any()
    # width not a multiple of 32
    with pytest.raises(ValueError):
        rode_spmm(csr, torch.zeros(k, 42, device=DEV))
    with pytest.raises(ValueError):
        rode_spmm(csr, torch.zeros(k + 1, 32, device=DEV))


def test_cxx_reference_signature_entry_points():
    """RoDeSpmm_n32 / RoDeSpmm_n128 / RoDeSDDMM_n32 / RoDeSDDMM_n128 with the reference's
    signatures (RoDeSpmm.h:4-8, RoDeSddmm.h:4-9), called through their mangled names
    on two side streams, as a C++ caller would."""
    import oracle
    from gpu_common import DEV, make_csr
    from helpers import random_csr, sddmm_row_l1_error, spmm_row_l1_error
    from rode_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    rng = np.random.default_rng(11)
    m, ncols = 1200, 1100
    rp, col, val = random_csr(rng, m, ncols, 40, long_rows=5, long_len=1000)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for name, mangled, width in [("spmm", "_Z12RoDeSpmm_n32iiiiPKfPKiS2_S2_S2_S2_S0_PfP12ihipStream_tS5_", 32),
                                 ("spmm", "_Z13RoDeSpmm_n128iiiiPKfPKiS2_S2_S2_S2_S0_PfP12ihipStream_tS5_", 128),
                                 ("sddmm", "_Z13RoDeSDDMM_n32iiiiPKiS0_S0_S0_S0_PKfS2_S2_PfP12ihipStream_tS5_", 32),
                                 ("sddmm", "_Z14RoDeSDDMM_n128iiiiPKiS0_S0_S0_S0_PKfS2_S2_PfP12ihipStream_tS5_", 128)]:
        fn = getattr(lib, mangled)
        fn.restype = None
        fn.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p] * 11 if name == "sddmm" else \
            [ctypes.c_int] * 4 + [ctypes.c_void_p] * 10
        seg = 32 if (name == "sddmm" and width == 128) else 512  # the reference's parameter sets
        csr = make_csr(rp, col, val, m, ncols, 32, seg)
        if name == "spmm":
            B = rng.standard_normal((ncols, width)).astype(np.float32)
            dB = torch.from_numpy(B).to(DEV)
            C = torch.zeros(m, width, device=DEV)
            torch.cuda.synchronize()
            fn(csr.m1, csr.m2, ncols, width, csr.values.data_ptr(), csr.column_indices.data_ptr(),
               csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(),
               csr.st_offsets.data_ptr(), dB.data_ptr(), C.data_ptr(), s1.cuda_stream, s2.cuda_stream)
            torch.cuda.synchronize()
            assert spmm_row_l1_error(C.cpu().numpy(), oracle.spmm_f64(rp, col, val, B)) <= 1e-4
        else:
            lhs = rng.standard_normal((m, width)).astype(np.float32)
            rhs = rng.standard_normal((ncols, width)).astype(np.float32)
            dl, dr = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)
            out = torch.full((len(val),), float("nan"), device=DEV)
            torch.cuda.synchronize()
            fn(csr.m1, csr.m2, ncols, width, csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(),
               csr.st_offsets.data_ptr(), csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(),
               csr.values.data_ptr(), dl.data_ptr(), dr.data_ptr(), out.data_ptr(), s1.cuda_stream, s2.cuda_stream)
            torch.cuda.synchronize()
            assert sddmm_row_l1_error(out.cpu().numpy(), oracle.sddmm_f64(rp, col, val, lhs, rhs), rp) <= 1e-4


@pytest.mark.parametrize("name,n", [("c1_uniform", 32), ("c2_lognormal", 32), ("c2_lognormal", 128)])
def test_benchmark_configs_against_oracle(name, n):
    from gpu_common import make_csr
    from rode_amd import workloads
    m, k, rp, col, val = workloads.config(name)
    B = np.random.default_rng(5000 + n).standard_normal((k, n)).astype(np.float32)
    for seg in (512, 32):
        _check(make_csr(rp, col, val, m, k, 32, seg), rp, col, val, B)


@pytest.mark.parametrize("name,n,half", [("c3_banded", 128, False), ("c4_powerlaw", 64, False),
                                         ("c5_attention", 64, False), ("c5_attention", 64, True)])
def test_large_configs_scaled_against_oracle(name, n, half):
    from gpu_common import make_csr
    from rode_amd import workloads
    scale = {"c3_banded": 1 / 16, "c4_powerlaw": 1 / 16, "c5_attention": 1 / 4}[name]
    m, k, rp, col, val = workloads.config(name, scale)
    B = np.random.default_rng(6000 + n).standard_normal((k, n)).astype(np.float32)
    _check(make_csr(rp, col, val, m, k, 32, 512), rp, col, val, B, half=half)


@pytest.mark.parametrize("name,n", [("c3_banded", 128), ("c4_powerlaw", 128), ("c4_powerlaw", 64), ("c5_attention", 64)])
def test_full_size_properties(name, n):
    """Full benchmark sizes through size-independent facts: B = 1 gives the row sums
    (checked against a segmented fp64 sum), the result is linear in B, and a checksum
    of C equals the checksum computed from column sums of the pattern."""
    from gpu_common import DEV, make_csr
    from rode_amd import rode_spmm, workloads
    m, k, rp, col, val = workloads.config(name)
    csr = make_csr(rp, col, val, m, k, 32, 512)
    C = rode_spmm(csr, torch.ones(k, n, device=DEV))
    nonempty = np.nonzero(np.diff(rp) > 0)[0]
    sums = np.zeros(m)
    sums[nonempty] = np.add.reduceat(val.astype(np.float64), rp[nonempty].astype(np.int64))
    abs_sums = np.zeros(m)
    abs_sums[nonempty] = np.add.reduceat(np.abs(val.astype(np.float64)), rp[nonempty].astype(np.int64))
    # every column holds the same sum (atomic accumulation order may differ per column)
    dsums = torch.from_numpy(sums).to(DEV)[:, None]
    dabs = torch.from_numpy(np.maximum(abs_sums, 1e-30)).to(DEV)[:, None]
    assert ((C.double() - dsums).abs() / dabs).max().item() <= 1e-5
    del C
    # checksum of checksums: sum_r C[r, j] = sum_c w[c] * B[c, j] with w = column sums of A
    g = torch.Generator(device=DEV).manual_seed(n)
    B = torch.randn(k, n, device=DEV, generator=g)
    C = rode_spmm(csr, B)
    w = np.bincount(col, weights=val.astype(np.float64), minlength=k)
    want = torch.from_numpy(w).to(DEV) @ B.double()
    wabs = torch.from_numpy(np.bincount(col, weights=np.abs(val.astype(np.float64)), minlength=k)).to(DEV) @ B.double().abs()
    assert ((C.double().sum(0) - want).abs() / wabs).max().item() < 1e-5
    # linearity
    B2 = torch.randn(k, n, device=DEV, generator=g)
    C2 = rode_spmm(csr, B2)
    C12 = rode_spmm(csr, B + B2)
    denom = torch.from_numpy(abs_sums).to(DEV).float()[:, None] * 8 + 1e-20
    assert ((C12 - (C + C2)).abs() / denom).max().item() < 1e-4


def test_dense_operand_beyond_2_gib():
    """B and rhs of 2.4 GB: byte offsets col * n * 4 exceed 2^31, where the reference's
    32-bit offset arithmetic (RoDeSpmm.cu:153,287) overflows.  Checked on the rows'
    exact expected values: B[c, j] = (c % 1000) + j / 256 is exactly representable."""
    from gpu_common import DEV, make_csr
    from rode_amd import rode_sddmm, rode_spmm
    rng = np.random.default_rng(31)
    m, n, k = 2000, 4_700_000, 128
    lens = rng.integers(0, 90, m)
    lens[7] = 3000
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens]).astype(np.int32)
    col[rp[7 + 1] - 1] = n - 1  # the very last dense row
    val = np.ones(len(col), np.float32)
    csr = make_csr(rp, col, val, m, n, k)
    B = (torch.arange(n, device=DEV) % 1000).float()[:, None] + torch.arange(k, device=DEV).float()[None, :] / 256
    assert B.numel() * 4 > 2**31
    C = rode_spmm(csr, B).cpu().numpy().astype(np.float64)
    colsum = np.zeros(m)
    nonempty = np.nonzero(lens > 0)[0]
    colsum[nonempty] = np.add.reduceat((col % 1000).astype(np.float64), rp[nonempty].astype(np.int64))
    want = colsum[:, None] + lens[:, None] * (np.arange(k) / 256.0)[None, :]
    # fp32 accumulation of up to 3000 terms per row
    assert (np.abs(C - want).max(axis=1) <= 1e-4 * np.abs(want).max(axis=1) + 1e-30).all()
    # SDDMM with lhs = e_0: out[idx] = rhs[col, 0] = col % 1000
    lhs = torch.zeros(m, k, device=DEV)
    lhs[:, 0] = 1
    out = rode_sddmm(csr, lhs, B).cpu().numpy()
    np.testing.assert_array_equal(out, (col % 1000).astype(np.float32))


def test_clear_rows_prepares_exactly_what_spmm_does_not_overwrite():
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import _lib, rode_sddmm_hip
    lib = _lib.load()
    rng = np.random.default_rng(13)
    m, k, n = 900, 800, 96
    rp, col, val = random_csr(rng, m, k, 30, long_rows=4, long_len=700, empty_frac=0.2)
    csr = make_csr(rp, col, val, m, k, 32)
    C = torch.full((m, n), float("nan"), device=DEV)
    assert lib.rode_hip_spmm_clear_rows(m, n, 4, csr.row_offsets.data_ptr(), C.data_ptr(), None) == 0
    torch.cuda.synchronize()
    aligned = np.diff(rp) + rp[:-1] % 4
    cleared = (aligned >= 32) | (aligned == 0)
    got = C.cpu().numpy()
    assert (got[cleared] == 0).all() and np.isnan(got[~cleared]).all()
    # SpMM on the prepared buffer == SpMM on a fully zeroed one
    B = torch.from_numpy(rng.standard_normal((k, n)).astype(np.float32)).to(DEV)
    args = (csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2, csr.row_offsets,
            csr.column_indices, csr.values, m, k, B)
    a = rode_sddmm_hip.spmm_forward(*args, out=C)
    b = rode_sddmm_hip.spmm_forward(*args, out=torch.zeros(m, n, device=DEV))
    assert torch.isfinite(a).all() and (a - b).abs().max().item() <= 1e-5 * b.abs().max().item()
    # fp64 element size, bad arguments
    C64 = torch.full((m, 6), float("nan"), dtype=torch.float64, device=DEV)
    assert lib.rode_hip_spmm_clear_rows(m, 6, 8, csr.row_offsets.data_ptr(), C64.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert (C64[torch.from_numpy(cleared).to(DEV)] == 0).all()
    assert lib.rode_hip_spmm_clear_rows(m, 6, 4, csr.row_offsets.data_ptr(), C64.data_ptr(), None) != 0  # 24-byte rows
    assert lib.rode_hip_spmm_clear_rows(m, 8, 2, csr.row_offsets.data_ptr(), C64.data_ptr(), None) != 0


@pytest.mark.parametrize("seg,half", [(32, False), (96, False), (512, False), (512, True), (160, True)])
def test_whole_row_mode_and_split_calls(seg, half):
    """With >= 16384 block segments and the whole-lists promise (what the Python op
    passes), rows of 32..1024 slots are summed by one wave, tail included; rows just
    outside that range, unaligned starts and empty rows sit next to them here.  The
    typed entry points make no such promise: a caller who feeds the two lists in
    separate calls, or the block list in two halves, must get the same matrix (with
    >= 16384 segments per call the block kernel still merges short segments of a row,
    within the slice it was given: seg 32 and 96 here)."""
    import oracle
    from gpu_common import DEV, TOL_F16, TOL_F32, make_csr, round_half, run_spmm
    from helpers import spmm_row_l1_error
    from rode_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(seg)
    m, k, n = 24000, 3000, 64
    lens = rng.choice([0, 1, 5, 31, 32, 33, 63, 64, 100, 500, 1000, 1020, 1021, 1024, 1025, 1056, 1500], size=m,
                      p=[.05, .05, .1, .05, .05, .05, .05, .05, .2, .1, .05, .03, .03, .03, .03, .03, .05])
    lens[::4000] = [2999, 2500, 2048, 1999, 2990, 1600]  # several merge windows per row (k = 3000 columns)
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(k, size=l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    B = rng.standard_normal((k, n)).astype(np.float32)
    csr = make_csr(rp, col, val, m, k, 32, seg)
    assert csr.m1 >= 16384
    ref = oracle.spmm_f64(rp, col, val, round_half(B) if half else B)
    tol = TOL_F16 if half else TOL_F32
    assert spmm_row_l1_error(run_spmm(csr, B, half), ref) <= tol
    if half:
        return
    dB = torch.from_numpy(B).to(DEV)
    if seg == 96:  # the fp64 instantiation through the same promise
        from rode_amd import rode_sddmm_hip
        C64 = rode_sddmm_hip.spmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                          csr.row_offsets, csr.column_indices, csr.values.double(), m, k,
                                          dB.double()).cpu().numpy()
        assert spmm_row_l1_error(C64, ref) <= 1e-12

    def typed(m1, m2, blk_ptr, st_ptr, C):
        _lib.check(lib.rode_hip_spmm_f32(m1, m2, k, n, csr.values.data_ptr(), csr.column_indices.data_ptr(),
                                         csr.row_offsets.data_ptr(), blk_ptr, csr.residue_indices.data_ptr(), st_ptr,
                                         dB.data_ptr(), C.data_ptr(), None, None), "spmm")

    C = torch.zeros(m, n, device=DEV)
    half_m1 = csr.m1 // 2  # very likely inside a row
    typed(half_m1, 0, csr.block_indices.data_ptr(), csr.st_offsets.data_ptr(), C)
    typed(csr.m1 - half_m1, 0, csr.block_indices.data_ptr() + 4 * half_m1, csr.st_offsets.data_ptr() + 4 * half_m1, C)
    typed(0, csr.m2, csr.block_indices.data_ptr(), csr.st_offsets.data_ptr(), C)
    torch.cuda.synchronize()
    assert spmm_row_l1_error(C.cpu().numpy(), ref) <= tol


def test_headline_configuration_full_size_against_oracle():
    """Power law, full size, width 128, through rode_spmm (whole-lists promise with >= 16384
    block segments: rows of 32..1024 slots are summed by one wave, longer rows by merged
    leaders plus atomics) against the fp64 oracle on a fixed sample of rows that holds the
    longest row and rows of every kind."""
    import oracle
    from gpu_common import DEV, TOL_F32, make_csr
    from helpers import spmm_row_l1_error
    from rode_amd import rode_spmm, workloads
    from test_gpu_sddmm import sample_rows, sub_csr
    m, k, rp, col, val = workloads.config("c4_powerlaw")
    n = 128
    csr = make_csr(rp, col, val, m, k, n)
    assert csr.m1 >= 16384
    g = torch.Generator(device=DEV).manual_seed(78)
    B = torch.randn(k, n, device=DEV, generator=g)
    C = rode_spmm(csr, B)
    rows = sample_rows(rp, np.random.default_rng(5))
    sub_rp, idx = sub_csr(rp, rows)
    ref, scale = oracle.spmm_f64(sub_rp, col[idx], val[idx], B.cpu().numpy(), with_abs=True)
    got = C[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    err = spmm_row_l1_error(got, ref)
    assert err <= TOL_F32, f"row-L1 error {err}"
    assert (np.abs(got - ref) / np.maximum(scale, 1e-30)).max() <= 2e-6
    print(f"c4 width 128 full size: {len(rows)} rows, {len(idx)} nnz, row-L1 error {err:.2e}")


def test_measurement_flags_launch_one_kernel_of_the_pair():
    """RODE_SPMM_ONLY_BLOCK + RODE_SPMM_ONLY_RESIDUE in two calls give the result of one
    normal call, also under the whole-lists promise (each kernel still skips what the
    other one sums)."""
    from gpu_common import DEV, make_csr
    from rode_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(9)
    m, k, n = 20000, 2500, 64
    lens = rng.choice([0, 3, 31, 40, 100, 700, 1100, 2400], size=m, p=[.1, .2, .1, .2, .2, .1, .05, .05])
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(k, size=l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    csr = make_csr(rp, col, val, m, k, n, 32)
    assert csr.m1 >= 16384
    B = torch.from_numpy(rng.standard_normal((k, n)).astype(np.float32)).to(DEV)

    def call(flags, C):
        _lib.check(lib.rode_hip_spmm_ex(0, flags, csr.m1, csr.m2, k, n, csr.values.data_ptr(),
                                        csr.column_indices.data_ptr(), csr.row_offsets.data_ptr(),
                                        csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(),
                                        csr.st_offsets.data_ptr(), B.data_ptr(), C.data_ptr(), None, None), "spmm")

    for base in (0, _lib.SPMM_WHOLE_LISTS):
        both, split = torch.zeros(m, n, device=DEV), torch.zeros(m, n, device=DEV)
        call(base, both)
        call(base | _lib.SPMM_ONLY_BLOCK, split)
        call(base | _lib.SPMM_ONLY_RESIDUE, split)
        torch.cuda.synchronize()
        assert (both - split).abs().max().item() <= 1e-4 * both.abs().max().item()
    assert lib.rode_hip_spmm_ex(0, 6, csr.m1, csr.m2, k, n, csr.values.data_ptr(), csr.column_indices.data_ptr(),
                                csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(),
                                csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(), B.data_ptr(),
                                both.data_ptr(), None, None) != 0


def _spmm_overwrite(csr, B, C, flags):
    import ctypes
    from rode_amd import _lib, rode_sddmm_hip
    lib = _lib.load()
    plans = rode_sddmm_hip.plans_struct(csr.plan, B.shape[1], 4, True, seg_length=csr.config["seg_length"])
    s = torch.cuda.current_stream().cuda_stream
    code = lib.rode_hip_spmm_planned(_lib.DENSE_CODE["f16" if B.dtype == torch.float16 else "f32"], flags, csr.m1, csr.m2, csr.n,
                                     B.shape[1], csr.values.data_ptr(), csr.column_indices.data_ptr(), csr.row_offsets.data_ptr(),
                                     csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(),
                                     B.data_ptr(), C.data_ptr(), ctypes.byref(plans), s, s)
    torch.cuda.synchronize()
    return code


@pytest.mark.parametrize("case", ["one_segment_rows", "short_rows_only", "segments_of_32", "every_row_in_a_group", "half"])
def test_overwrite_stores_rows_that_have_one_owner(case):
    """RODE_SPMM_OVERWRITE: C = A B into a C full of NaN, on matrices whose every row has slots
    and a single work item (rows summed whole by one wave, rows of fewer than 32 slots, rows of
    kept groups); ``RoDeCSR.spmm_stores_every_row`` says so and ``rode_spmm`` then clears nothing."""
    import oracle
    from gpu_common import DEV, TOL_F16, TOL_F32, make_csr, round_half
    from helpers import spmm_row_l1_error
    from rode_amd import _lib, rode_sddmm_hip, rode_spmm
    rng = np.random.default_rng(len(case))
    width, half, seg, locality = 64, case == "half", None, False
    if case in ("one_segment_rows", "half"):
        m, n = 6000, 3000
        lens = rng.integers(1, 900, m)     # aligned lengths up to 903 slots: whole rows (m1 >= 1024 segments)
    elif case == "short_rows_only":
        m, n = 5000, 3000
        lens = rng.integers(1, 28, m)      # residue rows only
    elif case == "segments_of_32":
        m, n, seg = 3000, 3000, 32
        lens = rng.integers(200, 1000, m)  # >= 16384 segments of 32 slots: a wave walks a chunk of them
    else:
        m, n, locality = 2000, 2400, True
        lens = None
    if lens is not None:
        rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        col = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens]).astype(np.int32)
    else:
        rows = [np.arange(r, r + 300, dtype=np.int32) for r in range(m)]  # a window that moves one column per row
        rp = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
        col = np.concatenate(rows)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    csr = make_csr(rp, col, val, m, n, width, seg, locality=locality)
    if case == "every_row_in_a_group":
        assert isinstance(csr.plan, rode_sddmm_hip.GroupPlan) and csr.plan.counts[2] == 0
    if case == "segments_of_32":
        assert csr.m1 >= 16384
    assert csr.spmm_stores_every_row()
    B = rng.standard_normal((n, width)).astype(np.float32)
    dB = torch.from_numpy(B).to(DEV, torch.float16 if half else torch.float32)
    C = torch.full((m, width), float("nan"), device=DEV)
    assert _spmm_overwrite(csr, dB, C, _lib.SPMM_WHOLE_LISTS | _lib.SPMM_OVERWRITE) == 0
    ref = oracle.spmm_f64(rp, col, val, round_half(B) if half else B)
    got = C.cpu().numpy()
    assert np.isfinite(got).all(), "a row was added to, or left alone"
    assert spmm_row_l1_error(got, ref) <= (TOL_F16 if half else TOL_F32)
    again = rode_spmm(csr, dB).cpu().numpy()  # the op: an uninitialised C and no clearing
    assert spmm_row_l1_error(again, ref) <= (TOL_F16 if half else TOL_F32)


def test_overwrite_leaves_other_rows_to_the_callers_clearing():
    """Rows of several work items are still added to and rows without slots still untouched under
    RODE_SPMM_OVERWRITE (C holds 7 on entry); the limit function says which rows are which, and
    the flag needs the whole-lists promise."""
    import oracle
    from gpu_common import DEV, make_csr
    from rode_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(77)
    m, n, width = 4000, 5000, 32
    lens = rng.integers(1, 600, m)
    lens[10], lens[11], lens[12] = 3000, 0, 1025   # several work items; no slots; one slot too many
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    csr = make_csr(rp, col, val, m, n, width, locality=False)
    assert not csr.spmm_stores_every_row()
    limit = lib.rode_hip_spmm_overwrite_limit(csr.m1, None)
    assert limit == 1024 and lib.rode_hip_spmm_overwrite_limit(1023, None) == 0
    B = rng.standard_normal((n, width)).astype(np.float32)
    dB = torch.from_numpy(B).to(DEV)
    C = torch.full((m, width), 7.0, device=DEV)
    assert _spmm_overwrite(csr, dB, C, _lib.SPMM_WHOLE_LISTS | _lib.SPMM_OVERWRITE) == 0
    aligned = lens + rp[:-1] % 4
    added = (aligned > limit) | (aligned == 0)
    want = oracle.spmm_f64(rp, col, val, B) + np.where(added[:, None], 7.0, 0.0)
    assert np.abs(C.cpu().numpy() - want).max() <= 1e-4 * max(1.0, np.abs(want).max())
    assert _spmm_overwrite(csr, dB, C, _lib.SPMM_OVERWRITE) != 0   # not without the whole-lists promise
