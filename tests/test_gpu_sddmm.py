"""SDDMM parity on the GPU, through the Python op and the C ABI.

Oracles: oracle.sddmm_f32 (the reference tests' own CPU loop, judged with the
reference tests' abs-AND-rel rule, tol 1e-3) and oracle.sddmm_f64 (judged with the
row-L1-normalised bound: 1e-4 for fp32 operands, 2e-3 for fp16 operands with fp32
accumulation)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

# The reference's own table, RoDe_SDDMM/run_test.py:81-132 (m, n, nnz_per_row).
REFERENCE_CONFIGS = [
    (64, 64, 8), (128, 128, 16), (256, 256, 32), (63, 67, 10), (97, 103, 15), (127, 131, 20),
    (512, 512, 32), (1024, 1024, 64), (2048, 2048, 128), (511, 517, 33), (1023, 1031, 65), (2047, 2053, 127),
    (2048, 256, 32), (4096, 512, 64), (1999, 257, 45), (256, 2048, 32), (512, 4096, 64), (257, 2003, 47),
    (1, 1000, 100), (1000, 1, 1), (17, 1999, 150), (1999, 17, 5), (31, 4097, 200),
    (1024, 1024, 1), (1024, 1024, 4), (1024, 1024, 16), (1024, 1024, 64), (1024, 1024, 256), (1024, 1024, 512),
    (32, 32, 16), (33, 31, 10), (128, 32, 8), (32, 128, 8),
    (127, 131, 23), (251, 257, 47), (509, 521, 67), (1021, 1031, 97),
    (4096, 4096, 128), (4093, 4099, 129),
]


WELL_CONDITIONED = 100.0


def _check(csr, rp, col, val, lhs, rhs, half=False, ref_rule=True):
    """Tolerances.  (1) Row-L1 bound of the target: max|err| over a row's outputs /
    sum|ref| over the row <= 1e-4 (fp32) or 2e-3 (fp16 operands), asserted on every row
    whose condition number sum|terms| / sum|ref| is <= 100.  A row that consists of one
    or two cancelling dot products can exceed it under ANY fp32 summation order; there the
    GPU must not be worse than twice the reference's own CPU loop (main.cu:65-91).
    (2) Per element, |err| <= 2e-6 * |val| * sum_k|lhs*rhs| (fp32 operands), everywhere.
    (3) The reference tests' own rule against the reference's CPU loop: no element with
    both abs and rel error > 1e-3."""
    import oracle
    from gpu_common import TOL_F16, TOL_F32, check_csr_decomposition, round_half, run_sddmm
    from helpers import reference_error_count, sddmm_row_l1_errors
    check_csr_decomposition(csr, rp)
    out = run_sddmm(csr, lhs, rhs, half)
    assert out.shape == (len(val),) and out.dtype == np.float32
    if half:
        lhs, rhs = round_half(lhs), round_half(rhs)
    tol = TOL_F16 if half else TOL_F32
    ref64, scale = oracle.sddmm_f64(rp, col, val, lhs, rhs, with_abs=True)
    err, cond = sddmm_row_l1_errors(out, ref64, scale, rp)
    good = cond <= WELL_CONDITIONED
    worst = float(err[good].max(initial=0.0))
    assert worst <= tol, f"row-L1 error {worst}"
    if (~good).any():
        cpu32 = oracle.sddmm_f32(rp, col, val, lhs, rhs)
        cpu_err, _ = sddmm_row_l1_errors(cpu32, ref64, scale, rp)
        assert float(err[~good].max()) <= max(tol, 2 * float(cpu_err[~good].max())), \
            f"ill-conditioned rows: GPU {err[~good].max()} vs reference CPU loop {cpu_err[~good].max()}"
    if not half:
        strict = np.abs(out - ref64) / np.maximum(scale, 1e-30)
        assert strict.max(initial=0.0) <= 2e-6, f"per-element error {strict.max()}"
        if ref_rule:
            assert reference_error_count(out, oracle.sddmm_f32(rp, col, val, lhs, rhs)) == 0
    return worst


@pytest.mark.parametrize("k", [128, 32])
def test_reference_table(k):
    """The reference's C++ test (test.cu for k=128, main.cu for k=32): its seeded
    generators (rows padded to 4 with explicit zeros), its decomposition parameters,
    its CPU loop and its pass rule."""
    from gpu_common import make_csr
    from rode_amd import RoDeCSR, workloads
    worst = 0.0
    for m, n, per_row in REFERENCE_CONFIGS:
        rp, col, val = workloads.reference_csr(m, n, per_row, poisson=(k == 128), pad_to=4, seed=42)
        lhs = workloads.reference_dense(m, k, 123)
        rhs = workloads.reference_dense(n, k, 456)
        ref_seg = RoDeCSR.REFERENCE_CONFIGS[k]["seg_length"]  # (512,32,4) for 32, (32,32,4) for 128
        for seg in sorted({ref_seg, RoDeCSR.CONFIGS[k]["seg_length"]}):
            csr = make_csr(rp, col, val, m, n, k, seg)
            worst = max(worst, _check(csr, rp, col, val, lhs, rhs))
    print(f"k={k}: worst row-L1 error over {len(REFERENCE_CONFIGS)} reference configs: {worst:.2e}")


def test_reference_stress():
    """run_test.py:427-439: random.seed(42), random shapes."""
    import random
    from gpu_common import make_csr
    from rode_amd import workloads
    random.seed(42)
    for _ in range(12):
        m, n = random.randint(10, 2000), random.randint(10, 2000)
        per_row = random.randint(1, min(n, 200))
        rp, col, val = workloads.reference_csr(m, n, per_row, poisson=True)
        csr = make_csr(rp, col, val, m, n, 128, 32)
        _check(csr, rp, col, val, workloads.reference_dense(m, 128, 123), workloads.reference_dense(n, 128, 456))


@pytest.mark.parametrize("k", [32, 64, 128])
@pytest.mark.parametrize("seg", [32, 64, 512])
def test_unpadded_rows(k, seg):
    """Rows that start at any offset mod 4 (the reference's Python test path,
    test_pytorch.py), long rows, empty rows, every K and several segment lengths."""
    from gpu_common import make_csr
    from helpers import random_csr
    rng = np.random.default_rng(1000 * k + seg)
    m, n = 1500, 1777
    rp, col, val = random_csr(rng, m, n, 37, long_rows=6, long_len=1700, empty_frac=0.15)
    assert (rp[:-1] % 4 != 0).any()
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    _check(make_csr(rp, col, val, m, n, k, seg), rp, col, val, lhs, rhs)


@pytest.mark.parametrize("k", [4, 8, 20, 48, 96, 100, 160, 256, 300, 384, 512])
def test_any_k(k):
    """k beyond the reference's 32 / 128: any multiple of 4 up to 512 (row tiles of 32 /
    64 / 128 elements, up to four slabs, the partial last slab guarded)."""
    from gpu_common import make_csr
    from helpers import random_csr
    rng = np.random.default_rng(k)
    m, n = 700, 800
    rp, col, val = random_csr(rng, m, n, 35, long_rows=4, long_len=750, empty_frac=0.1)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    csr = make_csr(rp, col, val, m, n, k)
    _check(csr, rp, col, val, lhs, rhs)
    if k % 8 == 0:
        _check(csr, rp, col, val, lhs, rhs, half=True)


@pytest.mark.parametrize("k", [32, 64, 128])
def test_fp16_operands(k):
    from gpu_common import make_csr
    from helpers import random_csr
    rng = np.random.default_rng(k)
    m, n = 900, 1200
    rp, col, val = random_csr(rng, m, n, 50, long_rows=4, long_len=1100)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    for seg in (32, 512):
        _check(make_csr(rp, col, val, m, n, k, seg), rp, col, val, lhs, rhs, half=True)


def test_fp16_subnormal_operands():
    """fp16 operands below the smallest normal number (2^-14) count with their value: the
    packed dot-product instruction of the fp16 kernels does not flush them."""
    from gpu_common import make_csr, run_sddmm
    rng = np.random.default_rng(3)
    m, n, k = 64, 64, 64
    rp = np.arange(0, m * 8 + 1, 8, dtype=np.int32)
    col = np.concatenate([np.sort(rng.choice(n, 8, replace=False)) for _ in range(m)]).astype(np.int32)
    csr = make_csr(rp, col, np.ones(len(col), dtype=np.float32), m, n, k)
    out = run_sddmm(csr, np.full((m, k), 2.0 ** -20, dtype=np.float32), np.full((n, k), 2.0 ** 10, dtype=np.float32), True)
    assert (out == k * 2.0 ** -10).all()   # every product and every partial sum is exact in fp32


def test_special_cases_and_edges():
    from gpu_common import DEV, make_csr, run_sddmm
    from helpers import random_csr
    from rode_amd import rode_sddmm
    rng = np.random.default_rng(9)
    m, n, k = 700, 650, 64
    rp, col, val = random_csr(rng, m, n, 45, long_rows=3, long_len=600)
    csr = make_csr(rp, col, val, m, n, k)
    # all-ones operands: out = k * val exactly
    out = run_sddmm(csr, np.ones((m, k), np.float32), np.ones((n, k), np.float32))
    np.testing.assert_array_equal(out, val * np.float32(k))
    # an Inf in an rhs row that one row references must not leak into other outputs
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    bad_col = int(col[rp[10]])
    rhs[bad_col, 3] = np.inf
    out = run_sddmm(csr, lhs, rhs)
    assert np.isfinite(out[col != bad_col]).all() and not np.isfinite(out[col == bad_col]).any()
    # empty matrix, matrix with empty rows only
    empty = make_csr(np.zeros(6, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), 5, 7, 32)
    assert (empty.m1, empty.m2) == (0, 0)
    assert rode_sddmm(empty, torch.zeros(5, 32, device=DEV), torch.zeros(7, 32, device=DEV)).numel() == 0
    # non-contiguous operands are made contiguous by the op
    lhs_t = torch.from_numpy(rng.standard_normal((k, m)).astype(np.float32)).to(DEV).t()
    rhs_t = torch.from_numpy(rng.standard_normal((n, k)).astype(np.float32)).to(DEV)
    a = rode_sddmm(csr, lhs_t, rhs_t)
    b = rode_sddmm(csr, lhs_t.contiguous(), rhs_t)
    assert torch.equal(a, b)


def test_argument_errors():
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import RoDeCSR, rode_sddmm, rode_sddmm_hip
    rng = np.random.default_rng(2)
    rp, col, val = random_csr(rng, 40, 50, 8)
    csr = make_csr(rp, col, val, 40, 50, 32)
    lhs, rhs = torch.zeros(40, 32, device=DEV), torch.zeros(50, 32, device=DEV)
    with pytest.raises(ValueError):
        RoDeCSR(torch.from_numpy(rp), torch.from_numpy(col), torch.from_numpy(val), DEV, 40, 50, 50)
    with pytest.raises(ValueError):
        rode_sddmm(csr, lhs[:, :16], rhs)
    with pytest.raises(ValueError):
        rode_sddmm(csr, lhs, rhs[:49])
    with pytest.raises(AssertionError):
        rode_sddmm(csr, lhs.cpu(), rhs)
    with pytest.raises(AssertionError):
        rode_sddmm(csr, lhs.double(), rhs.double())
    args = [csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2, csr.row_offsets,
            csr.column_indices, csr.values, 40, 50, lhs, rhs, 32]
    for pos, bad, msg in [(12, 50, "k_version must be"), (12, 128, "match k_version"), (8, 41, "rows must equal m"),
                          (7, csr.values.double(), "float32"), (6, csr.column_indices.long(), "int32"),
                          (10, lhs.cpu(), "CUDA tensor"), (11, rhs.t().contiguous().t(), "contiguous")]:
        a = list(args)
        a[pos] = bad
        with pytest.raises(RuntimeError, match=msg):
            rode_sddmm_hip.sddmm_forward(*a)


def test_torch_oracle_and_compare_results():
    """The reference's Python test flow (test_pytorch.py:163-207): RoDeCSR.from_random,
    torch.sparse.sampled_addmm as the oracle, compare_results as the judge."""
    from gpu_common import DEV
    from rode_amd import RoDeCSR, compare_results, rode_sddmm, torch_sddmm_reference
    torch.manual_seed(0)
    for k in (32, 128):
        csr = RoDeCSR.from_random(511, 517, 33, DEV, k)
        torch.manual_seed(123); lhs = torch.randn(511, k, device=DEV)
        torch.manual_seed(456); rhs = torch.randn(517, k, device=DEV)
        out = rode_sddmm(csr, lhs, rhs)
        ref = torch_sddmm_reference(csr.to_torch_sparse_csr(), lhs, rhs)
        stats = compare_results(out, ref, csr)
        assert stats["passed"] and stats["total_count"] == csr.nnz and stats["max_abs"] < 1e-3, stats
        assert "RoDeCSR(m=511" in repr(csr)


# the configuration list of the reference's Python driver (test_pytorch.py:66-91): small,
# irregular, medium, rectangular, sparsity sweep, prime dimensions, large irregular
PYTHON_DRIVER_CONFIGS = [(64, 64, 8), (128, 128, 16), (256, 256, 32), (63, 67, 10), (127, 131, 20), (511, 517, 33),
                         (512, 512, 32), (1024, 1024, 64), (2048, 2048, 128), (2048, 256, 32), (256, 2048, 32),
                         (1999, 257, 45), (1024, 1024, 4), (1024, 1024, 64), (1024, 1024, 256), (127, 131, 23),
                         (509, 521, 67), (4093, 4099, 128)]


@pytest.mark.parametrize("k", [128, 32])
def test_python_driver_configurations(k):
    """Every configuration of the reference's Python driver through its own flow
    (test_pytorch.py:163-222): from_random, rode_sddmm, torch.sparse.sampled_addmm,
    compare_results; K=128 is the driver's default, K=32 the other supported width."""
    from gpu_common import DEV
    from rode_amd import RoDeCSR, compare_results, rode_sddmm, torch_sddmm_reference
    for i, (m, n, per_row) in enumerate(PYTHON_DRIVER_CONFIGS):
        torch.manual_seed(1000 + i)
        csr = RoDeCSR.from_random(m, n, per_row, DEV, k)
        torch.manual_seed(123); lhs = torch.randn(m, k, device=DEV)
        torch.manual_seed(456); rhs = torch.randn(n, k, device=DEV)
        stats = compare_results(rode_sddmm(csr, lhs, rhs), torch_sddmm_reference(csr.to_torch_sparse_csr(), lhs, rhs), csr)
        assert stats["passed"] and stats["total_count"] == csr.nnz, (m, n, per_row, stats)


@pytest.mark.parametrize("name,k", [("c1_uniform", 32), ("c2_lognormal", 32), ("c2_lognormal", 128)])
def test_benchmark_configs_against_oracle(name, k):
    from gpu_common import make_csr
    from rode_amd import workloads
    m, n, rp, col, val = workloads.config(name)
    rng = np.random.default_rng(3000 + k)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    for seg in (512, 32):
        _check(make_csr(rp, col, val, m, n, k, seg), rp, col, val, lhs, rhs, ref_rule=(name == "c1_uniform"))


@pytest.mark.parametrize("name,k,half", [("c3_banded", 32, False), ("c4_powerlaw", 64, False),
                                         ("c5_attention", 64, False), ("c5_attention", 64, True)])
def test_large_configs_scaled_against_oracle(name, k, half):
    from gpu_common import make_csr
    from rode_amd import workloads
    scale = {"c3_banded": 1 / 16, "c4_powerlaw": 1 / 16, "c5_attention": 1 / 4}[name]
    m, n, rp, col, val = workloads.config(name, scale)
    rng = np.random.default_rng(4000 + k)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    _check(make_csr(rp, col, val, m, n, k, 512), rp, col, val, lhs, rhs, half=half, ref_rule=False)


@pytest.mark.parametrize("name,k", [("c3_banded", 128), ("c4_powerlaw", 128), ("c4_powerlaw", 64), ("c5_attention", 64)])
def test_full_size_properties(name, k):
    """Full benchmark sizes, checked through size-independent facts: with one-hot
    lhs rows and an rhs holding its own row number, out[idx] = val[idx] * col[idx]
    exactly; with all-ones operands out = k * val; and out is linear in lhs."""
    from gpu_common import DEV, make_csr
    from rode_amd import rode_sddmm, workloads
    m, n, rp, col, val = workloads.config(name)
    csr = make_csr(rp, col, val, m, n, k, 512)
    v = torch.from_numpy(val).to(DEV)
    ones = rode_sddmm(csr, torch.ones(m, k, device=DEV), torch.ones(n, k, device=DEV))
    assert torch.equal(ones, v * k)
    lhs = torch.zeros(m, k, device=DEV); lhs[:, k - 1] = 1
    rhs = torch.zeros(n, k, device=DEV); rhs[:, k - 1] = torch.arange(n, device=DEV, dtype=torch.float32) % 4096
    out = rode_sddmm(csr, lhs, rhs)
    assert torch.equal(out, v * (torch.from_numpy(col).to(DEV) % 4096).float())
    del lhs, rhs, ones, out
    g = torch.Generator(device=DEV).manual_seed(k)
    a = torch.randn(m, k, device=DEV, generator=g); b = torch.randn(m, k, device=DEV, generator=g)
    r = torch.randn(n, k, device=DEV, generator=g)
    oa, ob, oab = rode_sddmm(csr, a, r), rode_sddmm(csr, b, r), rode_sddmm(csr, a + b, r)
    scale = (oa.abs() + ob.abs()).clamp_min(1e-20)
    assert ((oab - (oa + ob)).abs() / (scale + v.abs() * 1e-1)).max().item() < 1e-3


@pytest.mark.parametrize("seg", [32, 96, 512])
def test_lists_passed_in_slices(seg):
    """A caller may feed the block list in pieces and the residue list separately (the
    typed entry point promises nothing about completeness).  Short segments are merged
    inside the kernel; at a slice boundary that only means an output computed twice."""
    import oracle
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(seg)
    m, n, k = 1200, 2600, 64
    rp, col, val = random_csr(rng, m, n, 50, long_rows=8, long_len=2500, empty_frac=0.1)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    csr = make_csr(rp, col, val, m, n, k, seg)
    dl, dr = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)
    out = torch.full((len(val),), float("nan"), device=DEV)

    def call(m1, m2, first):
        _lib.check(lib.rode_hip_sddmm_f32(m1, m2, n, k, csr.block_indices.data_ptr() + 4 * first,
                                          csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr() + 4 * first,
                                          csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(),
                                          csr.values.data_ptr(), dl.data_ptr(), dr.data_ptr(), out.data_ptr(),
                                          None, None), "sddmm")

    cuts = [0, csr.m1 // 3, csr.m1 // 3 + 1, (2 * csr.m1) // 3, csr.m1]
    for a, b in zip(cuts[:-1], cuts[1:]):
        call(b - a, 0, a)
    call(0, csr.m2, 0)
    torch.cuda.synchronize()
    ref, scale = oracle.sddmm_f64(rp, col, val, lhs, rhs, with_abs=True)
    got = out.cpu().numpy()
    assert np.isfinite(got).all()
    assert np.max(np.abs(got - ref) / np.maximum(scale, 1e-30)) <= 2e-6


@pytest.mark.parametrize("seg", [48, 80, 100])
def test_lists_of_an_unsupported_segment_length_stay_in_bounds(seg):
    """seg_length % 32 != 0 is outside the contract of the entry points (the Python class
    refuses it), but the C ABI cannot tell how its lists were made.  The kernels must then
    write exactly the entries that the host model of their index ranges lists
    (helpers.merged_block_ranges / residue_ranges: inside the arrays, inside the row),
    each with the right value, and nothing else -- canaries before out[0], after
    out[nnz-1] and on every entry no work item owns must survive."""
    import oracle
    from gpu_common import DEV
    from helpers import merged_block_ranges, random_csr, residue_ranges
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(seg)
    m, n, k = 700, 900, 64
    rp, col, val = random_csr(rng, m, n, 45, long_rows=6, long_len=850, empty_frac=0.1)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    nnz = len(val)
    d_rp = torch.from_numpy(rp).to(DEV)
    blk, st, res, m1, m2 = rode_sddmm_hip.preprocess_device(d_rp, nnz, seg, 32, 4)
    oblk, ost, ores = oracle.preprocess(rp, seg)
    assert blk.cpu().numpy()[:m1].tobytes() == oblk.tobytes() and st.cpu().numpy().tobytes() == ost.tobytes()
    expect = np.zeros(nnz, bool)
    for r, _, first, end in merged_block_ranges(rp, oblk, ost, 128):
        expect[first:end] = True
    for r, first, end in residue_ranges(rp, ores):
        expect[first:end] = True
    assert expect.sum() > 0
    pad = 256
    dcol = torch.zeros(nnz + 2 * pad, dtype=torch.int32, device=DEV)   # col / val with margins, so that a stray
    dval = torch.zeros(nnz + 2 * pad, dtype=torch.float32, device=DEV)  # read would be harmless and a stray write visible
    dcol[pad:pad + nnz] = torch.from_numpy(col).to(DEV)
    dval[pad:pad + nnz] = torch.from_numpy(val).to(DEV)
    from rode_amd import _lib
    lib = _lib.load()
    out = torch.full((nnz + 2 * pad,), -777.0, device=DEV)
    dl, dr = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)
    _lib.check(lib.rode_hip_sddmm_f32(m1, m2, n, k, blk.data_ptr(), res.data_ptr(), st.data_ptr(), d_rp.data_ptr(),
                                      dcol.data_ptr() + 4 * pad, dval.data_ptr() + 4 * pad, dl.data_ptr(), dr.data_ptr(),
                                      out.data_ptr() + 4 * pad, None, None), "sddmm")
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert (got[:pad] == -777.0).all() and (got[pad + nnz:] == -777.0).all(), "write outside out[0, nnz)"
    got = got[pad:pad + nnz]
    assert ((got != -777.0) == expect).all(), "written entries differ from the host model"
    ref, scale = oracle.sddmm_f64(rp, col, val, lhs, rhs, with_abs=True)
    assert np.max(np.abs(got[expect] - ref[expect]) / np.maximum(scale[expect], 1e-30)) <= 2e-6


def test_headline_configuration_full_size_against_oracle():
    """The configuration the benchmark reports -- power law, full size, K = 128, the
    library's default decomposition (>= 16384 block segments, so merged leaders are what
    runs) -- against the fp64 oracle on a fixed sample of rows: the longest row, rows of
    32..1024 slots, rows of more than 1024 slots, short rows."""
    import oracle
    from gpu_common import DEV, TOL_F32, make_csr
    from helpers import sddmm_row_l1_errors
    from rode_amd import rode_sddmm, workloads
    m, n, rp, col, val = workloads.config("c4_powerlaw")
    k = 128
    csr = make_csr(rp, col, val, m, n, k)
    assert csr.m1 >= 16384
    g = torch.Generator(device=DEV).manual_seed(77)
    lhs = torch.randn(m, k, device=DEV, generator=g)
    rhs = torch.randn(n, k, device=DEV, generator=g)
    out = rode_sddmm(csr, lhs, rhs)
    rows = sample_rows(rp, np.random.default_rng(4))
    sub_rp, idx = sub_csr(rp, rows)
    ref, scale = oracle.sddmm_f64(sub_rp, col[idx], val[idx], lhs[torch.from_numpy(rows).to(DEV)].cpu().numpy(),
                                  rhs.cpu().numpy(), with_abs=True)
    got = out[torch.from_numpy(idx).to(DEV)].cpu().numpy()
    assert np.max(np.abs(got - ref) / np.maximum(scale, 1e-30)) <= 2e-6
    err, cond = sddmm_row_l1_errors(got, ref, scale, sub_rp)
    assert err[cond <= 100].max() <= TOL_F32
    print(f"c4 K=128 full size: {len(rows)} rows, {len(idx)} nnz, worst row-L1 error {err.max():.2e} "
          f"({int((cond > 100).sum())} rows with condition > 100, worst {err[cond <= 100].max():.2e} on the others)")


def sample_rows(rp, rng):
    """Longest row, 200 rows of 32..1024 aligned slots, 20 rows above 1024, 500 shorter ones."""
    lens = np.diff(rp)
    N = lens + rp[:-1] % 4
    pick = [np.array([int(np.argmax(lens))])]
    for mask, count in (((N >= 32) & (N <= 1024), 200), (N > 1024, 20), ((N > 0) & (N < 32), 500)):
        cand = np.nonzero(mask)[0]
        pick.append(rng.choice(cand, size=min(count, len(cand)), replace=False))
    return np.unique(np.concatenate(pick)).astype(np.int64)


def sub_csr(rp, rows):
    """Row pointer of the matrix made of ``rows`` and the indices of their nonzeros."""
    lens = np.diff(rp)[rows]
    sub_rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    idx = np.concatenate([np.arange(rp[r], rp[r + 1], dtype=np.int64) for r in rows])
    return sub_rp, idx


@pytest.mark.parametrize("seg", [32, 64, 160])
def test_many_short_segments_write_exactly_their_entries(seg):
    """At least 16384 segments of a short length: a wave walks a chunk of consecutive segments
    from leader to leader (rode_items.hpp).  Through the typed entry point, whole lists and in
    two slices cut inside a row: every entry a work item owns is written with the right value,
    the entries of empty or absent work items keep their canary, nothing outside out[0, nnz)."""
    import oracle
    from gpu_common import DEV
    from helpers import merged_block_ranges, residue_ranges
    from rode_amd import _lib, rode_sddmm_hip
    rng = np.random.default_rng(1000 + seg)
    m, n, k = {32: 3000, 64: 4500, 160: 10000}[seg], 4000, 32
    lens = rng.choice([0, 5, 31, 33, 200, 700, 1500, 3900], size=m, p=[.05, .1, .1, .15, .2, .2, .15, .05])
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    nnz = len(val)
    d_rp = torch.from_numpy(rp).to(DEV)
    blk, st, res, m1, m2 = rode_sddmm_hip.preprocess_device(d_rp, nnz, seg, 32, 4)
    assert m1 >= 2 * 16384  # (each of the two slices below still has enough segments for the walk)
    oblk, ost, ores = oracle.preprocess(rp, seg)
    expect = np.zeros(nnz, bool)
    for r, _, first, end in merged_block_ranges(rp, oblk, ost, 512):
        expect[first:end] = True
    for r, first, end in residue_ranges(rp, ores):
        expect[first:end] = True
    ref, scale = oracle.sddmm_f64(rp, col, val, lhs, rhs, with_abs=True)
    lib = _lib.load()
    pad = 256
    dcol = torch.zeros(nnz + 2 * pad, dtype=torch.int32, device=DEV)
    dval = torch.zeros(nnz + 2 * pad, dtype=torch.float32, device=DEV)
    dcol[pad:pad + nnz] = torch.from_numpy(col).to(DEV)
    dval[pad:pad + nnz] = torch.from_numpy(val).to(DEV)
    dl, dr = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)

    def call(out, a, b, with_residue):
        _lib.check(lib.rode_hip_sddmm_f32(b - a, m2 if with_residue else 0, n, k, blk.data_ptr() + 4 * a, res.data_ptr(),
                                          st.data_ptr() + 4 * a, d_rp.data_ptr(), dcol.data_ptr() + 4 * pad,
                                          dval.data_ptr() + 4 * pad, dl.data_ptr(), dr.data_ptr(), out.data_ptr() + 4 * pad,
                                          None, None), "sddmm")

    inside = np.nonzero(oblk[1:] == oblk[:-1])[0] + 1   # segments that are not the first of their row
    cut = int(inside[np.searchsorted(inside, m1 // 2)])  # inside a row: the second slice starts with one of its later segments
    assert oblk[cut] == oblk[cut - 1] and m1 - cut >= 16384 <= cut
    for slices in ([(0, m1)], [(0, cut), (cut, m1)]):
        out = torch.full((nnz + 2 * pad,), -777.0, device=DEV)
        for i, (a, b) in enumerate(slices):
            call(out, a, b, i == 0)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert (got[:pad] == -777.0).all() and (got[pad + nnz:] == -777.0).all(), "write outside out[0, nnz)"
        got = got[pad:pad + nnz]
        assert ((got != -777.0) == expect).all(), "written entries differ from the host model"
        assert np.max(np.abs(got[expect] - ref[expect]) / np.maximum(scale[expect], 1e-30)) <= 2e-6


@pytest.mark.parametrize("seg", [32, 512])
def test_a_wrong_segment_length_hint_changes_no_result(seg):
    """``rode_hip_plans.seg_length`` only sizes the block kernels' grid and chunks: lists of
    more than 16384 segments made with one length, called with the hint of another (shorter,
    longer, not a power of two, absent) - SDDMM and SpMM against the oracle every time."""
    import oracle
    from gpu_common import DEV, TOL_F32
    from helpers import sddmm_row_l1_errors, spmm_row_l1_error
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(2000 + seg)
    m, n, k = (4000, 3000, 32) if seg == 32 else (24000, 3000, 32)
    lens = rng.choice([0, 7, 40, 300, 900, 2500], size=m, p=[.05, .15, .2, .3, .2, .1])
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = rng.standard_normal((n, k)).astype(np.float32)
    nnz = len(val)
    d_rp = torch.from_numpy(rp).to(DEV)
    blk, st, res, m1, m2 = rode_sddmm_hip.preprocess_device(d_rp, nnz, seg, 32, 4)
    assert m1 >= 16384
    dcol, dval = torch.from_numpy(col).to(DEV), torch.from_numpy(val).to(DEV)
    dl, dr = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)
    ref, scale = oracle.sddmm_f64(rp, col, val, lhs, rhs, with_abs=True)
    ref_c = oracle.spmm_f64(rp, col, val, rhs)
    for hint in (seg, 0, 32, 96, 512, 4096):
        out = rode_sddmm_hip.sddmm_forward(blk, res, st, m1, m2, d_rp, dcol, dval, m, n, dl, dr, k, seg_length=hint)
        err, cond = sddmm_row_l1_errors(out.cpu().numpy(), ref, scale, rp)
        assert float(err[cond <= 100].max(initial=0.0)) <= TOL_F32, (seg, hint)
        for whole in (True, False):
            C = rode_sddmm_hip.spmm_forward(blk, res, st, m1, m2, d_rp, dcol, dval, m, n, dr, whole_lists=whole,
                                            seg_length=hint)
            assert spmm_row_l1_error(C.cpu().numpy(), ref_c) <= TOL_F32, (seg, hint, whole)


def test_device_given_without_an_index():
    """``device="cuda"`` means the current GPU: the matrix reports the device its tensors
    report, so operands made with ``.to("cuda")`` pass the ops' device checks."""
    from rode_amd import RoDeCSR, rode_sddmm, rode_spmm
    torch.manual_seed(5)
    csr = RoDeCSR.from_random(300, 200, 20, "cuda", k=32)
    assert csr.device == csr.values.device and csr.device.index is not None
    lhs, rhs = torch.randn(300, 32).to("cuda"), torch.randn(200, 32).to("cuda")
    out = rode_sddmm(csr, lhs, rhs)
    C = rode_spmm(csr, rhs)
    dense = csr.to_torch_sparse_csr().to_dense()
    assert torch.allclose(C, dense @ rhs, atol=1e-4, rtol=1e-4)
    assert out.shape == (csr.nnz,) and torch.isfinite(out).all()
