"""Group plan: groups of four adjacent rows that share a long run of consecutive columns
are processed by kernels of their own (rode_group.hip, spmm_group_kernel,
sddmm_group_kernel).  The plan changes which kernel processes a row, never a result:
everything here is checked against the fp64 oracle with the tolerances of the unplanned
kernels."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _window_matrix(rng, m, n, window, extra, ragged=True):
    """Sliding window of `window` columns around the diagonal plus `extra` random columns
    per row; with `ragged`, some rows get holes in their window, some are empty, some short."""
    rows = []
    for r in range(m):
        lo, hi = max(0, r * n // m - window // 2), min(n, r * n // m + window // 2)
        c = set(range(lo, hi)) | set(rng.choice(n, extra, replace=False).tolist())
        if ragged and r % 37 == 5:
            c -= set(range(lo + 10, lo + 13))          # a hole: the longest run is only part of the window
        if ragged and r % 53 == 7:
            c = set()                                  # an empty row inside a group
        if ragged and r % 61 == 9:
            c = set(rng.choice(n, 5, replace=False).tolist())  # a short row without a run
        rows.append(np.array(sorted(c), dtype=np.int32))
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum([len(c) for c in rows])
    col = np.concatenate(rows).astype(np.int32) if rp[-1] else np.zeros(0, dtype=np.int32)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    return rp, col, val


def test_plan_contents():
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(0)
    m, n = 203, 900   # 203 rows: the last three are in no group
    rp, col, val = _window_matrix(rng, m, n, 200, 12)
    dev = torch.device("cuda:0")
    plan = rode_sddmm_hip.group_plan(torch.from_numpy(rp).to(dev), torch.from_numpy(col).to(dev), m)
    assert plan.counts[0] == m // 4
    desc = plan.groups()
    kept = 0
    for g in range(m // 4):
        runs = []
        for r in range(4 * g, 4 * g + 4):
            c = col[rp[r]:rp[r + 1]]
            best = (0, 0, 0)
            i = 0
            while i < len(c):                      # longest run of consecutive columns (the first of equals)
                j = i
                while j + 1 < len(c) and c[j + 1] == c[j] + 1:
                    j += 1
                if j - i + 1 > best[1]:
                    best = (int(c[i]), j - i + 1, i)
                i = j + 1
            runs.append(best)
        lo, hi = max(a for a, _, _ in runs), min(a + l for a, l, _ in runs)       # what the four runs have in common
        first, last = min(a for a, _, _ in runs), max(a + l for a, l, _ in runs)  # what they cover between them
        slots = rp[4 * g + 4] - rp[4 * g]
        keep = hi - lo >= 64 and 16 * (hi - lo) >= 3 * slots and lo - first <= 255 and last - hi <= 255
        if keep:
            kept += 1
            assert desc[g, 0] == first and desc[g, 1] == last - first
            assert desc[g, 2:6].tolist() == [p for _, _, p in runs]
            heads, tails = int(desc[g, 6]) & 0xffffffff, int(desc[g, 7]) & 0xffffffff
            assert [(heads >> (8 * r)) & 255 for r in range(4)] == [a - first for a, _, _ in runs]
            assert [(tails >> (8 * r)) & 255 for r in range(4)] == [last - a - l for a, l, _ in runs]
        else:
            assert desc[g, 1] == 0
    assert plan.counts[1] == kept and 0 < kept < m // 4   # the ragged rows break some groups
    assert plan.counts[2] == m - 4 * kept                 # rows left to the other kernels


@pytest.mark.parametrize("k,half", [(64, False), (128, False), (32, False), (64, True), (128, True), (200, False)])
def test_grouped_rows_against_oracle(k, half):
    import oracle
    from gpu_common import TOL_F16, TOL_F32, make_csr, round_half, run_sddmm, run_spmm
    from helpers import spmm_row_l1_error, sddmm_row_l1_errors
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(k)
    m, n = 441, 940
    rp, col, val = _window_matrix(rng, m, n, 300 if k != 32 else 77, 20)
    csr = make_csr(rp, col, val, m, n, k, locality=True)
    assert isinstance(csr.plan, rode_sddmm_hip.GroupPlan) and csr.plan.usable
    assert 0 < csr.plan.counts[1] < 128  # few groups: a workgroup per group
    B = rng.standard_normal((n, k)).astype(np.float32)
    L = rng.standard_normal((m, k)).astype(np.float32)
    Bq, Lq = (round_half(B), round_half(L)) if half else (B, L)
    tol = TOL_F16 if half else TOL_F32
    assert spmm_row_l1_error(run_spmm(csr, B, half), oracle.spmm_f64(rp, col, val, Bq)) <= tol
    ref64, scale = oracle.sddmm_f64(rp, col, val, Lq, Bq, with_abs=True)
    out = run_sddmm(csr, L, B, half)
    err, cond = sddmm_row_l1_errors(out, ref64, scale, rp)
    assert float(err[cond <= 100].max(initial=0.0)) <= tol
    if not half:
        assert (np.abs(out - ref64) / np.maximum(scale, 1e-30)).max() <= 2e-6
    if k == 64 and not half:  # fp64, and accumulation into a C that is not zero
        dev = csr.device
        C0 = torch.from_numpy(rng.standard_normal((m, k))).to(dev)
        C = C0.clone()
        rode_sddmm_hip.spmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                    csr.row_offsets, csr.column_indices, csr.values.double(), m, n,
                                    torch.from_numpy(B).to(dev).double(), out=C, plan=csr.plan)
        aligned = np.diff(rp) + rp[:-1] % 4
        kept = (aligned >= 32) | (aligned == 0)  # long rows are added to, rows in no list untouched, short rows overwritten
        want = oracle.spmm_f64(rp, col, val, B) + np.where(kept[:, None], C0.cpu().numpy(), 0.0)
        assert np.abs(C.cpu().numpy() - want).max() <= 1e-12 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("m,half", [(400, False), (9000, True)])
def test_runs_that_shift_from_row_to_row(m, half):
    """A window that moves eight columns per row: the four runs of a group start 0, 8, 16 and
    24 columns into the range they cover, and every row is left out of the kernels' walk at
    the columns it does not have.  400 rows: a workgroup per group; 9000 rows: a wave per group."""
    import oracle
    from gpu_common import TOL_F16, TOL_F32, make_csr, round_half, run_sddmm, run_spmm
    from helpers import spmm_row_l1_error, sddmm_row_l1_errors
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(m)
    k, window = 64, 200
    n = 8 * m + window
    rows = [np.array(sorted(set(range(8 * r, 8 * r + window)) | set(rng.choice(n, 10, replace=False).tolist())), dtype=np.int32)
            for r in range(m)]
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum([len(c) for c in rows])
    col = np.concatenate(rows)
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    csr = make_csr(rp, col, val, m, n, k, locality=True)
    assert isinstance(csr.plan, rode_sddmm_hip.GroupPlan) and (csr.plan.counts[1] >= 2048 if m > 8192 else 64 <= csr.plan.counts[1] < 128)
    desc = csr.plan.groups()
    g = np.nonzero(desc[:, 1] > 0)[0][0]
    heads = int(desc[g, 6]) & 0xffffffff
    assert sorted((heads >> (8 * r)) & 255 for r in range(4))[-1] >= 24 and desc[g, 1] >= window + 24
    B = rng.standard_normal((n, k)).astype(np.float32)
    L = rng.standard_normal((m, k)).astype(np.float32)
    Bq, Lq = (round_half(B), round_half(L)) if half else (B, L)
    tol = TOL_F16 if half else TOL_F32
    assert spmm_row_l1_error(run_spmm(csr, B, half), oracle.spmm_f64(rp, col, val, Bq)) <= tol
    ref64, scale = oracle.sddmm_f64(rp, col, val, Lq, Bq, with_abs=True)
    err, cond = sddmm_row_l1_errors(run_sddmm(csr, L, B, half), ref64, scale, rp)
    assert float(err[cond <= 100].max(initial=0.0)) <= tol
    if m > 8192:  # the fused attention forward on the same pattern, against the three kernels without a plan
        from rode_amd import sparse_attention
        plain = make_csr(rp, col, val, m, n, k, locality=False)
        dev = csr.device
        dt = torch.float16 if half else torch.float32
        q = torch.from_numpy(L).to(dev, dt)
        kk = torch.from_numpy(B).to(dev, dt)
        vv = torch.from_numpy(rng.standard_normal((n, k)).astype(np.float32)).to(dev, dt)
        a = sparse_attention(csr, q, kk, vv, scale=0.3, fused=True)
        b = sparse_attention(plain, q, kk, vv, scale=0.3, fused=False)
        assert (a - b).abs().max().item() <= 2e-3 * max(1.0, b.abs().max().item())


@pytest.mark.parametrize("k,half", [(64, False), (64, True), (48, False), (72, True), (32, False), (128, False)])
def test_one_wave_per_group(k, half):
    """From 128 groups with a run on, a group is the work of one wave instead of one
    workgroup (no sums through LDS): the same checks on a matrix with about 2250 such groups,
    at widths that fill a lane tile and at widths that do not (48, 72)."""
    import oracle
    from gpu_common import TOL_F16, TOL_F32, make_csr, round_half, run_sddmm, run_spmm
    from helpers import spmm_row_l1_error, sddmm_row_l1_errors
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(11)
    m, n = 12002, 12500
    rp, col, val = _window_matrix(rng, m, n, 96, 6)
    csr = make_csr(rp, col, val, m, n, k, locality=True)
    assert isinstance(csr.plan, rode_sddmm_hip.GroupPlan) and csr.plan.counts[1] >= 2048
    assert 0 < csr.plan.counts[2] < m   # some rows are left to the other kernels
    B = rng.standard_normal((n, k)).astype(np.float32)
    L = rng.standard_normal((m, k)).astype(np.float32)
    Bq, Lq = (round_half(B), round_half(L)) if half else (B, L)
    tol = TOL_F16 if half else TOL_F32
    assert spmm_row_l1_error(run_spmm(csr, B, half), oracle.spmm_f64(rp, col, val, Bq)) <= tol
    ref64, scale = oracle.sddmm_f64(rp, col, val, Lq, Bq, with_abs=True)
    err, cond = sddmm_row_l1_errors(run_sddmm(csr, L, B, half), ref64, scale, rp)
    assert float(err[cond <= 100].max(initial=0.0)) <= tol


def test_every_nonzero_has_one_owner_and_what_is_refused():
    import ctypes
    from gpu_common import DEV, make_csr
    from rode_amd import _lib, rode_sddmm_hip
    lib = _lib.load()
    rng = np.random.default_rng(9)
    m, n, k = 400, 1200, 64
    rp, col, val = _window_matrix(rng, m, n, 256, 16)
    csr = make_csr(rp, col, val, m, n, k, locality=False)
    plan = rode_sddmm_hip.group_plan(csr.row_offsets, csr.column_indices, m)
    assert plan.usable
    L = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(DEV)
    B = torch.from_numpy(rng.standard_normal((n, k)).astype(np.float32)).to(DEV)

    def plans(groups=True, hub=False):
        p = _lib.Plans()
        if groups:
            p.groups, p.group_counts = plan.data.data_ptr(), ctypes.addressof(plan._header)
        if hub:
            p.hub, p.hub_counts = plan.data.data_ptr(), ctypes.addressof(plan._header)
        return p

    def sddmm(flags, p):
        out = torch.full((len(val),), float("nan"), device=DEV)
        code = lib.rode_hip_sddmm_planned(0, flags, csr.m1, csr.m2, n, k, csr.block_indices.data_ptr(),
                                          csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(),
                                          csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(), csr.values.data_ptr(),
                                          L.data_ptr(), B.data_ptr(), out.data_ptr(), ctypes.byref(p), None, None)
        torch.cuda.synchronize()
        return code, out

    code, plain = sddmm(0, plans(False))
    code2, grouped = sddmm(0, plans())
    assert code == 0 and code2 == 0 and not torch.isnan(grouped).any()
    assert (grouped - plain).abs().max().item() <= 2e-5 * plain.abs().max().item()
    written = [~torch.isnan(sddmm(f, plans())[1]) for f in (_lib.SPMM_ONLY_BLOCK, _lib.SPMM_ONLY_RESIDUE, _lib.SPMM_ONLY_HUB)]
    assert (written[0].int() + written[1].int() + written[2].int() == 1).all()
    assert sddmm(0, plans(True, True))[0] != 0   # a group plan next to a hub plan

    def spmm(flags, p):
        C = torch.zeros(m, k, device=DEV)
        code = lib.rode_hip_spmm_planned(0, flags, csr.m1, csr.m2, n, k, csr.values.data_ptr(), csr.column_indices.data_ptr(),
                                         csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(),
                                         csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(), B.data_ptr(),
                                         C.data_ptr(), ctypes.byref(p), None, None)
        torch.cuda.synchronize()
        return code, C

    code, plain_c = spmm(_lib.SPMM_WHOLE_LISTS, plans(False))
    parts = [spmm(_lib.SPMM_WHOLE_LISTS | f, plans()) for f in (_lib.SPMM_ONLY_BLOCK, _lib.SPMM_ONLY_RESIDUE, _lib.SPMM_ONLY_HUB)]
    assert code == 0 and all(c == 0 for c, _ in parts)
    assert (sum(p for _, p in parts) - plain_c).abs().max().item() <= 2e-5 * plain_c.abs().max().item()
    assert spmm(0, plans())[0] != 0  # a group plan without the whole-lists promise

    # the attention entry point refuses a group plan made for another number of rows
    q = torch.zeros(m + 8, k, device=DEV)
    o = torch.zeros(m + 8, k, device=DEV)
    rp8 = torch.cat([csr.row_offsets, csr.row_offsets[-1:].repeat(8)])
    p = plans()
    args = (0, None, k, rp8.data_ptr(), csr.column_indices.data_ptr(), csr.values.data_ptr(), q.data_ptr(), B.data_ptr(),
            B.data_ptr(), ctypes.c_float(1.0), o.data_ptr(), None, ctypes.byref(p), None)
    assert lib.rode_hip_attention_forward(args[0], m + 8, *args[2:]) != 0
    assert lib.rode_hip_attention_forward(args[0], m, *args[2:]) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("d,half,m,window", [(64, False, 12002, 96), (64, True, 12002, 96), (128, False, 12002, 96),
                                             (32, True, 12002, 96), (32, False, 10000, 600)])
def test_fused_attention_of_groups(d, half, m, window):
    """rode_hip_attention_forward with a group plan of at least 2048 groups with a run (one
    wave per group: scores of the run for four rows at once, then their softmax, then P.V
    over the run) against fp64 on the host and against the same entry point without a plan;
    rows in no kept group, rows with holes, empty rows and short rows are all in the matrix.
    The last case has runs of more than 512 columns: the raw scores past the first 512 wait
    in the output array instead of LDS."""
    from gpu_common import DEV, make_csr
    from rode_amd import rode_sddmm_hip
    from rode_amd.autograd import _attention_call
    rng = np.random.default_rng(40 + d)
    n = m + 498
    rp, col, val = _window_matrix(rng, m, n, window, 6)
    val = rng.uniform(0.5, 1.5, len(col)).astype(np.float32)
    mask = make_csr(rp, col, val, m, n, d, locality=True)
    assert isinstance(mask.plan, rode_sddmm_hip.GroupPlan) and mask.plan.counts[1] >= 2048
    plain = make_csr(rp, col, val, m, n, d, locality=False)
    assert plain.plan is None
    dt = torch.float16 if half else torch.float32
    mk = lambda r, s: torch.from_numpy((s * rng.standard_normal((r, d))).astype(np.float32)).to(DEV, dt)
    q, k, v = mk(m, 1.2), mk(n, 1.2), mk(n, 1.0)
    scale = 0.4
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
    q64, k64, v64 = (t.double().cpu().numpy() for t in (q, k, v))
    lens = np.diff(rp)
    rows = np.repeat(np.arange(m), lens)
    sc = scale * val.astype(np.float64) * np.einsum("ij,ij->i", q64[rows], k64[col])
    top = np.full(m, -np.inf)
    np.maximum.at(top, rows, sc)
    e = np.exp(sc - top[rows])
    den = np.zeros(m)
    np.add.at(den, rows, e)
    ref_p = e / den[rows]
    ref_out = np.zeros((m, d))
    np.add.at(ref_out, rows, ref_p[:, None] * v64[col])
    tol = 2e-3 if half else 5e-5
    assert np.abs(probs.cpu().numpy() - ref_p).max() <= tol
    assert np.abs(out.cpu().numpy() - ref_out).max() <= tol * max(1.0, np.abs(ref_out).max())
    assert not out[torch.from_numpy(lens == 0).to(DEV)].any()
    out2, probs2, _ = _attention_call(plain, plain.values, q, k, v, scale, "probs")
    assert (out - out2).abs().max().item() <= tol * max(1.0, out2.abs().max().item())
    assert (probs - probs2).abs().max().item() <= tol


def _shifted_windows(m, shift, width, extra, seed):
    """Row r has the run [shift * r, shift * r + width) plus `extra` random columns: inside a
    group of four rows the runs start `shift` columns apart, so every group's range has
    columns that only some of its rows own."""
    rng = np.random.default_rng(seed)
    n = shift * m + width + 64
    rows = [np.union1d(np.arange(shift * r, shift * r + width), rng.choice(n, extra, replace=False)).astype(np.int32)
            for r in range(m)]
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum([len(c) for c in rows])
    return n, rp, np.concatenate(rows), rng.uniform(0.5, 1.5, rp[-1]).astype(np.float32)


@pytest.mark.parametrize("m", [400, 8400], ids=["workgroup_per_group", "wave_per_group"])
def test_non_finite_dense_rows_stay_in_the_rows_that_reference_them(m):
    """The group kernels load every dense row of a group's range for all four rows.  A row
    whose own run does not hold a column must not see that column's dense row: Inf there may
    only reach the rows that reference it (as in the list kernels and the reference)."""
    from gpu_common import DEV, make_csr
    from rode_amd import rode_sddmm_hip, rode_spmm, sparse_attention
    shift, width, d = 3, 200, 64
    n, rp, col, val = _shifted_windows(m, shift, width, 4, seed=m)
    csr = make_csr(rp, col, val, m, n, d)
    assert isinstance(csr.plan, rode_sddmm_hip.GroupPlan) and csr.plan.counts[1] == m // 4
    assert (csr.plan.counts[1] >= 128) == (m == 8400)
    # columns at the head of a range (owned by the group's first row only) and at its tail
    # (owned by its last row only), in every 50th group (a column is in the runs of 67 rows)
    groups = np.arange(0, m // 4, 50)
    bad = np.concatenate([4 * shift * groups + 1, 4 * shift * groups + 3 * shift + width - 1])
    touched = np.zeros(m, dtype=bool)
    touched[np.repeat(np.arange(m), np.diff(rp))[np.isin(col, bad)]] = True
    assert touched[4 * groups].all() and touched[4 * groups + 3].all()
    # the rows this test is about: inside such a group, not referencing the column (but for a stray random one)
    assert (~touched[4 * groups + 1]).sum() + (~touched[4 * groups + 2]).sum() >= len(groups)
    g = torch.Generator(device=DEV).manual_seed(1)
    B = torch.randn(n, d, device=DEV, generator=g)
    B[torch.from_numpy(bad).to(DEV)] = float("inf")
    C = rode_spmm(csr, B).cpu().numpy()
    assert np.isfinite(C[~touched]).all(), "a non-finite dense row reached rows that do not reference it"
    assert (~np.isfinite(C[touched])).any(axis=1).all()
    q, k = torch.randn(m, d, device=DEV, generator=g), torch.randn(n, d, device=DEV, generator=g)
    out = sparse_attention(csr, q, k, B, fused=True).cpu().numpy()
    assert np.isfinite(out[~touched]).all(), "a non-finite row of v reached rows that do not attend to it"
    assert (~np.isfinite(out[touched])).any(axis=1).all()


@pytest.mark.parametrize("d,half", [(64, False), (64, True), (128, False), (32, True)])
def test_fused_attention_gradients_of_groups(d, half):
    """The two gradient kernels with group plans of at least 2048 kept groups on the pattern
    (row pass: attention_backward_group_kernel) and on its transpose (column pass:
    attention_backward_cols_group_kernel), rows and columns outside kept groups included,
    against dense fp64 autograd and against the chain of separate kernels."""
    from gpu_common import DEV, make_csr
    from rode_amd import autograd, rode_sddmm_hip, sparse_attention
    from test_gpu_attention import _dense
    rng = np.random.default_rng(70 + d)
    m, window = 12002, 96
    n = m + 498
    rp, col, _ = _window_matrix(rng, m, n, window, 6, ragged=False)
    # a few irregular rows, far enough apart that most runs of rows survive in the transposed
    # pattern too: a hole in the window, an empty row, a short row without a run
    rows = [col[rp[r]:rp[r + 1]] for r in range(m)]
    for r in range(5, m, 997):
        rows[r] = np.concatenate([rows[r][:20], rows[r][23:]])
    for r in range(7, m, 1001):
        rows[r] = rows[r][:0]
    for r in range(9, m, 1499):
        rows[r] = np.sort(rng.choice(n, 5, replace=False)).astype(np.int32)
    rp = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(0.5, 1.5, len(col)).astype(np.float32)
    mask = make_csr(rp, col, val, m, n, d, locality=True)
    mask_t, _ = mask.transpose(with_values=False)
    for c in (mask, mask_t):
        assert isinstance(c.plan, rode_sddmm_hip.GroupPlan) and c.plan.counts[1] >= 2048 and c.plan.counts[2] > 0
    dt = torch.float16 if half else torch.float32
    mk = lambda r, s: torch.from_numpy((s * rng.standard_normal((r, d))).astype(np.float32)).to(DEV, dt)
    q, k, v = mk(m, 1.2).requires_grad_(), mk(n, 1.2).requires_grad_(), mk(n, 1.0).requires_grad_()
    w = mk(m, 1.0).float() * 1e-3  # small gradients: fp16 operands must not lose them
    scale = 0.4
    grads = {}
    for fused_backward in (True, False):
        autograd.FUSED_BACKWARD = fused_backward
        try:
            q.grad = k.grad = v.grad = None
            out = sparse_attention(mask, q, k, v, scale=scale, fused=True)
            (out * w).sum().backward()
        finally:
            autograd.FUSED_BACKWARD = "auto"
        grads[fused_backward] = (q.grad.clone(), k.grad.clone(), v.grad.clone())
    # the gradient entry points take either form of what the forward call kept: probabilities,
    # or scaled scores with every row's (maximum, 1 / sum)
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    g_out = w.contiguous()
    kept = {}
    for keep in ("probs", "scores"):
        out_k, per_nonzero, stats = autograd._attention_call(mask, mask.values, qd, kd, vd, scale, keep)
        kept[keep] = autograd._attention_backward_call(mask, mask_t, mask.transposed_slots(), per_nonzero, stats, g_out,
                                                       out_k, qd, kd, vd, scale)
    for a, b in zip(kept["probs"], kept["scores"]):
        assert (a - b).abs().max().item() <= 1e-5 * b.abs().max().item()
    q64, k64, v64 = (t.detach().double().requires_grad_() for t in (q, k, v))
    A = _dense(rp, col, val, m, n)
    has = torch.from_numpy(np.diff(rp) > 0).to(DEV)
    scores = (q64 @ k64.t()) * A * scale
    probs = torch.softmax(scores.masked_fill(A == 0, float("-inf"))[has], dim=1)  # (rows without nonzeros attend to nothing)
    ((probs @ v64) * w.double()[has]).sum().backward()
    tol = 3e-3 if half else 2e-5
    for got, chained, want in zip(grads[True], grads[False], (q64.grad, k64.grad, v64.grad)):
        bound = tol * want.abs().max().item()
        assert (got.double() - want).abs().max().item() <= bound
        assert (got.double() - chained.double()).abs().max().item() <= 2 * bound
