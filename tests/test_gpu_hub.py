"""Hub plan: rows with thousands of nonzeros are processed column slab by column slab by
kernels of their own (rode_hub.hip, spmm_hub_kernel, sddmm_hub_kernel).  The plan changes
where dense rows are found, never a result: everything here is checked against the fp64
oracle with the tolerances of the unplanned kernels."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _matrix(rng, m, n, hub_lens, sort_hubs=True, mean_len=20):
    """Short rows plus a few very long ones (sorted columns unless asked otherwise)."""
    lens = rng.poisson(mean_len, m)
    where = rng.choice(m, len(hub_lens), replace=False)
    lens[where] = hub_lens
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum(lens)
    col = np.empty(rp[-1], dtype=np.int32)
    for r in range(m):
        c = rng.choice(n, lens[r], replace=False)
        col[rp[r]:rp[r + 1]] = np.sort(c) if (sort_hubs or lens[r] < 1000) else c
    val = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    return rp, col, val, np.sort(where)


def test_plan_contents():
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(0)
    m, n = 3000, 50000
    rp, col, val, where = _matrix(rng, m, n, [5000, 9000, 4096, 4095, 20000])
    dev = torch.device("cuda:0")
    plan = rode_sddmm_hip.hub_plan(torch.from_numpy(rp).to(dev), torch.from_numpy(col).to(dev), m, n, 4096)
    lens = np.diff(rp) + rp[:-1] % 4
    hubs = np.nonzero(lens >= 4096)[0]
    assert plan.usable and plan.counts[0] == len(hubs) and plan.counts[1] == (n + 2047) // 2048 and plan.counts[2] == 4096
    assert np.array_equal(plan.hub_rows(), hubs)
    pieces = plan.pieces()
    for h, r in enumerate(hubs):
        c = col[rp[r]:rp[r + 1]]
        want = rp[r] + np.searchsorted(c, np.arange(plan.counts[1] + 1) * 2048, side="left")
        want[-1] = rp[r + 1]
        assert np.array_equal(pieces[h], want)
    # a hub row whose columns do not ascend makes the plan unusable
    rp2, col2, _, _ = _matrix(rng, 500, 40000, [6000], sort_hubs=False)
    bad = rode_sddmm_hip.hub_plan(torch.from_numpy(rp2).to(dev), torch.from_numpy(col2).to(dev), 500, 40000, 4096)
    assert bad.counts[0] == 1 and not bad.usable
    # no hub rows at all
    none = rode_sddmm_hip.hub_plan(torch.from_numpy(rp2).to(dev), torch.from_numpy(col2).to(dev), 500, 40000, 100000)
    assert none.counts[0] == 0 and not none.usable


@pytest.mark.parametrize("k,half", [(128, False), (64, False), (32, False), (128, True), (200, False)])
def test_hub_rows_against_oracle(k, half):
    """A matrix whose long rows the hub kernels take (min_len lowered so that pieces of one
    nonzero, empty pieces and pieces of hundreds occur), every width class and fp16."""
    import oracle
    from gpu_common import TOL_F16, TOL_F32, make_csr, round_half, run_sddmm, run_spmm
    from helpers import spmm_row_l1_error, sddmm_row_l1_errors
    from rode_amd import RoDeCSR, rode_sddmm_hip
    rng = np.random.default_rng(k)
    m, n = 2000, 70000
    rp, col, val, where = _matrix(rng, m, n, [5000, 300, 64, 12000, 700, 65, 33000])
    old = RoDeCSR.HUB_MIN_LEN, RoDeCSR.HUB_MIN_SLABS, RoDeCSR.HUB_MIN_SHARE
    RoDeCSR.HUB_MIN_LEN, RoDeCSR.HUB_MIN_SLABS, RoDeCSR.HUB_MIN_SHARE = 64, 1, 0.0
    try:
        csr = make_csr(rp, col, val, m, n, k)
    finally:
        RoDeCSR.HUB_MIN_LEN, RoDeCSR.HUB_MIN_SLABS, RoDeCSR.HUB_MIN_SHARE = old
    assert isinstance(csr.plan, rode_sddmm_hip.HubPlan) and csr.plan.usable
    assert csr.plan.counts[2] == max(64, 8 * ((n + 4095) // 4096)) and csr.plan.counts[0] >= 5
    B = rng.standard_normal((n, k)).astype(np.float32)
    L = rng.standard_normal((m, k)).astype(np.float32)
    Bq, Lq = (round_half(B), round_half(L)) if half else (B, L)
    tol = TOL_F16 if half else TOL_F32
    assert spmm_row_l1_error(run_spmm(csr, B, half), oracle.spmm_f64(rp, col, val, Bq)) <= tol
    if k == 64:  # fp64 through the same plan, and accumulation into a C that is not zero
        from rode_amd import rode_sddmm_hip
        dev = csr.device
        C0 = torch.from_numpy(rng.standard_normal((m, k))).to(dev)
        C = C0.clone()
        rode_sddmm_hip.spmm_forward(csr.block_indices, csr.residue_indices, csr.st_offsets, csr.m1, csr.m2,
                                    csr.row_offsets, csr.column_indices, csr.values.double(), m, n,
                                    torch.from_numpy(B).to(dev).double(), out=C, plan=csr.plan)
        ref = oracle.spmm_f64(rp, col, val, B)
        added = (np.diff(rp) + rp[:-1] % 4) >= 32  # long rows are added to, short rows overwritten
        want = ref + np.where(added[:, None], C0.cpu().numpy(), 0.0)
        assert spmm_row_l1_error(C.cpu().numpy(), want) <= 1e-12
    ref64, scale = oracle.sddmm_f64(rp, col, val, Lq, Bq, with_abs=True)
    out = run_sddmm(csr, L, B, half)
    err, cond = sddmm_row_l1_errors(out, ref64, scale, rp)
    assert float(err[cond <= 100].max(initial=0.0)) <= tol
    if not half:
        assert (np.abs(out - ref64) / np.maximum(scale, 1e-30)).max() <= 2e-6


@pytest.mark.parametrize("k", [64, 32])
def test_hub_plan_through_the_c_abi(k):
    """The planned entry points with a hub plan against the same calls without one; the
    atomic fallback of SpMM (no workspace); what is refused.  (k = 32: rows of one 128-byte
    tile, for which a locality plan is ignored - a hub plan and the flags are not.)"""
    import ctypes
    from gpu_common import DEV, make_csr
    from rode_amd import RoDeCSR, _lib, rode_sddmm_hip
    lib = _lib.load()
    rng = np.random.default_rng(3)
    m, n = 1500, 40000
    rp, col, val, _ = _matrix(rng, m, n, [4500, 8000, 2000])
    csr = make_csr(rp, col, val, m, n, k, locality=False)
    assert csr.plan is None
    plan = rode_sddmm_hip.hub_plan(csr.row_offsets, csr.column_indices, m, n, 2000)
    assert plan.usable and plan.counts[0] == 3
    B = torch.from_numpy(rng.standard_normal((n, k)).astype(np.float32)).to(DEV)
    L = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(DEV)

    def plans(hub, ws=None, window=None):
        p = _lib.Plans()
        if hub:
            p.hub, p.hub_counts = plan.data.data_ptr(), ctypes.addressof(plan._header)
        if ws is not None:
            p.hub_workspace, p.hub_workspace_bytes = ws.data_ptr(), ws.numel()
        if window is not None:
            p.window, p.window_rows = window.data_ptr(), window.data_ptr()
        return p

    def spmm(flags, hub, ws):
        C = torch.zeros(m, k, device=DEV)
        code = lib.rode_hip_spmm_planned(0, flags, csr.m1, csr.m2, n, k, csr.values.data_ptr(), csr.column_indices.data_ptr(),
                                         csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(),
                                         csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(), B.data_ptr(),
                                         C.data_ptr(), ctypes.byref(plans(hub, ws)), None, None)
        torch.cuda.synchronize()
        return code, C

    code, plain = spmm(_lib.SPMM_WHOLE_LISTS, False, None)
    assert code == 0
    ws = plan.workspace(k, 4)
    assert ws.numel() == lib.rode_hip_hub_workspace_bytes(ctypes.addressof(plan._header), k, 4) > 0
    scale = plain.abs().max().item()
    for workspace in (ws, None, ws[: ws.numel() // 2]):  # partial rows; atomics; too small a workspace -> atomics
        code, got = spmm(_lib.SPMM_WHOLE_LISTS, True, workspace)
        assert code == 0 and (got - plain).abs().max().item() <= 2e-5 * scale
    # the three kernel families one by one add up to the whole
    parts = [spmm(_lib.SPMM_WHOLE_LISTS | f, True, ws) for f in (_lib.SPMM_ONLY_BLOCK, _lib.SPMM_ONLY_RESIDUE, _lib.SPMM_ONLY_HUB)]
    assert all(c == 0 for c, _ in parts)
    assert (sum(p for _, p in parts) - plain).abs().max().item() <= 2e-5 * scale
    # refused: a hub plan without the whole-lists promise, two ONLY bits, a hub plan next to a locality plan
    assert spmm(0, True, ws)[0] != 0
    assert spmm(_lib.SPMM_WHOLE_LISTS | _lib.SPMM_ONLY_BLOCK | _lib.SPMM_ONLY_HUB, True, ws)[0] != 0

    def sddmm(flags, hub, window=None):
        out = torch.full((len(val),), float("nan"), device=DEV)
        code = lib.rode_hip_sddmm_planned(0, flags, csr.m1, csr.m2, n, k, csr.block_indices.data_ptr(),
                                          csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(),
                                          csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(), csr.values.data_ptr(),
                                          L.data_ptr(), B.data_ptr(), out.data_ptr(), ctypes.byref(plans(hub, None, window)),
                                          None, None)
        torch.cuda.synchronize()
        return code, out

    code, plain_out = sddmm(0, False)
    code2, hub_out = sddmm(0, True)
    assert code == 0 and code2 == 0 and not torch.isnan(hub_out).any()
    assert (hub_out - plain_out).abs().max().item() <= 2e-5 * plain_out.abs().max().item()
    # every output is written by exactly one of the three kernel families
    written = [~torch.isnan(sddmm(f, True)[1]) for f in (_lib.SPMM_ONLY_BLOCK, _lib.SPMM_ONLY_RESIDUE, _lib.SPMM_ONLY_HUB)]
    assert (written[0].int() + written[1].int() + written[2].int() == 1).all()
    fake = torch.zeros(64, dtype=torch.int32, device=DEV)
    assert sddmm(0, True, fake)[0] != 0
