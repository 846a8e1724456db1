"""The entry points queue work and allocate nothing, so a caller can record them into
a HIP graph; replays must reproduce the eager result every time.  Also: a Matrix
Market file through the whole path."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_hip_graph_replays_match_eager():
    from gpu_common import DEV, make_csr
    from helpers import random_csr
    from rode_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(0)
    m, n, k = 3000, 2500, 64
    rp, col, val = random_csr(rng, m, n, 40, long_rows=6, long_len=2000, empty_frac=0.1)
    csr = make_csr(rp, col, val, m, n, k)
    B = torch.randn(n, k, device=DEV)
    L = torch.randn(m, k, device=DEV)
    C = torch.zeros(m, k, device=DEV)
    out = torch.zeros(csr.nnz, device=DEV)

    def step(stream):
        C.zero_()  # a fill kernel, not a memset node
        _lib.check(lib.rode_hip_spmm_f32(csr.m1, csr.m2, n, k, csr.values.data_ptr(), csr.column_indices.data_ptr(),
                                         csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(),
                                         csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(), B.data_ptr(),
                                         C.data_ptr(), stream, stream), "spmm")
        _lib.check(lib.rode_hip_sddmm_f32(csr.m1, csr.m2, n, k, csr.block_indices.data_ptr(),
                                          csr.residue_indices.data_ptr(), csr.st_offsets.data_ptr(),
                                          csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(),
                                          csr.values.data_ptr(), L.data_ptr(), B.data_ptr(), out.data_ptr(),
                                          stream, stream), "sddmm")

    step(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    out_eager = out.clone()
    c_scale = C.abs().max().item()
    c_eager = C.clone()

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(4):
        # eager work and a synchronisation between replays; new operand values each time
        B.mul_(-1.0 if replay % 2 else 1.0)
        out.fill_(float("nan"))
        C.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        sign = -1.0 if replay % 2 else 1.0
        B.mul_(sign)  # restore
        assert torch.equal(out, out_eager * sign), f"replay {replay}: SDDMM differs"
        # SpMM sums with atomics, whose order may change between runs
        assert (C - c_eager * sign).abs().max().item() <= 1e-5 * c_scale, f"replay {replay}: SpMM differs"


def test_hip_graph_replays_of_the_attention_step():
    """The attention forward and its two gradient kernels allocate nothing either: recorded into
    one graph and replayed on new operands, against the eager calls."""
    import ctypes
    from gpu_common import DEV, make_csr
    from test_gpu_group import _window_matrix
    from rode_amd import _lib, rode_sddmm_hip
    lib = _lib.load()
    rng = np.random.default_rng(3)
    m, d = 6000, 64
    n = m + 300
    rp, col, val = _window_matrix(rng, m, n, 96, 6)
    val = rng.uniform(0.5, 1.5, len(col)).astype(np.float32)
    csr = make_csr(rp, col, val, m, n, d, locality=True)
    csr_t, _ = csr.transpose(with_values=False)
    t_slot = csr.transposed_slots()
    nnz = csr.nnz
    gen = torch.Generator(device=DEV).manual_seed(9)
    q, k, v, g = (torch.randn(r, d, device=DEV, generator=gen) for r in (m, n, n, m))
    out, kept, stats = torch.empty(m, d, device=DEV), torch.empty(nnz, device=DEV), torch.empty(m, 2, device=DEV)
    dq, dk, dv = torch.empty(m, d, device=DEV), torch.empty(n, d, device=DEV), torch.empty(n, d, device=DEV)
    pairs = torch.empty(2 * nnz, device=DEV)
    group = lambda c: c.plan if isinstance(c.plan, rode_sddmm_hip.GroupPlan) else None
    plans, plans_t = rode_sddmm_hip.plans_struct(group(csr)), rode_sddmm_hip.plans_struct(group(csr_t))
    kind = _lib.DENSE_CODE["f32"]

    def step(s):
        _lib.check(lib.rode_hip_attention_forward_batched(
            kind, 1, m, n, nnz, d, csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(), csr.values.data_ptr(),
            q.data_ptr(), k.data_ptr(), v.data_ptr(), 0.3, out.data_ptr(), kept.data_ptr(), stats.data_ptr(),
            ctypes.byref(plans), s), "forward")
        _lib.check(lib.rode_hip_attention_backward_rows(
            kind, 1, m, n, nnz, d, csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(), csr.values.data_ptr(),
            kept.data_ptr(), stats.data_ptr(), g.data_ptr(), out.data_ptr(), k.data_ptr(), v.data_ptr(), 0.3,
            t_slot.data_ptr(), dq.data_ptr(), pairs.data_ptr(), ctypes.byref(plans), s), "rows")
        _lib.check(lib.rode_hip_attention_backward_cols(
            kind, 1, m, n, nnz, d, csr_t.row_offsets.data_ptr(), csr_t.column_indices.data_ptr(), pairs.data_ptr(),
            g.data_ptr(), q.data_ptr(), dk.data_ptr(), dv.data_ptr(), ctypes.byref(plans_t), s), "cols")

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        q.copy_(torch.randn(m, d, device=DEV, generator=gen))  # new operands, eager work between the replays
        g.mul_(0.5)
        step(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want = [t.clone() for t in (out, dq, dk, dv)]
        for t in (out, dq, dk, dv, kept, pairs):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(("out", "dq", "dk", "dv"), (out, dq, dk, dv), want):
            assert torch.equal(got, ref), f"replay {replay}: {name} differs"


def test_matrix_market_file_through_the_path(tmp_path):
    import scipy.io
    import scipy.sparse as sp

    import oracle
    from gpu_common import make_csr, run_sddmm, run_spmm
    from helpers import spmm_row_l1_error
    from rode_amd import io as rio
    A = sp.random(700, 900, density=0.05, random_state=3, format="coo", dtype=np.float64)
    path = tmp_path / "m.mtx"
    scipy.io.mmwrite(str(path), A)
    m, n, rp, col, val = rio.read_matrix_market(path)
    rng = np.random.default_rng(1)
    B = rng.standard_normal((n, 32)).astype(np.float32)
    for rp_, col_, val_ in ((rp, col, val), rio.pad_rows(rp, col, val, 4)):
        csr = make_csr(rp_, col_, val_, m, n, 32)
        assert spmm_row_l1_error(run_spmm(csr, B), oracle.spmm_f64(rp_, col_, val_, B)) <= 1e-4
        lhs = rng.standard_normal((m, 32)).astype(np.float32)
        got = run_sddmm(csr, lhs, B)
        ref, scale = oracle.sddmm_f64(rp_, col_, val_, lhs, B, with_abs=True)
        assert np.max(np.abs(got - ref) / np.maximum(scale, 1e-30), initial=0.0) <= 2e-6
        assert not got[val_ == 0].any()  # padding entries produce zeros


def _transpose_reference(rp, col, m, n):
    """Stable sort by column on the host: (row_offsets_t, rows in that order, perm)."""
    rows = np.repeat(np.arange(m, dtype=np.int64), np.diff(rp))
    perm = np.argsort(col, kind="stable")
    rp_t = np.zeros(n + 1, dtype=np.int64)
    rp_t[1:] = np.cumsum(np.bincount(col, minlength=n))
    return rp_t, rows[perm], perm


@pytest.mark.parametrize("m,n,mean_len,seed", [
    (1, 1, 1, 0), (7, 5, 3, 1), (300, 17, 9, 2), (257, 70000, 40, 3), (5000, 4097, 30, 4), (40, 1 << 20, 500, 5),
])
def test_csr_transpose_is_the_stable_sort_by_column(m, n, mean_len, seed):
    """rode_hip_csr_transpose against numpy's stable argsort, exactly: one to six radix
    passes (n from 1 to 2^20), columns without nonzeros at both ends and in the middle,
    duplicate (row, column) entries (their input order is kept), empty rows."""
    from rode_amd import rode_sddmm_hip
    rng = np.random.default_rng(seed)
    lens = rng.poisson(mean_len, m)
    lens[rng.integers(0, m, max(1, m // 10))] = 0
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum(lens)
    lo, hi = (n // 8, n - n // 8) if n > 16 else (0, n)   # the first and last columns stay empty
    col = rng.integers(lo, max(hi, lo + 1), rp[-1]).astype(np.int32)   # with repetitions inside a row
    dev = torch.device("cuda:0")
    got = rode_sddmm_hip.csr_transpose(torch.from_numpy(rp).to(dev), torch.from_numpy(col).to(dev), m, n)
    want = _transpose_reference(rp, col, m, n)
    for g, w, name in zip(got, want, ("row_offsets_t", "column_indices_t", "perm")):
        assert g.dtype == torch.int32 and np.array_equal(g.cpu().numpy().astype(np.int64), w), name


def test_csr_transpose_edges_and_full_size():
    from rode_amd import _lib, rode_sddmm_hip, workloads
    dev = torch.device("cuda:0")
    # no nonzeros: offsets all zero
    rp = torch.zeros(6, dtype=torch.int32, device=dev)
    rp_t, col_t, perm = rode_sddmm_hip.csr_transpose(rp, torch.empty(0, dtype=torch.int32, device=dev), 5, 9)
    assert rp_t.shape == (10,) and not rp_t.any() and col_t.numel() == 0 and perm.numel() == 0
    # a workspace that is too small is refused
    lib = _lib.load()
    one = torch.zeros(2, dtype=torch.int32, device=dev)
    assert lib.rode_hip_csr_transpose(1, 1, 1, one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(),
                                      one.data_ptr(), one.data_ptr(), 8, None) != 0
    # the power-law benchmark pattern, 2 M x 2 M with 47.9 M nonzeros
    m, n, rp, col, val = workloads.config("c4_powerlaw")
    got = rode_sddmm_hip.csr_transpose(torch.from_numpy(rp).to(dev), torch.from_numpy(col).to(dev), m, n)
    want = _transpose_reference(rp, col, m, n)
    for g, w, name in zip(got, want, ("row_offsets_t", "column_indices_t", "perm")):
        assert np.array_equal(g.cpu().numpy().astype(np.int64), w), name


@pytest.mark.gpu
def test_permute_values():
    """rode_hip_permute_f32: values[perm] for lengths that are and are not multiples of four,
    and what it refuses."""
    from rode_amd import _lib, rode_sddmm_hip
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(3)
    for n in (0, 1, 5, 64, 1003, 200001):
        src = torch.randn(max(n, 1), generator=g).to(dev)
        perm = torch.randperm(max(n, 1), generator=g)[:n].to(torch.int32).to(dev)
        out = rode_sddmm_hip.permute(src, perm)
        assert out.shape == (n,) and torch.equal(out, src[perm.long()])
    lib = _lib.load()
    src = torch.randn(16, device=dev)
    idx = torch.arange(16, dtype=torch.int32, device=dev)
    assert lib.rode_hip_permute_f32(16, src.data_ptr(), idx.data_ptr(), src.data_ptr(), None) != 0   # in place
    assert lib.rode_hip_permute_f32(-1, src.data_ptr(), idx.data_ptr(), src.data_ptr(), None) != 0
    with pytest.raises(RuntimeError):
        rode_sddmm_hip.permute(src, idx.long())
