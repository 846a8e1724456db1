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
