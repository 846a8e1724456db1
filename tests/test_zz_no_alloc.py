"""The allocation-free preprocessing entry point (rode_hip_preprocess_static) against
rode_hip_preprocess with a caller workspace: byte-identical arrays and counts, on two
calls in a row, the second on a smaller matrix (the fixed scratch keeps the first call's
contents)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(lib, entry, rp, seg, dev):
    m = len(rp) - 1
    nnz = int(rp[-1])
    cap = (nnz + 3 * m) // seg + m
    d_rp = torch.from_numpy(rp).to(dev)
    blk = torch.full((cap + 1,), -1, dtype=torch.int32, device=dev)
    st = torch.full((cap + 2,), -1, dtype=torch.int32, device=dev)
    res = torch.full((max(m, 1),), -1, dtype=torch.int32, device=dev)
    cnt = torch.full((2,), -1, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "static":
        code = lib.rode_hip_preprocess_static(seg, 32, 4, m, d_rp.data_ptr(), blk.data_ptr(), st.data_ptr(),
                                              res.data_ptr(), cnt.data_ptr(), cnt.data_ptr() + 4, cap, stream)
    else:
        nbytes = lib.rode_hip_preprocess_workspace_bytes(m)
        ws = torch.empty((nbytes + 7) // 8, dtype=torch.int64, device=dev)
        code = lib.rode_hip_preprocess(seg, 32, 4, m, d_rp.data_ptr(), blk.data_ptr(), st.data_ptr(), res.data_ptr(),
                                       cnt.data_ptr(), cnt.data_ptr() + 4, cap, ws.data_ptr(), nbytes, stream)
    assert code == 0, (entry, code)
    torch.cuda.synchronize()
    return blk.cpu().numpy(), st.cpu().numpy(), res.cpu().numpy(), cnt.cpu().numpy()


def test_static_scratch_entry_point_matches_workspace_entry_point():
    from helpers import random_row_ptr
    from rode_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(11)
    big = random_row_ptr(rng, 700_000, 9, long_rows=30, long_len=60_000)
    small = random_row_ptr(rng, 5_000, 40, long_rows=3, long_len=4_000) + 2  # unaligned starts
    for rp, seg in ((big, 512), (small, 32), (big, 32), (np.zeros(1, np.int32), 512)):
        print("static preprocessing: rows", len(rp) - 1, "nnz", int(rp[-1]), "seg", seg, flush=True)
        want = _run(lib, "workspace", rp, seg, dev)
        got = _run(lib, "static", rp, seg, dev)
        for a, b, name in zip(got, want, ("block_r_ind", "st_off", "residue_r_ind", "counts")):
            assert a.tobytes() == b.tobytes(), f"{name} differs (rows {len(rp) - 1}, seg {seg})"
        assert got[3][0] > 0 or len(rp) == 1


def test_static_scratch_entry_point_rejects_what_it_cannot_hold():
    from rode_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    one = torch.zeros(8, dtype=torch.int32, device=dev)
    p = one.data_ptr()
    too_many = 4194304 + 1  # RODE_HIP_STATIC_MAX_ROWS + 1: refused before any launch, so the short arrays are never read
    assert lib.rode_hip_preprocess_static(512, 32, 4, too_many, p, p, p, p, p, p + 4, 16, None) == 2
    assert b"memory" in lib.rode_hip_error_string(2).lower()
    assert lib.rode_hip_preprocess_static(0, 32, 4, 4, p, p, p, p, p, p + 4, 16, None) == 1
    assert lib.rode_hip_preprocess_static(512, 32, 4, 4, None, p, p, p, p, p + 4, 16, None) == 1


def test_static_scratch_calls_from_several_host_threads_to_one_stream():
    """Host threads that call at the same time for the same stream: every call's two launches
    are queued together, so the calls run one after the other on the GPU and each finds the
    scratch as its own fill left it."""
    import threading
    from helpers import random_row_ptr
    from rode_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(12)
    inputs = [random_row_ptr(rng, 20_000 + 7_000 * i, 12, long_rows=4, long_len=3_000) for i in range(6)]
    want = [_run(lib, "workspace", rp, 128, dev) for rp in inputs]
    stream = torch.cuda.current_stream().cuda_stream
    arrays, codes = [], [None] * len(inputs)
    for rp in inputs:
        m, nnz = len(rp) - 1, int(rp[-1])
        cap = (nnz + 3 * m) // 128 + m
        arrays.append((m, cap, torch.from_numpy(rp).to(dev), torch.full((cap + 1,), -1, dtype=torch.int32, device=dev),
                       torch.full((cap + 2,), -1, dtype=torch.int32, device=dev),
                       torch.full((m,), -1, dtype=torch.int32, device=dev), torch.full((2,), -1, dtype=torch.int32, device=dev)))
    torch.cuda.synchronize()
    start = threading.Barrier(len(inputs))

    def call(i):
        m, cap, d_rp, blk, st, res, cnt = arrays[i]
        start.wait()
        for _ in range(20):  # (ctypes releases the interpreter lock during the call)
            codes[i] = lib.rode_hip_preprocess_static(128, 32, 4, m, d_rp.data_ptr(), blk.data_ptr(), st.data_ptr(),
                                                      res.data_ptr(), cnt.data_ptr(), cnt.data_ptr() + 4, cap, stream)
    threads = [threading.Thread(target=call, args=(i,)) for i in range(len(inputs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert codes == [0] * len(inputs)
    for (m, cap, d_rp, blk, st, res, cnt), ref in zip(arrays, want):
        for a, b, name in zip((blk, st, res, cnt), ref, ("block_r_ind", "st_off", "residue_r_ind", "counts")):
            assert a.cpu().numpy().tobytes() == b.tobytes(), f"{name} differs (rows {m})"


def test_static_scratch_entry_point_in_a_hip_graph():
    """What the entry point is for: recorded into a HIP graph (its scratch is cleared by a fill
    kernel, so no memset node is recorded) and replayed on new row pointers of the same shape,
    with eager work and synchronisations between the replays; every replay against the
    workspace entry point."""
    from helpers import random_row_ptr
    from rode_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(13)
    m, seg = 300_000, 128
    variants = [random_row_ptr(rng, m, mean, long_rows=8, long_len=20_000) for mean in (6, 30, 11, 19)]
    cap = max((int(rp[-1]) + 3 * m) // seg + m for rp in variants)
    d_rp = torch.zeros(m + 1, dtype=torch.int32, device=dev)
    blk = torch.empty(cap + 1, dtype=torch.int32, device=dev)
    st = torch.empty(cap + 2, dtype=torch.int32, device=dev)
    res = torch.empty(m, dtype=torch.int32, device=dev)
    cnt = torch.empty(2, dtype=torch.int32, device=dev)

    def call(stream):
        code = lib.rode_hip_preprocess_static(seg, 32, 4, m, d_rp.data_ptr(), blk.data_ptr(), st.data_ptr(), res.data_ptr(),
                                              cnt.data_ptr(), cnt.data_ptr() + 4, cap, stream)
        assert code == 0, code

    d_rp.copy_(torch.from_numpy(variants[0]))
    call(torch.cuda.current_stream().cuda_stream)  # (the first call on a device looks the scratch up: outside the capture)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for replay, rp in enumerate(variants + variants[:1]):
        d_rp.copy_(torch.from_numpy(rp))
        for t in (blk, st, res, cnt):
            t.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want_blk, want_st, want_res, want_cnt = _run(lib, "workspace", rp, seg, dev)
        n_blk, n_res = (int(x) for x in cnt.cpu().numpy())
        assert (n_blk, n_res) == tuple(int(x) for x in want_cnt), f"replay {replay}: counts differ"
        assert blk[:n_blk].cpu().numpy().tobytes() == want_blk[:n_blk].tobytes(), f"replay {replay}: block_r_ind differs"
        assert st[: n_blk + 1].cpu().numpy().tobytes() == want_st[: n_blk + 1].tobytes(), f"replay {replay}: st_off differs"
        assert res[:n_res].cpu().numpy().tobytes() == want_res[:n_res].tobytes(), f"replay {replay}: residue_r_ind differs"
