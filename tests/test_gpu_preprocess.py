"""GPU row decomposition == CPU oracle, byte for byte (integer work: bit-exact)."""
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

PARAM_SETS = [(512, 32, 4), (32, 32, 4), (256, 32, 4), (128, 32, 4), (2048, 32, 4)]
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "preprocess_handworked.json")


def test_handworked_vectors_on_gpu():
    from gpu_common import gpu_preprocess
    for c in json.load(open(GOLDEN))["cases"]:
        seg, kb, vl = c["params"]
        blk, st, res = gpu_preprocess(np.array(c["row_ptr"], np.int32), seg, kb, vl)
        assert res.tolist() == c["residue_r_ind"], c["name"]
        if "block_r_ind" in c:
            assert blk.tolist() == c["block_r_ind"] and st.tolist() == c["st_off"], c["name"]
        else:
            k = len(c["st_off_prefix"])
            assert len(blk) == c["n_blk"] and st[:k].tolist() == c["st_off_prefix"] and st[-1] == c["st_off_last"]


@pytest.mark.parametrize("params", PARAM_SETS)
def test_random_row_pointers(params):
    from gpu_common import assert_preprocess_bit_exact
    from helpers import random_row_ptr
    seg, kb, vl = params
    rng = np.random.default_rng(seg)
    for m, mean, nlong, llen in [(1, 5, 0, 0), (1, 0, 1, 100000), (7, 40, 2, 3000), (1023, 3, 5, 900),
                                 (1024, 20, 0, 0), (1025, 33, 9, 70000), (5000, 200, 0, 0),
                                 (300000, 6, 40, 50000)]:
        rp = random_row_ptr(rng, m, mean, long_rows=nlong, long_len=max(llen, 2))
        assert_preprocess_bit_exact(rp, seg, kb, vl)
        # same lengths starting at an unaligned offset
        assert_preprocess_bit_exact(rp + 3, seg, kb, vl)


def test_edge_cases():
    from gpu_common import assert_preprocess_bit_exact
    for seg in (512, 32):
        assert assert_preprocess_bit_exact(np.zeros(1, np.int32), seg) == (0, 0)            # no rows
        assert assert_preprocess_bit_exact(np.zeros(4097, np.int32), seg) == (0, 0)         # all rows empty
        assert assert_preprocess_bit_exact(np.arange(1001, dtype=np.int32) * 27, seg) == (0, 1000)
        assert assert_preprocess_bit_exact(np.arange(1001, dtype=np.int32) * 32, seg) == (1000, 0)
        assert_preprocess_bit_exact(np.array([0, 200000], np.int32), seg)                    # one huge row
        assert_preprocess_bit_exact(np.array([0, 2**31 - 8], np.int32), 2**20)               # largest offsets
    # k_block / vec_len other than the kernels' (the routine itself is generic)
    rng = np.random.default_rng(3)
    rp = np.concatenate([[0], rng.integers(0, 300, 5000)]).cumsum().astype(np.int32)
    for params in [(48, 16, 2), (100, 10, 1), (64, 64, 8), (96, 32, 4)]:
        assert_preprocess_bit_exact(rp, *params)


@pytest.mark.parametrize("name", ["c1_uniform", "c2_lognormal", "c3_banded", "c4_powerlaw", "c5_attention"])
def test_benchmark_configs_full_size(name):
    from gpu_common import assert_preprocess_bit_exact
    from rode_amd import workloads
    kind, rows, cols, p0, p1, _ = workloads.CONFIGS[name]
    # lengths only: the decomposition depends on row_ptr alone
    lens = np.empty(rows, np.int32)
    workloads._load().rode_wl_row_lengths(kind, rows, cols, p0, p1, workloads.SEEDS[name], lens)
    rp = np.concatenate([[0], np.cumsum(lens, dtype=np.int64)]).astype(np.int32)
    for seg in (512, 32, 256):
        nb, nr = assert_preprocess_bit_exact(rp, seg)
        if name == "c3_banded":
            assert (nb, nr) == (0, rows)
    print(name, "nnz", rp[-1])


def test_reference_module_surface():
    from rode_amd import rode_sddmm_hip
    rp = torch.tensor([0, 3, 40, 40, 600, 1700], dtype=torch.int32)
    blk, st, res, nb, nr = rode_sddmm_hip.preprocess(rp, 1700, 512, 32, 4)
    assert (nb, nr) == (6, 4) and blk.device.type == "cpu" and st.tolist() == [3, 40, 552, 600, 1112, 1624, 1700]
    blk, st, res, nb, nr = rode_sddmm_hip.preprocess(torch.zeros(5, dtype=torch.int32), 0, 512, 32, 4)
    assert (nb, nr) == (0, 0) and blk.numel() == 1 and st.tolist() == [0] and res.numel() == 1
    with pytest.raises(RuntimeError, match="must be on CPU"):
        rode_sddmm_hip.preprocess(rp.cuda(), 1700, 512, 32, 4)
    with pytest.raises(RuntimeError, match="int32"):
        rode_sddmm_hip.preprocess(rp.long(), 1700, 512, 32, 4)


@pytest.mark.parametrize("rows,longest", [(20000, 900), (4_500_000, 70)], ids=["fixed_scratch", "beyond_the_fixed_scratch"])
def test_cxx_reference_signature_entry_point(rows, longest):
    """RoDe_preprocess(N_SEG, blockX, vecLen, M, ...) with the reference's GPU
    signature (Preprocess_opt/_preprocess.cu:323), called through its mangled name: a matrix
    that the library's fixed scratch holds, and one with more rows than that (4 194 304), for
    which the call brings scratch of its own (550 tiles of 8192 rows in the scan)."""
    import ctypes
    import oracle
    from rode_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    fn = getattr(lib, "_Z15RoDe_preprocessiiiiPKiPiS1_S1_S1_S1_")
    fn.restype = None
    fn.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p] * 6
    rng = np.random.default_rng(5)
    rp = np.concatenate([[0], rng.integers(0, longest, rows)]).cumsum().astype(np.int32)
    d_rp = torch.from_numpy(rp).cuda()
    cap = int(rp[-1]) // 512 + len(rp) + 8
    blk = torch.empty(cap, dtype=torch.int32, device="cuda")
    st = torch.empty(cap + 1, dtype=torch.int32, device="cuda")
    res = torch.empty(len(rp), dtype=torch.int32, device="cuda")
    cnt = torch.zeros(2, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    fn(512, 32, 4, len(rp) - 1, d_rp.data_ptr(), blk.data_ptr(), st.data_ptr(), res.data_ptr(),
       cnt.data_ptr(), cnt.data_ptr() + 4)
    torch.cuda.synchronize()
    oblk, ost, ores = oracle.preprocess(rp, 512)
    nb, nr = cnt.tolist()
    assert (nb, nr) == (len(oblk), len(ores))
    assert blk[:nb].cpu().numpy().tobytes() == oblk.tobytes()
    assert st[: nb + 1].cpu().numpy().tobytes() == ost.tobytes()
    assert res[:nr].cpu().numpy().tobytes() == ores.tobytes()


def test_capacity_too_small_is_detected_not_overrun():
    """With room for fewer segments than the matrix has, nothing is written past the
    capacity and the true count comes back."""
    import oracle
    from rode_amd import _lib
    lib = _lib.load()
    rp = (np.arange(1001, dtype=np.int32) * 64)  # 1000 rows of 64 -> 2000 segments at seg 32
    d_rp = torch.from_numpy(rp).cuda()
    cap = 700
    blk = torch.full((cap + 8,), -7, dtype=torch.int32, device="cuda")
    st = torch.full((cap + 9,), -7, dtype=torch.int32, device="cuda")
    res = torch.empty(1000, dtype=torch.int32, device="cuda")
    cnt = torch.zeros(2, dtype=torch.int32, device="cuda")
    nbytes = lib.rode_hip_preprocess_workspace_bytes(1000)
    ws = torch.empty((nbytes + 7) // 8, dtype=torch.int64, device="cuda")
    code = lib.rode_hip_preprocess(32, 32, 4, 1000, d_rp.data_ptr(), blk.data_ptr(), st.data_ptr(), res.data_ptr(),
                                   cnt.data_ptr(), cnt.data_ptr() + 4, cap, ws.data_ptr(), nbytes, None)
    assert code == 0
    torch.cuda.synchronize()
    oblk, ost, _ = oracle.preprocess(rp, 32)
    assert cnt.tolist() == [2000, 0]
    assert blk[:cap].cpu().numpy().tobytes() == oblk[:cap].tobytes() and (blk[cap:] == -7).all()
    assert st[:cap].cpu().numpy().tobytes() == ost[:cap].tobytes() and (st[cap:] == -7).all()
    # bad arguments are rejected before any launch
    assert lib.rode_hip_preprocess(0, 32, 4, 1000, d_rp.data_ptr(), blk.data_ptr(), st.data_ptr(), res.data_ptr(),
                                   cnt.data_ptr(), cnt.data_ptr() + 4, cap, ws.data_ptr(), nbytes, None) != 0
    assert lib.rode_hip_preprocess(32, 32, 4, 1000, d_rp.data_ptr(), blk.data_ptr(), st.data_ptr(), res.data_ptr(),
                                   cnt.data_ptr(), cnt.data_ptr() + 4, cap, ws.data_ptr(), 16, None) != 0


def test_host_pointer_twins():
    """RoDe_preprocess_cpu (Preprocess_opt/_preprocess.cu:340 order: seg, k_block, vec_len) and
    the host overload of RoDe_preprocess (main.cu:114-123 order: seg, vec_len, k_block), called
    through their mangled names with host arrays and int& counts, and the C-ABI function
    beneath them."""
    import ctypes
    import oracle
    from rode_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    rng = np.random.default_rng(8)
    rp = (np.concatenate([[0], rng.integers(0, 700, 30000)]).cumsum() + 1).astype(np.int32)
    m = len(rp) - 1
    for name, order in (("_Z19RoDe_preprocess_cpuiiiiPKiPiS1_S1_RiS2_", "seg_kb_vl"),
                        ("_Z15RoDe_preprocessiiiiPKiPiS1_S1_RiS2_", "seg_vl_kb"), ("rode_hip_preprocess_host", "c")):
        for seg in (512, 32):
            oblk, ost, ores = oracle.preprocess(rp, seg)
            cap = (int(rp[-1]) + 3 * m) // seg + m + 1
            blk, st, res = np.full(cap, -1, np.int32), np.full(cap + 1, -1, np.int32), np.full(m, -1, np.int32)
            nb, nr = ctypes.c_int(-1), ctypes.c_int(-1)
            fn = getattr(lib, name)
            fn.restype = ctypes.c_int if order == "c" else None
            fn.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p] * 6
            a, b = (32, 4) if order != "seg_vl_kb" else (4, 32)
            ret = fn(seg, a, b, m, rp.ctypes.data, blk.ctypes.data, st.ctypes.data, res.ctypes.data,
                     ctypes.addressof(nb), ctypes.addressof(nr))
            assert order != "c" or ret == 0
            assert (nb.value, nr.value) == (len(oblk), len(ores)), name
            assert blk[:nb.value].tobytes() == oblk.tobytes() and (blk[nb.value:] == -1).all()
            assert st[:nb.value + 1].tobytes() == ost.tobytes() and (st[nb.value + 1:] == -1).all()
            assert res[:nr.value].tobytes() == ores.tobytes() and (res[nr.value:] == -1).all()
    # empty matrix, bad arguments
    z = np.zeros(1, np.int32)
    one = np.full(2, -1, np.int32)
    nb, nr = ctypes.c_int(-1), ctypes.c_int(-1)
    host = lib.rode_hip_preprocess_host
    host.restype, host.argtypes = ctypes.c_int, [ctypes.c_int] * 4 + [ctypes.c_void_p] * 6
    assert host(512, 32, 4, 0, z.ctypes.data, one.ctypes.data, one.ctypes.data, one.ctypes.data,
                ctypes.addressof(nb), ctypes.addressof(nr)) == 0
    assert (nb.value, nr.value) == (0, 0) and one[0] == 0
    assert host(0, 32, 4, 0, z.ctypes.data, one.ctypes.data, one.ctypes.data, one.ctypes.data,
                ctypes.addressof(nb), ctypes.addressof(nr)) != 0
