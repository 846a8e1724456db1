"""Helpers of the GPU parity tests: move numpy CSR data to the device, run the
product through its Python/C-ABI path, bring results back."""
import numpy as np
import torch

import oracle
from rode_amd import RoDeCSR, rode_sddmm, rode_spmm
from rode_amd import rode_sddmm_hip

DEV = torch.device("cuda:0")

# north-star tolerances: max over rows of |err|_inf / |ref row|_1
TOL_F32 = 1e-4
TOL_F16 = 2e-3


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


def make_csr(row_ptr, col, val, m, n, k, seg=None, locality="auto"):
    cfg = None if seg is None else {"seg_length": seg, "k_block": 32, "vec_len": 4}
    return RoDeCSR(t(row_ptr), t(col), t(val), DEV, m, n, k, config=cfg, locality=locality)


def gpu_preprocess(row_ptr, seg, kb=32, vl=4):
    rp = t(np.asarray(row_ptr, dtype=np.int32)).to(DEV)
    blk, st, res, nb, nr = rode_sddmm_hip.preprocess_device(rp, int(row_ptr[-1]), seg, kb, vl)
    return blk.cpu().numpy()[:nb], st.cpu().numpy(), res.cpu().numpy()[:nr]


def assert_preprocess_bit_exact(row_ptr, seg, kb=32, vl=4):
    blk, st, res = gpu_preprocess(row_ptr, seg, kb, vl)
    oblk, ost, ores = oracle.preprocess(row_ptr, seg, kb, vl)
    assert blk.dtype == np.int32 and st.dtype == np.int32 and res.dtype == np.int32
    assert blk.tobytes() == oblk.tobytes(), "block_r_ind differs"
    assert st.tobytes() == ost.tobytes(), "st_off differs"
    assert res.tobytes() == ores.tobytes(), "residue_r_ind differs"
    return len(blk), len(res)


def check_csr_decomposition(csr, row_ptr):
    oblk, ost, ores = oracle.preprocess(row_ptr, csr.config["seg_length"], csr.config["k_block"], csr.config["vec_len"])
    assert csr.m1 == len(oblk) and csr.m2 == len(ores)
    assert csr.block_indices.cpu().numpy()[: csr.m1].tobytes() == oblk.tobytes()
    assert csr.st_offsets.cpu().numpy().tobytes() == ost.tobytes()
    assert csr.residue_indices.cpu().numpy()[: csr.m2].tobytes() == ores.tobytes()


def run_sddmm(csr, lhs, rhs, half=False):
    dt = torch.float16 if half else torch.float32
    return rode_sddmm(csr, t(lhs).to(DEV, dt), t(rhs).to(DEV, dt)).cpu().numpy()


def run_spmm(csr, B, half=False):
    dt = torch.float16 if half else torch.float32
    return rode_spmm(csr, t(B).to(DEV, dt)).cpu().numpy()


def round_half(a):
    return a.astype(np.float16).astype(np.float32)
