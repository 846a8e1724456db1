"""ctypes front-end of ``liboracle.so`` (see ``rode_oracle.c`` for what each
function restates and what pins it).  Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")
_lib = None

_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile ``liboracle.so`` with gcc (a second or two)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
        os.path.join(_HERE, "rode_oracle.c")
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def _load():
    global _lib
    if _lib is not None:
        return _lib
    build()
    lib = ctypes.CDLL(_SO)
    c_int = ctypes.c_int
    lib.oracle_num_threads.restype = c_int
    lib.oracle_preprocess.argtypes = [c_int, c_int, c_int, c_int, _i32p, _i32p, _i32p, _i32p,
                                      ctypes.POINTER(c_int), ctypes.POINTER(c_int)]
    for name in ("oracle_sddmm_f32", "oracle_sddmm_f32_mt"):
        getattr(lib, name).argtypes = [c_int, c_int, _i32p, _i32p, _f32p, _f32p, _f32p, _f32p]
    lib.oracle_sddmm_f64.argtypes = [c_int, c_int, _i32p, _i32p, _f32p, _f32p, _f32p, _f64p, ctypes.c_void_p]
    for name in ("oracle_spmm_f32", "oracle_spmm_f32_mt"):
        getattr(lib, name).argtypes = [c_int, c_int, _i32p, _i32p, _f32p, _f32p, _f32p]
    lib.oracle_spmm_f64.argtypes = [c_int, c_int, _i32p, _i32p, _f32p, _f32p, _f64p, ctypes.c_void_p]
    lib.oracle_spmm_d.argtypes = [c_int, c_int, _i32p, _i32p, _f64p, _f64p, _f64p]
    _lib = lib
    return lib


def num_threads():
    return int(_load().oracle_num_threads())


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def preprocess(row_ptr, seg_length, k_block=32, vec_len=4):
    """Row decomposition -> (block_r_ind[n_blk], st_off[n_blk+1], residue_r_ind[n_res])."""
    row_ptr = _i32(row_ptr)
    M = row_ptr.size - 1
    nnz = int(row_ptr[-1]) if M >= 0 else 0
    # n_blk <= sum_i ceil((len_i + vec_len - 1) / seg) <= (nnz + (vec_len-1)*M)/seg + M
    cap = (nnz + (vec_len - 1) * max(M, 0)) // seg_length + max(M, 0) + 1
    blk = np.empty(cap, dtype=np.int32)
    st = np.empty(cap + 1, dtype=np.int32)
    res = np.empty(max(M, 1), dtype=np.int32)
    nb, nr = ctypes.c_int(0), ctypes.c_int(0)
    _load().oracle_preprocess(seg_length, k_block, vec_len, M, row_ptr, blk, st, res,
                              ctypes.byref(nb), ctypes.byref(nr))
    return blk[: nb.value].copy(), st[: nb.value + 1].copy(), res[: nr.value].copy()


def sddmm_f32(row_ptr, col, val, lhs, rhs, threads=1):
    """Reference-faithful fp32 SDDMM (main.cu:65-91)."""
    row_ptr, col, val, lhs, rhs = _i32(row_ptr), _i32(col), _f32(val), _f32(lhs), _f32(rhs)
    out = np.zeros(val.size, dtype=np.float32)
    fn = _load().oracle_sddmm_f32 if threads == 1 else _load().oracle_sddmm_f32_mt
    fn(row_ptr.size - 1, lhs.shape[1], row_ptr, col, val, lhs, rhs, out)
    return out


def sddmm_f64(row_ptr, col, val, lhs, rhs, with_abs=False):
    row_ptr, col, val, lhs, rhs = _i32(row_ptr), _i32(col), _f32(val), _f32(lhs), _f32(rhs)
    out = np.zeros(val.size, dtype=np.float64)
    ab = np.zeros(val.size, dtype=np.float64) if with_abs else None
    _load().oracle_sddmm_f64(row_ptr.size - 1, lhs.shape[1], row_ptr, col, val, lhs, rhs, out,
                             ab.ctypes.data if with_abs else None)
    return (out, ab) if with_abs else out


def spmm_f32(row_ptr, col, val, B, threads=1):
    """Textbook CSR SpMM in fp32 (the reference has no CPU SpMM)."""
    row_ptr, col, val, B = _i32(row_ptr), _i32(col), _f32(val), _f32(B)
    m, n = row_ptr.size - 1, B.shape[1]
    C = np.zeros((m, n), dtype=np.float32)
    fn = _load().oracle_spmm_f32 if threads == 1 else _load().oracle_spmm_f32_mt
    fn(m, n, row_ptr, col, val, B, C)
    return C


def spmm_f64(row_ptr, col, val, B, with_abs=False):
    row_ptr, col, val, B = _i32(row_ptr), _i32(col), _f32(val), _f32(B)
    m, n = row_ptr.size - 1, B.shape[1]
    C = np.zeros((m, n), dtype=np.float64)
    ab = np.zeros((m, n), dtype=np.float64) if with_abs else None
    _load().oracle_spmm_f64(m, n, row_ptr, col, val, B, C, ab.ctypes.data if with_abs else None)
    return (C, ab) if with_abs else C


def spmm_d(row_ptr, col, val, B):
    """SpMM with fp64 values and operands (the reference's double overloads)."""
    row_ptr, col = _i32(row_ptr), _i32(col)
    val, B = np.ascontiguousarray(val, dtype=np.float64), np.ascontiguousarray(B, dtype=np.float64)
    m, n = row_ptr.size - 1, B.shape[1]
    C = np.zeros((m, n), dtype=np.float64)
    _load().oracle_spmm_d(m, n, row_ptr, col, val, B, C)
    return C
