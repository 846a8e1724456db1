"""Seeded synthetic CSR workloads (numpy arrays, host side): the five benchmark
configurations and the generators of the reference's C++ tests.  Backed by
``librode_workloads.so`` (``csrc/workloads.cpp``)."""
import ctypes
import os

import numpy as np

from . import _lib

_wl = None
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")

# name -> (generator id, rows, cols, p0, p1, description)
CONFIGS = {
    "c1_uniform": (1, 4096, 4096, 0.01, 0.0, "4096x4096, every entry kept with p=0.01, values U(-1,1)"),
    "c2_lognormal": (2, 65536, 65536, 16.0, 1.5, "65536x65536, row length lognormal(mean 16, sigma 1.5) capped 20000"),
    "c3_banded": (3, 1_000_000, 1_000_000, 27.0, 256.0, "1Mx1M, 27 nonzeros per row inside a band of width 256"),
    "c4_powerlaw": (4, 2_000_000, 2_000_000, 2.1, 6.0,
                    "2Mx2M, degree 6*(Zipf(2.1)-1)+U{1..6} in [1,200000], values 1/degree"),
    "c5_attention": (5, 16384, 16384, 512.0, 64.0, "16384x16384, sliding window 512 + 64 random columns, values 1"),
}
SEEDS = {"c1_uniform": 1001, "c2_lognormal": 1002, "c3_banded": 1003, "c4_powerlaw": 1004, "c5_attention": 1005}


def _load():
    global _wl
    if _wl is None:
        if not os.path.exists(_lib.WORKLOADS_PATH):
            raise RuntimeError(f"{_lib.WORKLOADS_PATH} is missing: build it with `make -C rode_amd/csrc`")
        wl = ctypes.CDLL(_lib.WORKLOADS_PATH)
        c_int, c_dbl, c_u64 = ctypes.c_int, ctypes.c_double, ctypes.c_uint64
        wl.rode_wl_row_lengths.argtypes = [c_int, c_int, c_int, c_dbl, c_dbl, c_u64, _i32p]
        wl.rode_wl_fill.argtypes = [c_int, c_int, c_int, c_dbl, c_dbl, c_u64, _i32p, _i32p, _f32p]
        wl.rode_wl_ref_csr_create.restype = ctypes.c_void_p
        wl.rode_wl_ref_csr_create.argtypes = [c_int, c_int, c_int, c_int, c_int, ctypes.c_uint]
        wl.rode_wl_ref_csr_nnz.argtypes = [ctypes.c_void_p]
        wl.rode_wl_ref_csr_copy.argtypes = [ctypes.c_void_p, _i32p, _i32p, _f32p]
        wl.rode_wl_ref_csr_free.argtypes = [ctypes.c_void_p]
        wl.rode_wl_ref_dense.argtypes = [ctypes.c_longlong, ctypes.c_uint, _f32p]
        _wl = wl
    return _wl


def generate(kind, rows, cols, p0, p1, seed):
    """CSR (row_ptr int32[rows+1], col int32[nnz], val float32[nnz]) of generator
    ``kind`` (1 uniform, 2 lognormal, 3 banded, 4 power law, 5 attention mask)."""
    wl = _load()
    lens = np.empty(rows, dtype=np.int32)
    wl.rode_wl_row_lengths(kind, rows, cols, p0, p1, seed, lens)
    row_ptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(lens, out=row_ptr[1:])
    if row_ptr[-1] >= 2**31:
        raise ValueError("more than 2^31-1 nonzeros")
    row_ptr = row_ptr.astype(np.int32)
    col = np.empty(int(row_ptr[-1]), dtype=np.int32)
    val = np.empty(int(row_ptr[-1]), dtype=np.float32)
    wl.rode_wl_fill(kind, rows, cols, p0, p1, seed, row_ptr, col, val)
    return row_ptr, col, val


def config(name, scale=1.0, seed=None):
    """One of ``CONFIGS`` by name; ``scale`` < 1 shrinks rows and columns for tests."""
    kind, rows, cols, p0, p1, _ = CONFIGS[name]
    rows, cols = max(1, int(rows * scale)), max(1, int(cols * scale))
    row_ptr, col, val = generate(kind, rows, cols, p0, p1, SEEDS[name] if seed is None else seed)
    return rows, cols, row_ptr, col, val


def reference_csr(m, n, nnz_per_row, poisson=False, pad_to=4, seed=42):
    """The matrix of the reference's C++ tests: ``generate_random_csr`` of
    RoDe_SDDMM/main.cu:181-234 (``poisson=False``) or test.cu:121-169
    (``poisson=True``), rows padded to a multiple of ``pad_to`` with explicit zeros."""
    wl = _load()
    h = wl.rode_wl_ref_csr_create(m, n, nnz_per_row, int(poisson), pad_to, seed)
    try:
        nnz = wl.rode_wl_ref_csr_nnz(h)
        row_ptr = np.empty(m + 1, dtype=np.int32)
        col = np.empty(nnz, dtype=np.int32)
        val = np.empty(nnz, dtype=np.float32)
        wl.rode_wl_ref_csr_copy(h, row_ptr, col, val)
    finally:
        wl.rode_wl_ref_csr_free(h)
    return row_ptr, col, val


def reference_dense(rows, cols, seed):
    """``generate_random_dense`` of RoDe_SDDMM/main.cu:239-251: U(-1,1), mt19937(seed)."""
    out = np.empty((rows, cols), dtype=np.float32)
    _load().rode_wl_ref_dense(rows * cols, seed, out.reshape(-1))
    return out
