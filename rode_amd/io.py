"""Matrix ingest for the RoDe path: Matrix Market files -> CSR arrays, and the row
padding the reference's generators apply.  (The reference's own loader,
``matrix_utils.h`` / ``SPC::SparseMatrix`` used at Preprocess_opt/_preprocess.cu:2,406-413,
is missing from its tree; this covers the same step: a SuiteSparse ``.mtx`` file in,
CSR with ascending columns out.)  Host side: a multi-threaded C++ parser
(``rode_amd/csrc/mtx.cpp``, in the host library next to the workload generators), with a
numpy implementation of the same rules for a tree where that library is not built.
"""
import ctypes
import gzip
import os

import numpy as np

from . import _lib

_native = None


def _load_native():
    global _native
    if _native is None:
        if not os.path.exists(_lib.WORKLOADS_PATH):
            _native = False
        else:
            lib = ctypes.CDLL(_lib.WORKLOADS_PATH)
            lib.rode_mtx_parse.restype = ctypes.c_void_p
            lib.rode_mtx_parse.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_int),
                                           ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_longlong),
                                           ctypes.c_char_p, ctypes.c_int]
            i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
            f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
            lib.rode_mtx_copy.argtypes = [ctypes.c_void_p, i32p, i32p, f32p]
            lib.rode_mtx_free.argtypes = [ctypes.c_void_p]
            _native = lib
    return _native


def read_matrix_market(path, native=None):
    """Read a ``coordinate`` Matrix Market file (real / integer / pattern; general,
    symmetric or skew-symmetric) and return ``(m, n, row_ptr, col, val)`` as int32 /
    float32 CSR with ascending columns per row.  Pattern files get value 1.0;
    duplicate entries are summed; the mirrored half of a symmetric file is added.
    ``native``: True / False picks the C++ or the numpy parser, None the C++ one when its
    library is built."""
    lib = _load_native() if native is not False else False
    if native is True and not lib:
        raise RuntimeError(f"{_lib.WORKLOADS_PATH} is missing: build it with `make -C rode_amd/csrc`")
    if lib:
        opener = gzip.open if str(path).endswith(".gz") else open
        with opener(path, "rb") as f:
            text = f.read()
        m, n, nnz = ctypes.c_int(), ctypes.c_int(), ctypes.c_longlong()
        err = ctypes.create_string_buffer(256)
        handle = lib.rode_mtx_parse(text, len(text), ctypes.byref(m), ctypes.byref(n), ctypes.byref(nnz), err, 256)
        if not handle:
            raise ValueError(f"{path}: {err.value.decode()}")
        try:
            row_ptr = np.empty(m.value + 1, dtype=np.int32)
            col = np.empty(nnz.value, dtype=np.int32)
            val = np.empty(nnz.value, dtype=np.float32)
            lib.rode_mtx_copy(handle, row_ptr, col, val)
        finally:
            lib.rode_mtx_free(handle)
        return m.value, n.value, row_ptr, col, val
    opener = gzip.open if str(path).endswith(".gz") else open
    with opener(path, "rt") as f:
        header = f.readline().strip().split()
        if len(header) < 5 or header[0] != "%%MatrixMarket" or header[1].lower() != "matrix":
            raise ValueError(f"{path}: not a Matrix Market matrix file")
        layout, field, symmetry = (h.lower() for h in header[2:5])
        if layout != "coordinate":
            raise ValueError(f"{path}: only the coordinate (sparse) layout is supported, got {layout}")
        if field not in ("real", "integer", "pattern", "double"):
            raise ValueError(f"{path}: unsupported field {field}")
        if symmetry not in ("general", "symmetric", "skew-symmetric"):
            raise ValueError(f"{path}: unsupported symmetry {symmetry}")
        line = f.readline()
        while line.startswith("%") or not line.strip():
            line = f.readline()
        m, n, entries = (int(t) for t in line.split()[:3])
        if symmetry != "general" and m != n:
            raise ValueError(f"{path}: a {symmetry} matrix must be square, got {m} x {n}")
        data = np.loadtxt(f, dtype=np.float64, ndmin=2, comments="%") if entries else np.zeros((0, 3))
    if data.shape[0] != entries:
        raise ValueError(f"{path}: header promises {entries} entries, file has {data.shape[0]}")
    rows = data[:, 0].astype(np.int64) - 1
    cols = data[:, 1].astype(np.int64) - 1
    vals = np.ones(entries) if field == "pattern" else data[:, 2]
    if entries and (rows.min() < 0 or rows.max() >= m or cols.min() < 0 or cols.max() >= n):
        raise ValueError(f"{path}: index out of range")
    if symmetry != "general":
        off = rows != cols
        sign = -1.0 if symmetry == "skew-symmetric" else 1.0
        rows, cols, vals = (np.concatenate([rows, cols[off]]), np.concatenate([cols, rows[off]]),
                            np.concatenate([vals, sign * vals[off]]))
    return coo_to_csr(m, n, rows, cols, vals)


def coo_to_csr(m, n, rows, cols, vals):
    """Coordinate triples -> ``(m, n, row_ptr, col, val)``; columns ascending in every
    row, duplicates summed."""
    rows, cols = np.asarray(rows, dtype=np.int64), np.asarray(cols, dtype=np.int64)
    vals = np.asarray(vals, dtype=np.float64)
    key = rows * n + cols
    order = np.argsort(key, kind="stable")
    key, vals = key[order], vals[order]
    if len(key):
        first = np.concatenate([[True], key[1:] != key[:-1]])
        starts = np.nonzero(first)[0]
        vals = np.add.reduceat(vals, starts)
        key = key[starts]
    if len(key) >= 2**31:
        raise ValueError("more than 2^31-1 nonzeros")
    row_ptr = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(np.bincount(key // n, minlength=m), out=row_ptr[1:])
    return m, n, row_ptr.astype(np.int32), (key % n).astype(np.int32), vals.astype(np.float32)


def pad_rows(row_ptr, col, val, multiple=4):
    """Pad every row to a multiple of ``multiple`` entries with (last column of the row,
    0.0), as the reference's generators do (RoDe_SDDMM/main.cu:217-228, test.cu:153-163),
    so that every row starts on a 128-bit boundary.  Empty rows stay empty.  Padding is
    optional for this library (rows may start anywhere); it only reproduces the
    reference's input convention."""
    row_ptr = np.asarray(row_ptr, dtype=np.int64)
    lens = np.diff(row_ptr)
    padded = (lens + multiple - 1) // multiple * multiple
    new_ptr = np.zeros(len(row_ptr), dtype=np.int64)
    np.cumsum(padded, out=new_ptr[1:])
    new_col = np.zeros(int(new_ptr[-1]), dtype=np.int32)
    new_val = np.zeros(int(new_ptr[-1]), dtype=np.float32)
    src = np.arange(int(row_ptr[-1]), dtype=np.int64)
    row_of = np.repeat(np.arange(len(lens)), lens)
    dst = src - row_ptr[row_of] + new_ptr[row_of]
    new_col[dst] = col
    new_val[dst] = val
    # pads repeat the row's last real column
    pad_rows_idx = np.repeat(np.arange(len(lens)), padded - lens)
    if len(pad_rows_idx):
        within = np.arange(len(pad_rows_idx)) - np.repeat(np.cumsum(padded - lens) - (padded - lens), padded - lens)
        pad_dst = new_ptr[pad_rows_idx] + lens[pad_rows_idx] + within
        new_col[pad_dst] = np.asarray(col)[row_ptr[pad_rows_idx] + lens[pad_rows_idx] - 1]
    return new_ptr.astype(np.int32), new_col, new_val
