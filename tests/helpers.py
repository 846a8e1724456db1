"""Shared pieces of the test-suite: independent numpy restatements used to pin
the oracle, error metrics, and input builders."""
import numpy as np


# ---- independent statement of the decomposition (closed form, vectorised) ----
def closed_form_preprocess(row_ptr, seg, kblock=32, veclen=4):
    """Per-row closed form of Preprocess_opt/_preprocess.cu:262-270 (valid when
    seg % kblock == 0) + exclusive prefix sums + the start-offset closed form
    (segment j of a row starts at s if j == 0, else (s - s % veclen) + j * seg)."""
    assert seg % kblock == 0
    rp = np.asarray(row_ptr, dtype=np.int64)
    s, e = rp[:-1], rp[1:]
    pad = s % veclen
    N = e - s + pad
    long_row = N > seg
    rest = np.where(long_row, N % seg, N)
    bn = np.where(long_row, N // seg, 0) + (rest >= kblock)
    rn = (rest % kblock != 0) & (N > 0)
    bn = np.where(N > 0, bn, 0)
    rows = np.repeat(np.arange(len(s)), bn)
    first = np.cumsum(bn) - bn
    j = np.arange(bn.sum()) - np.repeat(first, bn)
    st = np.where(j == 0, s[rows], (s[rows] - pad[rows]) + j * seg)
    st = np.concatenate([st, rp[-1:]])
    return rows.astype(np.int32), st.astype(np.int32), np.nonzero(rn)[0].astype(np.int32)


def coverage_counts(row_ptr, blk, st, res, kblock=32, veclen=4):
    """How often every nonzero index is processed by the block kernels' ranges
    (RoDeSpmm.cu:210-234) and the residue kernels' ranges (RoDeSpmm.cu:71-82),
    and the row each range attributes it to."""
    rp = np.asarray(row_ptr, dtype=np.int64)
    nnz = int(rp[-1])
    hits = np.zeros(nnz, dtype=np.int32)
    owner = np.full(nnz, -1, dtype=np.int64)
    for i, r in enumerate(blk):
        start = int(st[i])
        end = min(int(rp[r + 1]), int(st[i + 1]))
        mask = start % veclen
        base = start - mask
        cnt = (end - start + mask) // kblock * kblock
        hits[base + mask: base + cnt] += 1
        owner[base + mask: base + cnt] = r
    for r in res:
        s, e = int(rp[r]), int(rp[r + 1])
        pad = s % veclen
        N = e - s + pad
        if N >= kblock:
            first, cnt = (s - pad) + N // kblock * kblock, N % kblock
        else:
            first, cnt = s, e - s
        hits[first: first + cnt] += 1
        owner[first: first + cnt] = r
    return hits, owner


def merged_block_ranges(row_ptr, blk, st, merge_slots, kblock=32, veclen=4):
    """Host model of what the merging block kernels touch (sddmm_block_kernel with
    merge_slots = 128; spmm_block_kernel under the whole-lists promise with 512, for rows
    it does not sum whole): consecutive segments of a row whose starts fall into one window
    of merge_slots slots are handled by the first of them.  Returns one tuple per leader:
    (row, first index read, first index written, end) -- the kernel reads col/val in
    [first read, end) and writes out in [first written, end)."""
    rp = np.asarray(row_ptr, dtype=np.int64)
    out = []
    n = len(blk)
    i = 0
    while i < n:
        r = int(blk[i])
        row_base = int(rp[r]) - int(rp[r]) % veclen
        window = (int(st[i]) - row_base) // merge_slots
        j = i + 1
        while j < n and int(blk[j]) == r and (int(st[j]) - row_base) // merge_slots == window:
            j += 1
        block_end = row_base + (int(rp[r + 1]) - row_base) // kblock * kblock
        end = min(block_end, int(st[j]))
        start = int(st[i])
        base = start - start % veclen
        if end > base:
            out.append((r, base, start, end))
        i = j
    return out


def residue_ranges(row_ptr, res, kblock=32, veclen=4):
    """(row, first, end) of the slots each residue work item owns (RoDeSpmm.cu:71-82)."""
    rp = np.asarray(row_ptr, dtype=np.int64)
    out = []
    for r in res:
        s, e = int(rp[r]), int(rp[r + 1])
        pad = s % veclen
        N = e - s + pad
        first = (s - pad) + N // kblock * kblock if N >= kblock else s
        if e > first:
            out.append((int(r), first, e))
    return out


def row_of_index(row_ptr):
    rp = np.asarray(row_ptr, dtype=np.int64)
    return np.repeat(np.arange(len(rp) - 1), np.diff(rp))


# ---- numeric references in fp64 (numpy only) ---------------------------------
def sddmm_numpy64(row_ptr, col, val, lhs, rhs):
    rows = row_of_index(row_ptr)
    out = np.empty(len(col), dtype=np.float64)
    step = 1 << 18
    lhs64, rhs64 = lhs.astype(np.float64), rhs.astype(np.float64)
    for a in range(0, len(col), step):
        b = min(len(col), a + step)
        out[a:b] = np.einsum("ik,ik->i", lhs64[rows[a:b]], rhs64[col[a:b]])
    return out * val.astype(np.float64)


def spmm_scipy64(row_ptr, col, val, B, m, k):
    import scipy.sparse as sp
    A = sp.csr_matrix((val.astype(np.float64), col, row_ptr), shape=(m, k))
    return A @ B.astype(np.float64)


# ---- error metrics --------------------------------------------------------------
def sddmm_row_l1_error(got, ref64, row_ptr):
    """max over rows of  max|got-ref| / sum|ref|  over the row's output slice."""
    rp = np.asarray(row_ptr, dtype=np.int64)
    if len(got) == 0:
        return 0.0
    nonempty = np.nonzero(np.diff(rp) > 0)[0]
    err = np.abs(got.astype(np.float64) - ref64)
    emax = np.maximum.reduceat(err, rp[nonempty])
    l1 = np.add.reduceat(np.abs(ref64), rp[nonempty])
    return float(np.max(emax / np.maximum(l1, 1e-30)))


def sddmm_row_l1_errors(got, ref64, scale, row_ptr):
    """Per non-empty row: (max|got-ref| / sum|ref|, condition number sum(scale) / sum|ref|),
    where scale[idx] = |val| * sum_k |lhs*rhs| is the magnitude of the summed terms."""
    rp = np.asarray(row_ptr, dtype=np.int64)
    nonempty = np.nonzero(np.diff(rp) > 0)[0]
    if len(nonempty) == 0:
        return np.zeros(0), np.zeros(0)
    err = np.abs(got.astype(np.float64) - ref64)
    emax = np.maximum.reduceat(err, rp[nonempty])
    l1 = np.maximum(np.add.reduceat(np.abs(ref64), rp[nonempty]), 1e-300)
    cond = np.add.reduceat(scale, rp[nonempty]) / l1
    return emax / l1, cond


def spmm_row_l1_error(got, ref64):
    """max over rows of  max_j|got-ref| / sum_j|ref|."""
    err = np.abs(got.astype(np.float64) - ref64).max(axis=1)
    l1 = np.abs(ref64).sum(axis=1)
    ok = l1 > 0
    worst_zero = float(err[~ok].max()) if (~ok).any() else 0.0
    assert worst_zero == 0.0, "non-zero output in a row whose reference is all zero"
    return float((err[ok] / l1[ok]).max()) if ok.any() else 0.0


def reference_error_count(got, ref, tol=1e-3, eps=1e-6):
    """The reference tests' rule (test.cu:221-237): an element is wrong iff both
    its absolute and its relative difference exceed tol."""
    diff = np.abs(got.astype(np.float32) - ref.astype(np.float32))
    rel = diff / (np.abs(ref.astype(np.float32)) + np.float32(eps))
    return int(((diff > tol) & (rel > tol)).sum())


# ---- inputs -----------------------------------------------------------------------
def random_row_ptr(rng, m, mean_len, long_rows=0, long_len=2000, empty_frac=0.1):
    lens = rng.poisson(mean_len, size=m)
    lens[rng.random(m) < empty_frac] = 0
    if long_rows:
        idx = rng.choice(m, size=min(long_rows, m), replace=False)
        lens[idx] = rng.integers(long_len // 2, long_len + 1, size=len(idx))
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum(lens)
    return rp


def random_csr(rng, m, n, mean_len, **kw):
    rp = random_row_ptr(rng, m, min(mean_len, n), **{k: v for k, v in kw.items()})
    lens = np.minimum(np.diff(rp), n)
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum(lens)
    col = np.empty(rp[-1], dtype=np.int32)
    for r in range(m):
        col[rp[r]:rp[r + 1]] = np.sort(rng.choice(n, size=lens[r], replace=False))
    val = rng.uniform(-1, 1, size=rp[-1]).astype(np.float32)
    return rp, col, val
