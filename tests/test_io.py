"""Matrix Market ingest and row padding (host side, no GPU)."""
import gzip

import numpy as np
import pytest
import scipy.io
import scipy.sparse as sp

from rode_amd import io as rio


def _same(csr, ref):
    m, n, rp, col, val = csr
    ref = sp.csr_matrix(ref)
    ref.sum_duplicates()
    ref.sort_indices()
    assert (m, n) == ref.shape
    np.testing.assert_array_equal(rp, ref.indptr)
    np.testing.assert_array_equal(col, ref.indices)
    np.testing.assert_allclose(val, ref.data.astype(np.float32), rtol=1e-6)


@pytest.fixture(params=[True, False], ids=["cxx", "numpy"], autouse=True)
def parser(request, monkeypatch):
    """Every test of the reader runs with the C++ parser and with the numpy one."""
    read = rio.read_matrix_market
    monkeypatch.setattr(rio, "read_matrix_market", lambda path, native=None: read(path, native=request.param))
    return request.param


@pytest.mark.parametrize("symmetry", ["general", "symmetric", "skew-symmetric"])
def test_reads_what_scipy_reads(tmp_path, symmetry):
    rng = np.random.default_rng(0)
    A = sp.random(60, 60, density=0.08, random_state=1, format="coo")
    if symmetry == "symmetric":
        A = sp.coo_matrix(sp.tril(A) + sp.tril(A, -1).T)
    elif symmetry == "skew-symmetric":
        A = sp.coo_matrix(sp.tril(A, -1) - sp.tril(A, -1).T)
    path = tmp_path / "a.mtx"
    scipy.io.mmwrite(str(path), A, symmetry=symmetry if symmetry != "general" else "general")
    _same(rio.read_matrix_market(path), scipy.io.mmread(str(path)))


def test_pattern_rectangular_duplicates_and_gzip(tmp_path):
    text = "%%MatrixMarket matrix coordinate pattern general\n% comment\n\n3 5 5\n1 1\n3 5\n3 2\n1 1\n2 4\n"
    path = tmp_path / "p.mtx.gz"
    with gzip.open(path, "wt") as f:
        f.write(text)
    m, n, rp, col, val = rio.read_matrix_market(path)
    assert (m, n) == (3, 5) and rp.tolist() == [0, 1, 2, 4] and col.tolist() == [0, 3, 1, 4]
    assert val.tolist() == [2.0, 1.0, 1.0, 1.0]  # the duplicate (1,1) is summed
    empty = tmp_path / "e.mtx"
    empty.write_text("%%MatrixMarket matrix coordinate real general\n4 4 0\n")
    m, n, rp, col, val = rio.read_matrix_market(empty)
    assert rp.tolist() == [0] * 5 and len(col) == 0


def test_large_file_in_parallel_pieces(tmp_path, parser):
    """Several hundred thousand entries (the C++ parser cuts the text into one piece per
    thread), integer field, exponent notation, CRLF line ends, a comment between entries."""
    rng = np.random.default_rng(3)
    m, n, e = 5000, 7000, 300000 if parser else 20000
    rows, cols = rng.integers(1, m + 1, e), rng.integers(1, n + 1, e)
    vals = rng.integers(-50, 50, e)
    lines = [f"{r} {c} {v}" for r, c, v in zip(rows, cols, vals)]
    lines.insert(e // 2, "% a comment in the middle")
    path = tmp_path / "big.mtx"
    path.write_bytes(("%%MatrixMarket matrix coordinate integer general\r\n" + f"{m} {n} {e}\r\n" + "\r\n".join(lines) + "\r\n").encode())
    _same(rio.read_matrix_market(path), sp.coo_matrix((vals.astype(np.float64), (rows - 1, cols - 1)), shape=(m, n)))
    small = tmp_path / "exp.mtx"
    small.write_text("%%MatrixMarket matrix coordinate real general\n2 2 2\n1 2 1.5e+01\n2 1 -2.5E-1\n")
    mm, nn, rp, col, val = rio.read_matrix_market(small)
    assert rp.tolist() == [0, 1, 2] and col.tolist() == [1, 0] and val.tolist() == [15.0, -0.25]


@pytest.mark.parametrize("native", [True, False])
def test_rejects_symmetric_files_that_are_not_square_and_sizes_beyond_memory(tmp_path, native):
    """The mirrored entry of a symmetric file lands in row `column`: a non-square one is
    refused before anything is counted.  A size line that no machine can hold comes back as
    an error as well (nothing is thrown through the C boundary)."""
    bad = tmp_path / "s.mtx"
    for kind in ("symmetric", "skew-symmetric"):
        bad.write_text(f"%%MatrixMarket matrix coordinate real {kind}\n2 100000 2\n1 99999 1.0\n2 100000 2.0\n")
        with pytest.raises(ValueError, match="must be square"):
            rio.read_matrix_market(bad, native=native)


def test_a_size_line_beyond_memory_is_an_error_not_an_abort(tmp_path):
    """A size line whose tables cannot be allocated comes back as ValueError: nothing is
    thrown through the C boundary.  Run in a child process with its address space capped at
    4 GiB, so that the 16 GB table of row starts fails at once instead of being allocated."""
    import subprocess
    import sys
    bad = tmp_path / "huge.mtx"
    bad.write_text("%%MatrixMarket matrix coordinate real general\n2000000000 2000000000 0\n")
    code = (
        "import resource, sys\n"
        "sys.path.insert(0, %r)\n"
        "from rode_amd import io as rio\n"
        "rio._load_native()\n"
        "resource.setrlimit(resource.RLIMIT_AS, (4 << 30, 4 << 30))\n"
        "try:\n"
        "    rio.read_matrix_market(%r, native=True)\n"
        "except ValueError as e:\n"
        "    print('ValueError:', e)\n"
    ) % (str(__import__("pathlib").Path(__file__).resolve().parents[1]), str(bad))
    done = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stderr[-2000:]
    assert "ValueError" in done.stdout and "memory" in done.stdout


def test_rejects_bad_files(tmp_path):
    bad = tmp_path / "b.mtx"
    bad.write_text("%%MatrixMarket matrix array real general\n2 2\n1\n2\n3\n4\n")
    with pytest.raises(ValueError, match="coordinate"):
        rio.read_matrix_market(bad)
    bad.write_text("%%MatrixMarket matrix coordinate real general\n2 2 2\n1 1 1.0\n")
    with pytest.raises(ValueError, match="promises"):
        rio.read_matrix_market(bad)
    bad.write_text("%%MatrixMarket matrix coordinate real general\n2 2 1\n3 1 1.0\n")
    with pytest.raises(ValueError, match="out of range"):
        rio.read_matrix_market(bad)
    bad.write_text("hello\n")
    with pytest.raises(ValueError, match="not a Matrix Market"):
        rio.read_matrix_market(bad)
    bad.write_text("")
    with pytest.raises(ValueError):
        rio.read_matrix_market(bad)
    bad.write_text("%%MatrixMarket matrix coordinate real general\n2 2 1\n1 1 1.5abc\n")
    with pytest.raises(ValueError):
        rio.read_matrix_market(bad)


def test_a_number_of_any_length(tmp_path):
    """A value written with more digits than any buffer guess (80 here) is read whole."""
    f = tmp_path / "long.mtx"
    f.write_text("%%MatrixMarket matrix coordinate real general\n2 2 2\n1 1 0." + "3" * 80 + "\n2 2 " + "1" + "0" * 79 + "e-70\n")
    m, n, rp, col, val = rio.read_matrix_market(f)
    assert (m, n) == (2, 2) and rp.tolist() == [0, 1, 2] and col.tolist() == [0, 1]
    np.testing.assert_allclose(val, np.array([1 / 3, 1e9], dtype=np.float32), rtol=1e-6)


def test_pad_rows_matches_the_reference_generators():
    """The reference generators emit exactly `pad_rows(unpadded)`: drop their explicit
    zeros, pad again, get the same arrays back."""
    from rode_amd import workloads
    rp, col, val = workloads.reference_csr(97, 103, 15, poisson=True, pad_to=4, seed=42)
    assert (rp % 4 == 0).all()
    raw_rp, raw_col, raw_val = workloads.reference_csr(97, 103, 15, poisson=True, pad_to=1, seed=42)
    prp, pcol, pval = rio.pad_rows(raw_rp, raw_col, raw_val, 4)
    np.testing.assert_array_equal(prp, rp)
    np.testing.assert_array_equal(pcol, col)
    np.testing.assert_array_equal(pval, val)
    # empty rows stay empty; already aligned rows are untouched
    prp, pcol, pval = rio.pad_rows([0, 0, 4, 5], [1, 2, 3, 4, 9], np.arange(5, dtype=np.float32) + 1)
    assert prp.tolist() == [0, 0, 4, 8] and pcol.tolist() == [1, 2, 3, 4, 9, 9, 9, 9]
    assert pval.tolist() == [1, 2, 3, 4, 5, 0, 0, 0]
