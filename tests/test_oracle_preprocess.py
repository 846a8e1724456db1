"""Pins oracle.preprocess (the restatement of RoDe_SDDMM/main.cu:114-163) without
running the reference: hand-worked vectors, the independent closed form of
Preprocess_opt/_preprocess.cu:262-270 + prefix sums, the exact-once coverage
invariant of the kernels' index ranges, ordering invariants, analytic cases and a
brute-force walk on tiny inputs."""
import json
import os

import numpy as np
import pytest

import oracle
from helpers import closed_form_preprocess, coverage_counts, random_row_ptr

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "preprocess_handworked.json")
PARAM_SETS = [(512, 32, 4), (32, 32, 4), (256, 32, 4), (64, 32, 4), (1024, 32, 4)]


def test_handworked_vectors():
    cases = json.load(open(GOLDEN))["cases"]
    assert len(cases) >= 6
    for c in cases:
        seg, kb, vl = c["params"]
        blk, st, res = oracle.preprocess(c["row_ptr"], seg, kb, vl)
        assert res.tolist() == c["residue_r_ind"], c["name"]
        if "block_r_ind" in c:
            assert blk.tolist() == c["block_r_ind"], c["name"]
            assert st.tolist() == c["st_off"], c["name"]
        else:
            assert len(blk) == c["n_blk"], c["name"]
            k = len(c["st_off_prefix"])
            assert blk[:k].tolist() == c["block_r_ind_prefix"], c["name"]
            assert st[:k].tolist() == c["st_off_prefix"], c["name"]
            assert st[-1] == c["st_off_last"], c["name"]


@pytest.mark.parametrize("params", PARAM_SETS)
@pytest.mark.parametrize("seed", range(4))
def test_matches_closed_form_and_invariants(params, seed):
    seg, kb, vl = params
    rng = np.random.default_rng(seed)
    rp = random_row_ptr(rng, 3000, [3, 20, 40, 200][seed], long_rows=12, long_len=[700, 5000, 2100, 40000][seed])
    blk, st, res = oracle.preprocess(rp, seg, kb, vl)
    cblk, cst, cres = closed_form_preprocess(rp, seg, kb, vl)
    np.testing.assert_array_equal(blk, cblk)
    np.testing.assert_array_equal(st, cst)
    np.testing.assert_array_equal(res, cres)
    # ordering
    assert (np.diff(blk) >= 0).all() and (np.diff(res) > 0).all() and (np.diff(st) > 0).all()
    assert st[-1] == rp[-1]
    # every nonzero is processed exactly once, by its own row, and no segment is longer than seg
    hits, owner = coverage_counts(rp, blk, st, res, kb, vl)
    assert (hits == 1).all()
    np.testing.assert_array_equal(owner, np.repeat(np.arange(len(rp) - 1), np.diff(rp)))
    seg_len = np.minimum(rp[blk.astype(np.int64) + 1], st[1:]) - st[:-1] + st[:-1] % vl
    assert (seg_len // kb * kb <= seg).all() and (seg_len >= kb).all()


def test_analytic_cases():
    M = 1000
    # 27 per row at stride 27: N in {27..30} < 32 -> residues only, for both reference parameter sets
    rp = np.arange(M + 1) * 27
    for seg in (512, 32):
        blk, st, res = oracle.preprocess(rp, seg)
        assert len(blk) == 0 and st.tolist() == [27 * M] and res.tolist() == list(range(M))
    # 32 per row, aligned: one block each, no residue
    rp = np.arange(M + 1) * 32
    blk, st, res = oracle.preprocess(rp, 512)
    assert blk.tolist() == list(range(M)) and st.tolist() == rp.tolist() and len(res) == 0
    # 576 per row (aligned): seg 512 -> 2 blocks + residue? 576 = 512 + 64 -> (s), (s+512), 64 % 32 == 0 -> no residue
    rp = np.arange(M + 1) * 576
    blk, st, res = oracle.preprocess(rp, 512)
    assert len(blk) == 2 * M and len(res) == 0
    blk, st, res = oracle.preprocess(rp, 32)
    assert len(blk) == 18 * M and len(res) == 0
    # one row of 200000: ceil-style split, 200000 = 390*512 + 320 -> 391 blocks, 320 % 32 == 0
    blk, st, res = oracle.preprocess([0, 200000], 512)
    assert len(blk) == 391 and len(res) == 0 and st[1] == 512 and st[-2] == 390 * 512
    # zero rows
    blk, st, res = oracle.preprocess([7], 512)
    assert len(blk) == 0 and len(res) == 0 and st.tolist() == [7]


def _brute_force(rp, seg, kb, vl):
    """Element-by-element walk: label every aligned slot of a row with the work
    item that must own it, then read the lists off the labels."""
    blk, st, res = [], [], []
    for r in range(len(rp) - 1):
        s, e = rp[r], rp[r + 1]
        a0 = s - s % vl
        slots = list(range(a0, e))  # aligned slots of the row
        pos = 0
        first = True
        while len(slots) - pos > seg:
            blk.append(r); st.append(s if first else slots[pos]); first = False
            pos += seg
        rest = len(slots) - pos
        if rest > 0:
            if rest >= kb:
                blk.append(r); st.append(s if first else slots[pos])
            if rest % kb:
                res.append(r)
    st.append(rp[-1])
    return blk, st, res


def test_brute_force_tiny():
    rng = np.random.default_rng(7)
    for _ in range(300):
        m = int(rng.integers(1, 6))
        seg, kb, vl = [(8, 4, 2), (8, 8, 4), (16, 4, 4), (12, 4, 2), (32, 32, 4)][int(rng.integers(5))]
        lens = rng.integers(0, 4 * seg, size=m)
        rp = np.concatenate([[int(rng.integers(0, 5))], lens]).cumsum()
        blk, st, res = oracle.preprocess(rp, seg, kb, vl)
        b2, s2, r2 = _brute_force(rp.tolist(), seg, kb, vl)
        assert blk.tolist() == b2 and st.tolist() == s2 and res.tolist() == r2, (rp, seg, kb, vl)


@pytest.mark.parametrize("seg", [32, 64, 96, 512, 48, 80, 100, 36, 16])
def test_block_kernel_ranges_stay_in_their_row_for_any_segment_length(seg):
    """The SpMM/SDDMM entry points are specified for seg_length % 32 == 0, where every
    nonzero is covered exactly once.  Lists made with another segment length (the C ABI
    cannot tell) must still keep every access of the merging block kernels inside the
    arrays and inside the leader's own row, with no index written twice; they may leave
    nonzeros out (the reference's kernels drop slots there too)."""
    import oracle
    from helpers import merged_block_ranges, residue_ranges
    rng = np.random.default_rng(seg)
    for trial in range(40):
        m = int(rng.integers(1, 60))
        lens = rng.choice([0, 1, 3, 31, 32, 33, 47, 48, 49, 95, 96, 97, 130, 500, 1300], size=m)
        rp = np.concatenate([[int(rng.integers(0, 4))], lens]).cumsum().astype(np.int32)
        blk, st, res = oracle.preprocess(rp, seg)
        nnz = int(rp[-1])
        for merge in (128, 512):
            hits = np.zeros(nnz, np.int32)
            for r, first_read, first_written, end in merged_block_ranges(rp, blk, st, merge):
                assert 0 <= first_read and end <= nnz, "read outside col/val"
                assert rp[r] <= first_written and end <= rp[r + 1], "write outside the leader's row"
                hits[first_written:end] += 1
            for r, first, end in residue_ranges(rp, res):
                assert rp[r] <= first and end <= rp[r + 1]
                hits[first:end] += 1
            assert hits.max(initial=0) <= 1, "an index is written by two work items"
            if seg % 32 == 0:
                assert (hits[rp[0]:] == 1).all(), "a nonzero is left out"
