"""Host-side logic that needs no GPU: argument checks that fire before any device
call, the workload generators, the result comparison."""
import numpy as np
import pytest
import torch

from rode_amd import RoDeCSR, compare_results, rode_sddmm_hip, workloads


def test_config_tables():
    assert RoDeCSR.REFERENCE_CONFIGS == {32: {"seg_length": 512, "k_block": 32, "vec_len": 4},
                                         128: {"seg_length": 32, "k_block": 32, "vec_len": 4}}
    assert set(RoDeCSR.CONFIGS) == {32, 64, 128}
    for cfg in RoDeCSR.CONFIGS.values():
        assert cfg["k_block"] == 32 and cfg["vec_len"] == 4 and cfg["seg_length"] % 32 == 0


def test_errors_raised_before_any_device_work():
    rp = torch.tensor([0, 2, 4], dtype=torch.int32)
    with pytest.raises(ValueError, match="k must be"):
        RoDeCSR(rp, torch.zeros(4, dtype=torch.int32), torch.zeros(4), "cpu", 2, 4, k=50)
    with pytest.raises(ValueError, match="k must be"):
        RoDeCSR(rp, torch.zeros(4, dtype=torch.int32), torch.zeros(4), "cpu", 2, 4, k=1024)
    for bad in ({"seg_length": 48, "k_block": 32, "vec_len": 4}, {"seg_length": 512, "k_block": 16, "vec_len": 4},
                {"seg_length": 512, "k_block": 32, "vec_len": 2}, {"seg_length": 0, "k_block": 32, "vec_len": 4}):
        with pytest.raises(ValueError, match="config must have"):
            RoDeCSR(rp, torch.zeros(4, dtype=torch.int32), torch.zeros(4), "cpu", 2, 4, k=32, config=bad)
    with pytest.raises(RuntimeError, match="int32"):
        rode_sddmm_hip.preprocess(rp.long(), 4, 512, 32, 4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        rode_sddmm_hip.preprocess_device(rp, 4, 512, 32, 4)
    cpu = torch.zeros(4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        rode_sddmm_hip.sddmm_forward(rp, rp, rp, 0, 0, rp, rp, cpu, 2, 4, cpu, cpu, 32)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        rode_sddmm_hip.spmm_forward(rp, rp, rp, 0, 0, rp, rp, cpu, 2, 4, cpu)


def test_capacity_bound_holds():
    import oracle
    rng = np.random.default_rng(0)
    for seg in (32, 64, 512):
        for _ in range(50):
            m = int(rng.integers(1, 40))
            lens = rng.integers(0, 3 * seg, size=m)
            rp = np.concatenate([[int(rng.integers(0, 4))], lens]).cumsum().astype(np.int32)
            blk, _, res = oracle.preprocess(rp, seg)
            assert len(blk) <= rode_sddmm_hip.preprocess_capacity(m, int(rp[-1]), seg, 4)
            assert len(res) <= m


def test_workloads_are_deterministic_and_well_formed():
    for name in workloads.CONFIGS:
        m, n, rp, col, val = workloads.config(name, scale=1 / 64)
        m2, n2, rp2, col2, val2 = workloads.config(name, scale=1 / 64)
        assert rp.tobytes() == rp2.tobytes() and col.tobytes() == col2.tobytes() and val.tobytes() == val2.tobytes()
        assert rp[0] == 0 and (np.diff(rp) >= 0).all() and len(col) == rp[-1] == len(val)
        assert col.min(initial=0) >= 0 and col.max(initial=0) < n
        for r in range(0, m, max(1, m // 97)):
            assert (np.diff(col[rp[r]:rp[r + 1]]) > 0).all(), "columns ascending and distinct"
    m, n, rp, col, val = workloads.config("c3_banded", 1 / 64)
    assert (np.diff(rp) == 27).all()
    m, n, rp, col, val = workloads.config("c4_powerlaw", 1 / 16)
    lens = np.diff(rp)
    assert lens.min() == 1 and 15 < lens.mean() < 35 and lens.max() > 2000
    np.testing.assert_allclose(val[rp[5]:rp[6]], 1.0 / lens[5])
    m, n, rp, col, val = workloads.config("c5_attention", 1 / 8)
    assert (val == 1).all() and np.diff(rp).max() <= 512 + 64


def test_reference_generators():
    rp, col, val = workloads.reference_csr(64, 64, 8)
    assert (rp % 4 == 0).all() and rp[-1] == len(col)
    lens = np.diff(rp)
    assert lens.min() >= 4 and lens.max() <= 16
    pads = val == 0
    assert pads.sum() > 0 and (np.abs(val[~pads]) <= 1).all()
    rp2, col2, val2 = workloads.reference_csr(64, 64, 8)
    assert col.tobytes() == col2.tobytes() and val.tobytes() == val2.tobytes()
    rp3, _, _ = workloads.reference_csr(1000, 1, 1, poisson=True)
    assert (np.diff(rp3) == 4).all()  # one real entry + three pads
    d = workloads.reference_dense(3, 5, 123)
    assert d.shape == (3, 5) and (np.abs(d) <= 1).all()
    np.testing.assert_array_equal(d, workloads.reference_dense(3, 5, 123))
    # first value of std::mt19937(123) through uniform_real_distribution<float>(-1, 1)
    first = np.float32(2.0) * np.float32(2991312382 / 4294967296.0) - np.float32(1.0)
    assert abs(d[0, 0] - first) < 1e-6


def test_compare_results_rule():
    class Fake:
        values = torch.tensor([1.0, 0.0, 2.0, 3.0])
    ref = torch.sparse_csr_tensor(torch.tensor([0, 3]), torch.tensor([0, 1, 2]), torch.tensor([1.0, 2.0, 3.0]), size=(1, 4))
    ok = compare_results(torch.tensor([1.0, 99.0, 2.0005, 3.0]), ref, Fake())
    assert ok["passed"] and ok["total_count"] == 3 and ok["error_count"] == 0  # padding skipped, small error tolerated
    bad = compare_results(torch.tensor([1.0, 0.0, 2.1, 3.0]), ref, Fake())
    assert not bad["passed"] and bad["error_count"] == 1
    size = compare_results(torch.tensor([1.0, 5.0, 2.0, 3.0]), ref, type("F", (), {"values": torch.ones(4)})())
    assert not size["passed"] and size["error_count"] == -1


def test_auto_config_picks_the_segment_length_from_the_row_lengths():
    """The choice follows the measured sweep: 128 for small matrices, else one segment per
    row where possible (512..2048), 512 when no row has block segments (reference table:
    rode_sddmm.py:35-38)."""
    from rode_amd import workloads
    want = {"c1_uniform": (1.0, 128), "c2_lognormal": (1.0, 128), "c3_banded": (0.05, 512),
            "c4_powerlaw": (0.25, 512), "c5_attention": (1.0, 1024)}
    for name, (scale, seg) in want.items():
        _, _, rp, _, _ = workloads.config(name, scale)
        cfg = RoDeCSR.auto_config(torch.from_numpy(rp))
        assert cfg == {"seg_length": seg, "k_block": 32, "vec_len": 4}, (name, cfg)
    # rows of about 1500 slots, many of them: one segment per row
    rp = np.zeros(40001, dtype=np.int64)
    rp[1:] = np.cumsum(np.full(40000, 1500))
    assert RoDeCSR.auto_config(torch.from_numpy(rp))["seg_length"] == 2048
    assert RoDeCSR.auto_config(torch.zeros(5, dtype=torch.int32))["seg_length"] == 512


def test_auto_config_with_more_rows_than_a_library_quantile_takes():
    """17 M rows with block segments (torch.quantile refuses more than 16 M elements): the
    90th percentile is taken as an order statistic, whatever the count."""
    m = 17_000_000
    lens = torch.full((m,), 40, dtype=torch.int64)
    lens[: m // 5] = 1500  # 20 % long rows: the 90th percentile is 1500 -> 2048
    rp = torch.zeros(m + 1, dtype=torch.int64)
    rp[1:] = torch.cumsum(lens, 0)
    assert RoDeCSR.auto_config(rp)["seg_length"] == 2048
    lens[: m // 5] = 40
    lens[: m // 20] = 1500  # 5 % long rows: the 90th percentile is 40 (+ 0..3 of alignment) -> 512
    rp[1:] = torch.cumsum(lens, 0)
    assert RoDeCSR.auto_config(rp)["seg_length"] == 512
