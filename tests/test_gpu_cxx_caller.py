"""A compiled C++ program that includes the reference-signature headers and links
librode_hip.so (tests/cxx/api_caller.cpp, built by __graft_entry__.build())."""
import json
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cxx", "api_caller")


@pytest.mark.parametrize("args", [(64, 64, 8, 128), (511, 517, 33, 32), (1023, 1031, 65, 128), (2047, 2053, 40, 32),
                                  (300, 5000, 60, 128, 512), (1, 1000, 100, 32), (1000, 3, 1, 128)])
def test_cxx_caller(args):
    assert os.path.exists(BIN), "build it with __graft_entry__.build()"
    run = subprocess.run([BIN] + [str(a) for a in args], capture_output=True, text=True, timeout=100)
    line = run.stdout.strip().splitlines()[-1] if run.stdout.strip() else ""
    assert line.startswith("{"), (run.stdout, run.stderr)
    res = json.loads(line)
    assert run.returncode == 0 and res["passed"], (res, run.stderr)
    assert res["sddmm_errors"] == 0 and res["spmm_rowL1_err"] <= 1e-4
    assert res["host_twins_equal"], "RoDe_preprocess_cpu / host RoDe_preprocess differ from the device routine"
