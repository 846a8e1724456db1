"""The C-ABI library loads and exports every symbol include/rode_hip.h declares
(no compute call is made: this runs without a GPU)."""
import ctypes
import os
import re
import subprocess

from rode_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "rode_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rode_hip_\w+)\s*\(", text)))


def test_library_is_built():
    assert os.path.exists(_lib.LIB_PATH), "run `make -C rode_amd/csrc` (or __graft_entry__.build())"


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared_symbols()
    assert len(names) >= 8
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), f"{name} declared in include/rode_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "rode_amd/_lib.py must bind exactly the declared symbols"


def test_reference_signature_entry_points_are_exported():
    out = subprocess.check_output(["nm", "-D", "--defined-only", "-C", _lib.LIB_PATH], text=True)
    for name in ("RoDeSpmm_n32(", "RoDeSpmm_n128(", "RoDeSDDMM_n32(", "RoDeSDDMM_n128(", "RoDe_preprocess(",
                 "RoDe_preprocess_cpu(int, int, int, int, int const*, int*, int*, int*, int&, int&)",
                 "RoDe_preprocess(int, int, int, int, int const*, int*, int*, int*, int&, int&)"):
        assert name in out, f"C++ entry point {name}...) missing"


def test_version_and_workspace_need_no_gpu():
    lib = _lib.load()
    assert lib.rode_hip_version() >= 1
    small, big = lib.rode_hip_preprocess_workspace_bytes(10), lib.rode_hip_preprocess_workspace_bytes(2_000_000)
    assert 0 < small < big < 64 * 2**20
    assert b"invalid" in lib.rode_hip_error_string(1).lower()
