"""Loader of ``librode_hip.so`` (the C ABI declared in ``include/rode_hip.h``).

There is no fallback: if the library has not been built, or a call returns an
error code, a ``RuntimeError`` is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librode_hip.so")
WORKLOADS_PATH = os.path.join(_HERE, "lib", "librode_workloads.so")

c_int, c_void_p, c_size_t = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); must list every symbol include/rode_hip.h declares.
SIGNATURES = {
    "rode_hip_version": (c_int, []),
    "rode_hip_error_string": (ctypes.c_char_p, [c_int]),
    "rode_hip_preprocess_workspace_bytes": (c_size_t, [c_int]),
    "rode_hip_preprocess": (c_int, [c_int] * 4 + [c_void_p] * 6 + [c_int, c_void_p, c_size_t, c_void_p]),
    "rode_hip_preprocess_host": (c_int, [c_int] * 4 + [c_void_p] * 6),
    "rode_hip_preprocess_static": (c_int, [c_int] * 4 + [c_void_p] * 6 + [c_int, c_void_p]),
    "rode_hip_spmm_f32": (c_int, [c_int] * 4 + [c_void_p] * 10),
    "rode_hip_spmm_f16": (c_int, [c_int] * 4 + [c_void_p] * 10),
    "rode_hip_spmm_f64": (c_int, [c_int] * 4 + [c_void_p] * 10),
    "rode_hip_spmm_ex": (c_int, [c_int] * 6 + [c_void_p] * 10),
    "rode_hip_window_plan_bytes": (c_size_t, [c_int]),
    "rode_hip_window_plan": (c_int, [c_int] * 2 + [c_void_p] * 4 + [c_size_t, c_void_p, c_void_p]),
    "rode_hip_window_rows_bytes": (c_size_t, [c_int]),
    "rode_hip_window_rows": (c_int, [c_int] + [c_void_p] * 5 + [c_size_t, c_void_p]),
    "rode_hip_group_plan_bytes": (c_size_t, [c_int]),
    "rode_hip_group_plan": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
    "rode_hip_hub_plan_bytes": (c_size_t, [c_int] * 4),
    "rode_hip_hub_plan": (c_int, [c_int] * 4 + [c_void_p] * 3 + [c_size_t, c_void_p, c_void_p]),
    "rode_hip_hub_workspace_bytes": (c_size_t, [c_void_p, c_int, c_int]),
    "rode_hip_spmm_planned": (c_int, [c_int] * 6 + [c_void_p] * 11),
    "rode_hip_spmm_clear_rows": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "rode_hip_sddmm_f32": (c_int, [c_int] * 4 + [c_void_p] * 11),
    "rode_hip_sddmm_f16": (c_int, [c_int] * 4 + [c_void_p] * 11),
    "rode_hip_sddmm_planned": (c_int, [c_int] * 6 + [c_void_p] * 12),
    "rode_hip_csr_softmax_f32": (c_int, [c_int, c_void_p, c_void_p, c_void_p, ctypes.c_float, c_void_p]),
    "rode_hip_csr_softmax_backward_f32": (c_int, [c_int] + [c_void_p] * 4 + [ctypes.c_float, c_void_p]),
    "rode_hip_csr_transpose_workspace_bytes": (c_size_t, [c_int]),
    "rode_hip_csr_transpose": (c_int, [c_int] * 3 + [c_void_p] * 6 + [c_size_t, c_void_p]),
    "rode_hip_permute_f32": (c_int, [c_int] + [c_void_p] * 4),
    "rode_hip_spmm_overwrite_limit": (c_int, [c_int, c_void_p]),
    "rode_hip_attention_forward": (c_int, [c_int] * 3 + [c_void_p] * 6 + [ctypes.c_float] + [c_void_p] * 4),
    "rode_hip_attention_forward_batched": (c_int, [c_int] * 6 + [c_void_p] * 6 + [ctypes.c_float] + [c_void_p] * 5),
    "rode_hip_attention_backward_rows": (c_int, [c_int] * 6 + [c_void_p] * 9 + [ctypes.c_float] + [c_void_p] * 5),
    "rode_hip_attention_backward_cols": (c_int, [c_int] * 6 + [c_void_p] * 9),
}

class Plans(ctypes.Structure):
    """``rode_hip_plans`` of include/rode_hip.h."""
    _fields_ = [("window", c_void_p), ("window_rows", c_void_p), ("window_counts", c_void_p),
                ("hub", c_void_p), ("hub_counts", c_void_p), ("hub_workspace", c_void_p),
                ("hub_workspace_bytes", c_size_t), ("groups", c_void_p), ("group_counts", c_void_p),
                ("seg_length", c_int)]


DENSE_CODE = {"f32": 0, "f16": 1, "f64": 2}  # RODE_DENSE_* of include/rode_hip.h
SPMM_WHOLE_LISTS, SPMM_ONLY_BLOCK, SPMM_ONLY_RESIDUE, SPMM_ONLY_HUB, SPMM_OVERWRITE = 1, 2, 4, 8, 16  # RODE_SPMM_* flags

_lib = None


def load():
    """Return the ctypes handle of ``librode_hip.so`` (loaded once)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C rode_amd/csrc` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no CPU fallback"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(code, what):
    if code != 0:
        msg = load().rode_hip_error_string(code).decode()
        raise RuntimeError(f"{what} failed: {msg} (hipError {code})")
