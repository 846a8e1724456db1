"""CPU oracle for the RoDe hot path -- test infrastructure only.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline``
leg may import this package; the product (``rode_amd``) never does.
"""
from .oracle import (  # noqa: F401
    build,
    num_threads,
    preprocess,
    sddmm_f32,
    sddmm_f64,
    spmm_f32,
    spmm_d,
    spmm_f64,
)
