#!/usr/bin/env python3
"""Benchmark of the RoDe hot path on one MI355X.

A step is one pass over one synthetic matrix: clear the rows of C that SpMM adds to
(or all of C with --memset-c, the reference's contract), SpMM (C = A @ B), SDDMM
(out = A (.) (L @ R^T)), all through the C ABI with every operand already in
HBM.  Default workload: the power-law configuration at K = 128.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--k K] [--seg SEG]

Prints one JSON line: GFLOP/s (2*nnz*K per operation), the roofline figures of
the kernel that takes the most time (algorithmic bytes / measured duration
against 8 TB/s), and the CPU baseline (the oracle, timed on this host).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
CLOCK_HZ = 2.4e9        # MI355X peak engine clock
CUS, SIMDS = 256, 1024
# fp32 multiply-adds of the vector units without packed instructions (this build compiles none):
# 1024 SIMDs x 16 lanes x 2 flop x 2.4 GHz; the published 157.3 TFLOP/s counts two per lane and clock
VALU_PEAK_TFLOPS = 78.6
# LDS reads: 107 bytes per clock and CU is what ds_read_b128 of random rows sustains on this GPU
# (measured with a stand-alone gather loop; conflict-free reads reach 205)
LDS_PEAK_GBS = 107.0 * CUS * CLOCK_HZ / 1e9
# Vector memory pipe (address unit + L1 of a CU): 64 bytes per clock and CU; a stand-alone loop of
# 16-byte-per-lane gathers of 128..512-byte rows sustains 57-60 B/clk/CU from an L1-resident table and
# 53-55 from an L2-resident one on this GPU
VMEM_PEAK_GBS = 64.0 * CUS * CLOCK_HZ / 1e9
TOL = {"f32": 1e-4, "f16": 2e-3}  # max over rows of |err|_inf / |ref row|_1


def kernel_sources_fingerprint():
    """Hash of the code of the SpMM / SDDMM kernel sources (comments and blank lines left
    out, so that rewording a comment does not disown a measurement).  Every entry of
    profiles/traffic.json carries the fingerprint of the sources it was measured on; an
    entry measured on other sources is not reported."""
    import hashlib
    import re
    h = hashlib.sha256()
    for name in ("rode_device.hpp", "rode_items.hpp", "rode_units.hpp", "rode_window.hpp", "rode_spmm.hip", "rode_sddmm.hip",
                 "rode_spmm_window.hip", "rode_sddmm_window.hip", "rode_attention.hip", "rode_attention_backward.hip",
                 "rode_group.hip", "rode_hub.hip"):
        with open(os.path.join(ROOT, "rode_amd", "csrc", name), "r", encoding="utf-8") as f:
            for line in f:
                code = re.sub(r"//.*$", "", line).strip()
                if code:
                    h.update(code.encode("utf-8") + b"\n")
    return h.hexdigest()[:16]


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=20)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--workload", default="c4_powerlaw")
    p.add_argument("--k", type=int, default=128, help="dense width (SpMM n, SDDMM k)")
    p.add_argument("--seg", type=int, default=0,
                   help="segment length (0: picked from the row lengths by RoDeCSR.auto_config; -1: the fixed table)")
    p.add_argument("--dtype", default="f32", choices=["f32", "f16"], help="dense operand type (accumulation is fp32)")
    p.add_argument("--scale", type=float, default=1.0, help="shrink the matrix (debugging only)")
    p.add_argument("--cpu-seconds", type=float, default=8.0, help="CPU time budget per operation of the baseline")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    p.add_argument("--no-contract", action="store_true",
                   help="skip the extra timing of SpMM under the reference's calling contract (for profiler runs: its "
                        "launches of the same kernels on other arguments would enter the per-kernel averages)")
    p.add_argument("--two-streams", action="store_true",
                   help="residue kernels on a second stream (forked from / joined to the first with events)")
    p.add_argument("--fused", choices=["no", "yes", "probs", "scores"], default="no",
                   help="with --chain: the step is the one-kernel attention forward (rode_hip_attention_forward_batched); "
                        "\"probs\" also writes the probabilities a gradient needs, \"scores\" the scaled scores and every "
                        "row's (maximum, 1 / sum) instead (what sparse_attention keeps for its gradient)")
    p.add_argument("--chain", action="store_true",
                   help="step = SDDMM scores -> row softmax -> clear C -> SpMM with those values (sparse attention)")
    p.add_argument("--heads", type=int, default=1,
                   help="with --chain --fused yes/probs/scores: attention heads on the one mask, all in the same launches")
    p.add_argument("--train", action="store_true",
                   help="with --chain --fused probs|scores: the step is the attention forward with what a gradient needs written "
                        "plus the two gradient kernels (rode_hip_attention_backward_rows / _cols)")
    p.add_argument("--memset-c", action="store_true",
                   help="clear all of C before SpMM (the reference's contract) instead of only the rows SpMM adds to")
    p.add_argument("--no-plan", action="store_true",
                   help="do not use the locality plan (window kernels for chunks whose dense rows fit an LDS window)")
    p.add_argument("--graph", action="store_true",
                   help="capture one step in a HIP graph and time its replays (launch-bound workloads)")
    p.add_argument("--calibrate", action="store_true",
                   help="also run one plain device copy of 256 MiB (a known size to scale profiler counters by)")
    return p.parse_args()


def work_split(row_ptr, col, ncols, owned_slots=0, hub_min_len=0, group_rows=None):
    """Which nonzeros the residue kernels own (tail rule of RoDeSpmm.cu:71-82) and how
    many distinct dense rows each kernel family touches.  ``owned_slots``: rows of
    32..owned_slots aligned slots are summed, tail included, by the SpMM block kernel.
    ``hub_min_len`` > 0: rows of at least that many aligned slots belong, whole, to the
    hub kernels.  ``group_rows``: mask of the rows that belong, whole, to the group kernels
    (counted under the same "hub" keys: a plan is one or the other)."""
    rp = row_ptr.astype(np.int64)
    s, e = rp[:-1], rp[1:]
    pad = s % 4
    N = e - s + pad
    hub_row = (N >= hub_min_len) if hub_min_len > 0 else np.zeros(len(N), dtype=bool)
    if group_rows is not None:
        hub_row = group_rows
    tail_first = np.where(N >= 32, s - pad + N // 32 * 32, s)
    tail_first = np.where((N >= 32) & (N <= owned_slots), e, tail_first)
    in_hub = np.repeat(hub_row, e - s)
    in_res = (np.arange(rp[-1], dtype=np.int64) >= np.repeat(tail_first, e - s)) & ~in_hub
    in_blk = ~in_res & ~in_hub
    nnz_res, nnz_hub = int(in_res.sum()), int(in_hub.sum())
    distinct = lambda mask: int((np.bincount(col[mask], minlength=ncols) > 0).sum())
    rows_blk = int(((N >= 32) & ~hub_row).sum())
    rows_res = int((((N % 32) != 0) & (N > 0) & ~((N >= 32) & (N <= owned_slots)) & ~hub_row).sum())
    return {"nnz_res": nnz_res, "nnz_blk": int(rp[-1]) - nnz_res - nnz_hub, "nnz_hub": nnz_hub,
            "distinct_res": distinct(in_res), "distinct_blk": distinct(in_blk), "distinct_hub": distinct(in_hub),
            "rows_blk": rows_blk, "rows_res": rows_res, "rows_hub": int(hub_row.sum())}


def algorithmic_bytes(kernel, split, m1, m2, k, elem):
    """Compulsory traffic of one launch: every array element it needs, once."""
    if kernel.endswith("block"):
        nnz, rows, distinct, meta = split["nnz_blk"], split["rows_blk"], split["distinct_blk"], m1 * 12 + 4
    elif kernel.endswith("hub") or kernel.endswith("group"):  # (a group: 32 bytes of plan for four rows)
        nnz, rows, distinct, meta = split["nnz_hub"], split["rows_hub"], split["distinct_hub"], split["rows_hub"] * 12
    else:
        nnz, rows, distinct, meta = split["nnz_res"], m2, split["distinct_res"], m2 * 12
    if kernel.startswith("spmm"):
        # (col, val) + metadata + distinct B rows + C rows (atomic rows are read and written)
        c_bytes = rows * k * 4 * (2 if kernel.endswith("block") else 1)  # (hub rows and short rows are stored)
        return nnz * 8 + meta + distinct * k * elem + c_bytes
    # sddmm: (col, val) + metadata + lhs rows + distinct rhs rows + out
    return nnz * 8 + meta + rows * k * elem + distinct * k * elem + nnz * 4


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this build has no multi-GPU path)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from rode_amd import RoDeCSR, _lib, rode_sddmm_hip, workloads

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    lib = _lib.load()
    k = args.k
    elem = 4 if args.dtype == "f32" else 2
    tdtype = torch.float32 if args.dtype == "f32" else torch.float16

    t0 = time.time()
    m, n, row_ptr, col, val = workloads.config(args.workload, args.scale)
    nnz = int(row_ptr[-1])
    cfg = "auto" if args.seg == 0 else None if args.seg < 0 else {"seg_length": args.seg, "k_block": 32, "vec_len": 4}
    csr = RoDeCSR(torch.from_numpy(row_ptr), torch.from_numpy(col), torch.from_numpy(val), dev, m, n,
                  k if k in RoDeCSR.CONFIGS else 128, config=cfg, locality=False if args.no_plan else "auto")
    gen = torch.Generator(device=dev).manual_seed(3000)
    B = torch.randn(n, k, device=dev, generator=gen).to(tdtype)     # SpMM dense operand, also SDDMM rhs
    L = torch.randn(m, k, device=dev, generator=gen).to(tdtype)     # SDDMM lhs
    C = torch.zeros(m, k, device=dev)
    out = torch.empty(nnz, device=dev)
    setup_s = time.time() - t0

    stream = torch.cuda.current_stream().cuda_stream
    import ctypes
    hub = csr.plan if isinstance(csr.plan, rode_sddmm_hip.HubPlan) else None
    grp = csr.plan if isinstance(csr.plan, rode_sddmm_hip.GroupPlan) else None
    lists_run = grp is None or grp.counts[2] > 0  # (with every row in a group the list kernels are not launched)
    spmm_plans = ctypes.byref(rode_sddmm_hip.plans_struct(csr.plan, k, 4, seg_length=csr.config["seg_length"]))
    sddmm_plans = ctypes.byref(rode_sddmm_hip.plans_struct(csr.plan, seg_length=csr.config["seg_length"]))

    # Every row of C stored by its one work item (no row without slots, none cut into several work items):
    # then C needs no clearing, and the kernels are told to store instead of add.
    stores_c = csr.spmm_stores_every_row() and not args.memset_c
    spmm_flags = _lib.SPMM_WHOLE_LISTS | (_lib.SPMM_OVERWRITE if stores_c else 0)

    def spmm_fn(*a, flags=0):  # the whole decomposition is passed, and the library is told so
        return lib.rode_hip_spmm_planned(_lib.DENSE_CODE[args.dtype], spmm_flags | flags, *a[:-2],
                                         spmm_plans, *a[-2:])

    def sddmm_fn(*a, flags=0):
        return lib.rode_hip_sddmm_planned(_lib.DENSE_CODE[args.dtype], flags, *a[:-2], sddmm_plans, *a[-2:])

    main_stream = torch.cuda.current_stream()
    side = torch.cuda.Stream() if args.two_streams else None

    def fork():
        if side is None:
            return stream
        side.wait_stream(main_stream)
        return side.cuda_stream

    def join():
        if side is not None:
            main_stream.wait_stream(side)

    def spmm_only(flag):  # one kernel of the pair, every other decision as in the full call
        _lib.check(spmm_fn(csr.m1, csr.m2, n, k, csr.values.data_ptr(), csr.column_indices.data_ptr(),
                           csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(),
                           csr.st_offsets.data_ptr(), B.data_ptr(), C.data_ptr(), stream, stream, flags=flag), "spmm")

    def spmm_reference_contract():
        # what a caller of the reference-signature API does (RoDeSpmm.cu:492-509): memset all of C,
        # then the typed entry point, which is promised nothing about the lists
        C.zero_()
        fn = {"f32": lib.rode_hip_spmm_f32, "f16": lib.rode_hip_spmm_f16}[args.dtype]
        _lib.check(fn(csr.m1, csr.m2, n, k, csr.values.data_ptr(), csr.column_indices.data_ptr(),
                      csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(),
                      csr.st_offsets.data_ptr(), B.data_ptr(), C.data_ptr(), stream, stream), "spmm")

    def spmm(m1, m2):
        s2 = fork()
        _lib.check(spmm_fn(m1, m2, n, k, csr.values.data_ptr(), csr.column_indices.data_ptr(),
                           csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(),
                           csr.st_offsets.data_ptr(), B.data_ptr(), C.data_ptr(), stream, s2), "spmm")
        join()

    def sddmm(m1, m2, flags=0):
        s2 = fork()
        _lib.check(sddmm_fn(m1, m2, n, k, csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(),
                            csr.st_offsets.data_ptr(), csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(),
                            csr.values.data_ptr(), L.data_ptr(), B.data_ptr(), out.data_ptr(), stream, s2, flags=flags),
                   "sddmm")
        join()

    H = args.heads
    if H > 1 and not (args.chain and args.fused != "no"):
        print("bench.py: --heads needs --chain --fused yes|probs|scores", file=sys.stderr)
        sys.exit(2)
    probs = torch.empty(H * nnz, device=dev) if args.chain else None
    # (--fused scores: the forward kernel leaves scaled scores in `probs` and every row's (maximum, 1 / sum) here)
    row_stats = torch.empty(H * m, 2, device=dev) if args.chain and args.fused == "scores" else None
    if H > 1:  # (every head its own q, k, v)
        B = torch.randn(H * n, k, device=dev, generator=gen).to(tdtype)
        L = torch.randn(H * m, k, device=dev, generator=gen).to(tdtype)
        C = torch.zeros(H * m, k, device=dev)
    if args.chain:
        args.no_cpu = True  # (the CPU leg and its parity gate are those of SpMM + SDDMM; the chain is checked by the tests)
    if args.train:
        if not (args.chain and args.fused in ("probs", "scores")):
            print("bench.py: --train needs --chain --fused probs|scores", file=sys.stderr)
            sys.exit(2)
        csr_t, _ = csr.transpose(with_values=False)
        t_slot = csr.transposed_slots()
        grp_t = csr_t.plan if isinstance(csr_t.plan, rode_sddmm_hip.GroupPlan) else None
        plans_t = ctypes.byref(rode_sddmm_hip.plans_struct(grp_t))
        G = torch.randn(H * m, k, device=dev, generator=gen)  # gradient of the loss with respect to the output
        dQ, dK, dV = (torch.empty(H * r, k, device=dev) for r in (m, n, n))
        pairs = torch.empty(2 * H * nnz, device=dev)

    def backward_rows():
        _lib.check(lib.rode_hip_attention_backward_rows(
            _lib.DENSE_CODE[args.dtype], H, m, n, nnz, k, csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(),
            csr.values.data_ptr(), probs.data_ptr(), row_stats.data_ptr() if row_stats is not None else None, G.data_ptr(),
            C.data_ptr(), B.data_ptr(), B.data_ptr(),
            float(k) ** -0.5, t_slot.data_ptr(), dQ.data_ptr(), pairs.data_ptr(), sddmm_plans, stream),
            "attention backward, rows")

    def backward_cols():
        _lib.check(lib.rode_hip_attention_backward_cols(
            _lib.DENSE_CODE[args.dtype], H, m, n, nnz, k, csr_t.row_offsets.data_ptr(), csr_t.column_indices.data_ptr(),
            pairs.data_ptr(), G.data_ptr(), L.data_ptr(), dK.data_ptr(), dV.data_ptr(), plans_t, stream),
            "attention backward, columns")

    def clear_c():
        if stores_c:
            return
        if args.memset_c:
            C.zero_()
        else:
            _lib.check(lib.rode_hip_spmm_clear_rows(m, k, 4, csr.row_offsets.data_ptr(), C.data_ptr(), stream), "clear")

    def spmm_chain():
        _lib.check(spmm_fn(csr.m1, csr.m2, n, k, probs.data_ptr(), csr.column_indices.data_ptr(),
                           csr.row_offsets.data_ptr(), csr.block_indices.data_ptr(), csr.residue_indices.data_ptr(),
                           csr.st_offsets.data_ptr(), B.data_ptr(), C.data_ptr(), stream, stream), "spmm")

    def attention_forward():
        _lib.check(lib.rode_hip_attention_forward_batched(
            _lib.DENSE_CODE[args.dtype], H, m, n, nnz, k, csr.row_offsets.data_ptr(), csr.column_indices.data_ptr(),
            csr.values.data_ptr(), L.data_ptr(), B.data_ptr(), B.data_ptr(), float(k) ** -0.5, C.data_ptr(),
            probs.data_ptr() if args.fused in ("probs", "scores") else None,
            row_stats.data_ptr() if row_stats is not None else None, sddmm_plans, stream), "attention")

    def step():
        if args.chain and args.fused != "no":
            attention_forward()
            if args.train:
                backward_rows()
                backward_cols()
            return
        if args.chain:
            sddmm(csr.m1, csr.m2)
            _lib.check(lib.rode_hip_csr_softmax_f32(m, csr.row_offsets.data_ptr(), out.data_ptr(), probs.data_ptr(),
                                                    float(k) ** -0.5, stream), "softmax")
            clear_c()
            spmm_chain()
            return
        clear_c()
        spmm(csr.m1, csr.m2)
        sddmm(csr.m1, csr.m2)

    run_step = step
    if args.graph:
        # the step allocates nothing and never waits for the host, so it can be captured as it is
        side_stream = torch.cuda.Stream()
        side_stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side_stream):
            stream = side_stream.cuda_stream
            step()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side_stream):
                step()
        stream = torch.cuda.current_stream().cuda_stream
        run_step = graph.replay
    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    flops_per_step = (6 if args.train else 2) * (2.0 * nnz * k) * args.heads  # (a gradient: four more products)
    gflops = flops_per_step / (ms_per_step * 1e-3) / 1e9

    # ---- per-kernel durations, HIP events on the launch stream ----------------
    def event_time(fn, reps):
        fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        b.synchronize()
        return a.elapsed_time(b) / reps  # ms

    # preprocessing (excluded from the step, reported on its own): the two launches of one call
    from rode_amd import rode_sddmm_hip
    cap = rode_sddmm_hip.preprocess_capacity(m, nnz, csr.config["seg_length"], 4)
    p_blk = torch.empty(cap + 1, dtype=torch.int32, device=dev)
    p_st = torch.empty(cap + 2, dtype=torch.int32, device=dev)
    p_res = torch.empty(max(m, 1), dtype=torch.int32, device=dev)
    p_cnt = torch.empty(2, dtype=torch.int32, device=dev)
    ws_bytes = lib.rode_hip_preprocess_workspace_bytes(m)
    p_ws = torch.empty((ws_bytes + 7) // 8, dtype=torch.int64, device=dev)

    def preprocess():
        _lib.check(lib.rode_hip_preprocess(csr.config["seg_length"], 32, 4, m, csr.row_offsets.data_ptr(),
                                           p_blk.data_ptr(), p_st.data_ptr(), p_res.data_ptr(), p_cnt.data_ptr(),
                                           p_cnt.data_ptr() + 4, cap, p_ws.data_ptr(), ws_bytes, stream), "preprocess")

    reps = max(3, min(args.steps, 20))
    preprocess_ms = event_time(preprocess, reps)
    pre_bytes = (m + 1) * 4 + (2 * csr.m1 + 1 + csr.m2) * 4
    del p_blk, p_st, p_res, p_ws
    kernels = {}
    if csr.m1 > 0 and lists_run:
        kernels["spmm_block"] = event_time(lambda: spmm_only(_lib.SPMM_ONLY_BLOCK), reps)  # incl. rows summed whole
        kernels["sddmm_block"] = event_time(lambda: sddmm(csr.m1, csr.m2, _lib.SPMM_ONLY_BLOCK), reps)
    if csr.m2 > 0 and lists_run:
        kernels["spmm_residue"] = event_time(lambda: spmm_only(_lib.SPMM_ONLY_RESIDUE), reps)
        kernels["sddmm_residue"] = event_time(lambda: sddmm(csr.m1, csr.m2, _lib.SPMM_ONLY_RESIDUE), reps)
    if hub is not None:  # the rows of the hub plan: piece kernel (+ the sum of the partial rows of C for SpMM)
        kernels["spmm_hub"] = event_time(lambda: spmm_only(_lib.SPMM_ONLY_HUB), reps)
        kernels["sddmm_hub"] = event_time(lambda: sddmm(csr.m1, csr.m2, _lib.SPMM_ONLY_HUB), reps)
    if grp is not None:  # the rows of the group plan's groups (the same flag selects them)
        kernels["spmm_group"] = event_time(lambda: spmm_only(_lib.SPMM_ONLY_HUB), reps)
        kernels["sddmm_group"] = event_time(lambda: sddmm(csr.m1, csr.m2, _lib.SPMM_ONLY_HUB), reps)
    if args.chain and args.fused != "no":
        kernels["attention_forward"] = event_time(attention_forward, reps)
    if args.train:
        kernels["attention_backward_rows"] = event_time(backward_rows, reps)
        kernels["attention_backward_cols"] = event_time(backward_cols, reps)
    spmm_ms = event_time(lambda: (clear_c(), spmm(csr.m1, csr.m2)), reps)
    sddmm_ms = event_time(lambda: sddmm(csr.m1, csr.m2), reps)
    spmm_contract_ms = float("nan") if args.no_contract else event_time(spmm_reference_contract, reps)

    if args.calibrate:
        src = torch.ones(64 * 2**20, device=dev)  # 256 MiB read + 256 MiB written by one elementwise copy kernel
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # the SpMM block kernel sums rows of 32..1024 slots whole when there are >= 1024 segments (kOwnedMinSegments)
    hub_min_len = hub.counts[2] if hub is not None else 0
    group_rows = None
    if grp is not None:
        group_rows = np.zeros(m, dtype=bool)
        group_rows[: 4 * grp.counts[0]] = np.repeat(grp.groups()[:, 1] > 0, 4)
    split_sddmm = work_split(row_ptr, col, n, 0, hub_min_len, group_rows)
    split_spmm = work_split(row_ptr, col, n, 1024 if csr.m1 >= 1024 else 0, hub_min_len, group_rows)
    per_kernel = {}
    for name, ms in kernels.items():
        if name.startswith("attention"):
            # row pass: (col, val, p, slot in the transposed pattern) read, (p, dz) written, rows of g, out,
            # dq, every k and v row once; column pass: row and (p, dz) read, rows of dk, dv, every g and q row once
            # forward: (col, val) read, probabilities written if asked for, q and out rows, every k and v row once
            if name.endswith("forward"):
                kept = 4 * nnz if args.fused in ("probs", "scores") else 0
                kept += 8 * m if args.fused == "scores" else 0
                ab = nnz * 8 + kept + m * k * (elem + 4) + 2 * n * k * elem
            elif name.endswith("rows"):
                ab = nnz * (16 + 8) + 3 * m * k * 4 + 2 * n * k * elem
            else:
                ab = nnz * (4 + 8) + 2 * n * k * 4 + m * k * (4 + elem)
            ab *= H
            per_kernel[name] = {"ms": round(ms, 4), "algorithmic_bytes": ab, "algorithmic_GBs": round(ab / ms / 1e6, 1),
                                "gather_model_GBs": round(H * nnz * (16 + 2 * k * elem) / ms / 1e6, 1),
                                "GFLOPs": round(H * 2 * 2.0 * nnz * k / ms / 1e6, 1)}
            continue
        split = split_spmm if name.startswith("spmm") else split_sddmm
        m2_eff = csr.m2
        if name == "spmm_residue":
            m2_eff = split["rows_res"]
        ab = algorithmic_bytes(name, split, csr.m1, m2_eff, k, elem)
        knnz = split["nnz_" + {"block": "blk", "residue": "res", "hub": "hub", "group": "hub"}[name.split("_")[1]]]
        per_kernel[name] = {"ms": round(ms, 4), "algorithmic_bytes": ab,
                            "algorithmic_GBs": round(ab / ms / 1e6, 1),
                            "gather_model_GBs": round((knnz * (8 + k * elem)) / ms / 1e6, 1),
                            "GFLOPs": round(2.0 * knnz * k / ms / 1e6, 1)}
    dominant = max(kernels, key=kernels.get)
    traffic, traffic_note, entry, windowed = None, "no counter run of this workload under profiles/", None, False
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        table = json.load(open(tpath))
        prefix = f"{args.workload}/k{k}/{args.dtype}/seg{csr.config['seg_length']}/"
        # with a locality plan the residue rows are the window kernel's
        windowed = csr.plan is not None and hub is None and grp is None and dominant.endswith("residue") and k * elem > 128
        entry = table.get(prefix + dominant + "_window") if windowed else None
        entry = entry or table.get(prefix + dominant)
        if entry is not None and entry.get("sources") == kernel_sources_fingerprint():
            traffic, traffic_note = entry["bytes"], entry.get("kernel")
        elif entry is not None:
            traffic_note = "stale: the counter run under profiles/ was made on other kernel sources"
            entry = None
    dom = per_kernel[dominant]
    dom_ms = kernels[dominant]
    hbm = {"achieved": dom["algorithmic_GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": round(dom["algorithmic_GBs"] / HBM_PEAK_GBS, 4),
           # the same kernel's measured HBM bytes over its time: how busy the memory system was
           "traffic_GBs": None if traffic is None else round(traffic / dom_ms / 1e6, 1),
           "traffic_frac": None if traffic is None else round(traffic / dom_ms / 1e6 / HBM_PEAK_GBS, 4),
           "gather_model_frac": round(dom["gather_model_GBs"] / HBM_PEAK_GBS, 4)}
    # Which resource binds the kernel: HBM when its measured traffic moves at half the peak or
    # more; else whichever is busiest of the vector ALUs (instructions issued x 4 clocks per
    # wavefront instruction over the SIMD-clocks of the launch), the LDS pipe (its active cycles
    # over the CU-clocks of the launch) and the vector memory pipe (the bytes its loads ask for over
    # 64 bytes per clock and CU; the bytes are the smaller of two upper estimates: vector loads
    # issued x 1024, i.e. every load taken as 16 bytes per lane, which the gathers are, and a dense
    # row plus 8 bytes per nonzero, which is what kernels without row sharing gather), from the
    # counters of the same profile.
    bound, busy = "hbm", {}
    if entry is not None and traffic is not None and "valu_insts" in entry:
        clocks = dom_ms * 1e-3 * CLOCK_HZ
        vmem_GBs = min(entry["vmem_reads"] * 1024 / dom_ms / 1e6, dom["gather_model_GBs"])
        busy = {"hbm": hbm["traffic_frac"], "valu": round(entry["valu_insts"] * 4 / (clocks * SIMDS), 4),
                "lds": round(entry["lds_active_cycles"] / (clocks * CUS), 4),
                "vmem": round(vmem_GBs / VMEM_PEAK_GBS, 4)}
        if windowed:  # the window kernels read every nonzero's dense row from LDS: bytes over the measured read rate
            busy["lds"] = max(busy["lds"], round(dom["GFLOPs"] * dom_ms * 1e6 / (2.0 * k) * k * elem / dom_ms / 1e6 / LDS_PEAK_GBS, 4))
        if busy["hbm"] < 0.5:
            bound = max(busy, key=busy.get)
    knnz_dom = dom["GFLOPs"] * dom_ms * 1e6 / (2.0 * k)  # nonzeros of the dominant kernel
    if bound == "valu":
        ach = dom["GFLOPs"] / 1e3
        top = {"achieved": round(ach, 2), "peak": VALU_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / VALU_PEAK_TFLOPS, 4),
               "peak_is": "fp32 vector multiply-adds without packed instructions (published 157.3 TFLOP/s counts packed pairs)"}
    elif bound == "lds":
        ach = knnz_dom * k * elem / dom_ms / 1e6  # every nonzero's dense row read from LDS once
        top = {"achieved": round(ach, 1), "peak": round(LDS_PEAK_GBS, 1), "unit": "GB/s", "frac": round(ach / LDS_PEAK_GBS, 4),
               "peak_is": "LDS read pipe: 107 B per clock and CU for 128-bit reads of random rows (measured), x 256 CUs x 2.4 GHz"}
    elif bound == "vmem":
        top = {"achieved": round(vmem_GBs, 1), "peak": round(VMEM_PEAK_GBS, 1), "unit": "GB/s",
               "frac": round(vmem_GBs / VMEM_PEAK_GBS, 4),
               "peak_is": "vector memory pipe: 64 B per clock and CU x 256 CUs x 2.4 GHz; achieved = bytes the vector loads ask for"}
    else:
        top = {k2: hbm[k2] for k2 in ("achieved", "peak", "unit", "frac")}
    roofline = {"bound": bound, "kernel": dominant, **top, "traffic": traffic, "traffic_source": traffic_note,
                "busy": busy or None, "hbm": hbm,
                "traffic_GBs": hbm["traffic_GBs"], "traffic_frac": hbm["traffic_frac"], "gather_model_frac": hbm["gather_model_frac"]}

    # ---- CPU baseline: the oracle on a bounded sample of the same matrix --------
    cpu = None
    if not args.no_cpu:
        import oracle
        Bh, Lh = B.float().cpu().numpy(), L.float().cpu().numpy()

        def cpu_ops(rows, threads):
            rp = row_ptr[: rows + 1]
            cnt = int(rp[-1])
            t = time.perf_counter()
            c_ref = oracle.spmm_f32(rp, col[:cnt], val[:cnt], Bh, threads=threads)
            t_spmm = time.perf_counter() - t
            t = time.perf_counter()
            o_ref = oracle.sddmm_f32(rp, col[:cnt], val[:cnt], Lh[:rows], Bh, threads=threads)
            t_sddmm = time.perf_counter() - t
            return cnt, t_spmm, t_sddmm, c_ref, o_ref

        probe_rows = min(m, 20000)
        cnt, a, b, _, _ = cpu_ops(probe_rows, 1)
        per_nnz = max((a + b) / max(cnt, 1), 1e-12)
        target_nnz = min(nnz, int(2 * args.cpu_seconds / per_nnz))
        rows = int(np.searchsorted(row_ptr, target_nnz, side="right")) - 1
        rows = max(1, min(m, rows))
        cnt, t_spmm, t_sddmm, c_ref, o_ref = cpu_ops(rows, 1)
        threads = oracle.num_threads()
        _, mt_spmm, mt_sddmm, _, _ = cpu_ops(rows, threads)
        # the same rows from the GPU run, as a parity gate of this very benchmark (into a C and an
        # `out` full of NaN: a row or an element that the step leaves alone, or adds to, shows)
        C.fill_(float("nan"))
        out.fill_(float("nan"))
        step()
        torch.cuda.synchronize()
        c_gpu, o_gpu = C[:rows].cpu().numpy(), out[:cnt].cpu().numpy()
        # SpMM: max over rows of |err|_inf / |ref row|_1 (reference values in fp64)
        c64 = oracle.spmm_f64(row_ptr[: rows + 1], col[:cnt], val[:cnt], Bh)
        l1 = np.abs(c64).sum(axis=1)
        spmm_err = float(np.max(np.abs(c_gpu - c64).max(axis=1) / np.maximum(l1, 1e-30)))
        # SDDMM: the same per CSR row over rows with condition number <= 100 (a row made of
        # one cancelling dot product defeats any fp32 summation), and per element against
        # the magnitude of the summed terms everywhere
        o64, scale = oracle.sddmm_f64(row_ptr[: rows + 1], col[:cnt], val[:cnt], Lh[:rows], Bh, with_abs=True)
        nonempty = np.nonzero(np.diff(row_ptr[: rows + 1]) > 0)[0]
        starts = row_ptr[:rows][nonempty].astype(np.int64)
        row_l1 = np.maximum(np.add.reduceat(np.abs(o64), starts), 1e-300)
        row_err = np.maximum.reduceat(np.abs(o_gpu - o64), starts) / row_l1
        good = np.add.reduceat(scale, starts) / row_l1 <= 100.0
        sddmm_err = float(row_err[good].max(initial=0.0))
        sddmm_err_all = float(row_err.max(initial=0.0))
        # the excluded rows: what the reference's own fp32 CPU loop (main.cu:65-91) gets on them
        cpu_row_err = np.maximum.reduceat(np.abs(o_ref - o64), starts) / row_l1
        cpu_err_bad = float(cpu_row_err[~good].max(initial=0.0))
        gpu_err_bad = float(row_err[~good].max(initial=0.0))
        sddmm_strict = float(np.max(np.abs(o_gpu - o64) / np.maximum(scale, 1e-30)))
        # the reference tests' own rule against its fp32 CPU loop: abs AND rel error above 1e-3
        diff = np.abs(o_gpu - o_ref)
        ref_rule_errors = int(((diff > 1e-3) & (diff / (np.abs(o_ref) + 1e-6) > 1e-3)).sum())
        # GPU row decomposition against the CPU routine, for the segment length in use and for
        # both parameter sets of the reference, (512,32,4) and (32,32,4); the CPU time is reported
        bit_exact, t_pre = True, 0.0
        for seg_len in sorted({csr.config["seg_length"], 512, 32}):
            t = time.perf_counter()
            oblk, ost, ores = oracle.preprocess(row_ptr, seg_len)
            if seg_len == csr.config["seg_length"]:
                t_pre = time.perf_counter() - t
            gblk, gst, gres, gm1, gm2 = rode_sddmm_hip.preprocess_device(csr.row_offsets, nnz, seg_len, 32, 4)
            bit_exact = bool(bit_exact and gm1 == len(oblk) and gm2 == len(ores)
                             and gblk.cpu().numpy()[:gm1].tobytes() == oblk.tobytes()
                             and gst.cpu().numpy().tobytes() == ost.tobytes()
                             and gres.cpu().numpy()[:gm2].tobytes() == ores.tobytes())
        cpu = {"value": round(2 * (2.0 * cnt * k) / (t_spmm + t_sddmm) / 1e9, 3), "unit": "GFLOP/s", "cores": 1,
               "kind": "port",
               "sample": f"first {rows} rows ({cnt} nnz) of the same matrix, SpMM (textbook CSR stand-in: the "
                         f"reference has no CPU SpMM) + SDDMM (restated main.cu:65-91), fp32, one thread",
               "spmm_ms": round(t_spmm * 1e3, 1), "sddmm_ms": round(t_sddmm * 1e3, 1),
               "preprocess_ms": round(t_pre * 1e3, 2),
               "all_cores": {"cores": threads,
                             "value": round(2 * (2.0 * cnt * k) / (mt_spmm + mt_sddmm) / 1e9, 3)},
               "parity_vs_gpu": {"tolerance": TOL[args.dtype], "rows_checked": int(len(nonempty)),
                                 "spmm_rowL1_err": spmm_err,
                                 "sddmm_rowL1_err_all_rows": sddmm_err_all,
                                 "sddmm_rowL1_err_cond_le_100": sddmm_err,
                                 "sddmm_rows_cond_gt_100": int((~good).sum()),
                                 "sddmm_rowL1_err_on_those_rows": {"gpu": gpu_err_bad, "reference_cpu_fp32_loop": cpu_err_bad,
                                                                   "gpu_over_cpu": round(gpu_err_bad / cpu_err_bad, 3)
                                                                   if cpu_err_bad > 0 else None},
                                 "sddmm_err_over_term_magnitude": sddmm_strict,
                                 "sddmm_reference_rule_errors": ref_rule_errors,
                                 "preprocess_bit_exact": bool(bit_exact)}}
        # the gate: a wrong result must not leave a headline number behind
        tol = TOL[args.dtype]
        failures = []
        if not bit_exact:
            failures.append("preprocessing differs from the CPU routine")
        if not spmm_err <= tol:
            failures.append(f"SpMM row-L1 error {spmm_err:.3g} > {tol}")
        if not sddmm_err <= tol:
            failures.append(f"SDDMM row-L1 error {sddmm_err:.3g} > {tol} on rows with condition <= 100")
        # (on those rows both errors are one draw each of rounding noise of size condition x eps,
        # in different summation orders, and the maximum is over a handful of rows: the ratio is
        # a sanity bound; the binding check for them is the per-element one below)
        if gpu_err_bad > max(10.0 * cpu_err_bad, tol):
            failures.append(f"SDDMM error {gpu_err_bad:.3g} on ill-conditioned rows exceeds ten times the reference CPU "
                            f"loop's {cpu_err_bad:.3g}")
        if not sddmm_strict <= (2e-6 if args.dtype == "f32" else 2e-3):
            failures.append(f"SDDMM per-element error {sddmm_strict:.3g} of the summed terms' magnitude")
        if args.dtype == "f32" and ref_rule_errors:
            failures.append(f"{ref_rule_errors} outputs fail the reference tests' rule")
        cpu["parity_vs_gpu"]["passed"] = not failures
        cpu["parity_vs_gpu"]["failures"] = failures

    line = {
        "metric": "SpMM & SDDMM GFLOP/s (2*nnz*K/t)", "value": round(gflops, 1), "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32" if elem == 4 else "f16->f32",
        "data": "synthetic",
        "config": {"workload": f"{args.workload} ({workloads.CONFIGS[args.workload][5]}), K={k}, "
                               + (("step = fused attention forward (one kernel" + (", probabilities written)" if args.fused == "probs" else ", scores and row statistics written)" if args.fused == "scores" else ")")
                                   + (" + gradient (row pass + column pass)" if args.train else "")
                                   if args.fused != "no" else "step = SDDMM -> row softmax -> clear C -> SpMM (chained)")
                                  if args.chain
                                  else ("step = SpMM (C = A B into an uninitialised C: every row is stored by its one work item) + SDDMM"
                                        if stores_c else "step = clear C rows + SpMM + SDDMM")),
                   "rows": m, "cols": n, "nnz": nnz, "K": k, "heads": args.heads, "seg_length": csr.config["seg_length"],
                   "block_segments": csr.m1, "residue_rows": csr.m2, "scale": args.scale,
                   "locality_plan": None if csr.plan is None or hub is not None or grp is not None else
                   {"residue_chunks": csr.plan.counts[0], "chunks_with_lds_window": csr.plan.counts[1]},
                   "hub_plan": None if hub is None else
                   {"hub_rows": hub.counts[0], "shortest": hub.counts[2], "nnz_share": round(split_sddmm["nnz_hub"] / nnz, 3),
                    "column_slabs": hub.counts[1], "slab_rows": 2048},
                   "group_plan": None if grp is None else
                   {"groups_of_four_rows": grp.counts[0], "groups_with_a_shared_run": grp.counts[1],
                    "rows_left_to_the_list_kernels": grp.counts[2], "nnz_share": round(split_sddmm["nnz_hub"] / nnz, 3)}},
        "spmm": {"ms": round(spmm_ms, 4), "GFLOPs": round(2.0 * nnz * k / spmm_ms / 1e6, 1), "includes": "clearing C" if not stores_c else "nothing to clear: every row of C is stored by its one work item",
                 "reference_contract_ms": None if args.no_contract else round(spmm_contract_ms, 4),
                 "reference_contract": "memset of all of C + the typed entry point without the whole-lists promise "
                                       "(RoDeSpmm.cu:492-509 semantics)"},
        "sddmm": {"ms": round(sddmm_ms, 4), "GFLOPs": round(2.0 * nnz * k / sddmm_ms / 1e6, 1)},
        "kernels": per_kernel,
        "preprocess": {"ms": round(preprocess_ms, 4), "rows_per_s": round(m / preprocess_ms * 1e3),
                       "note": "GPU row decomposition (a fill of the scan's status words + one kernel), not part of the step",
                       # compulsory bytes: row_ptr read once, both lists, the segment starts and the sentinel written once
                       "roofline": {"bound": "hbm", "algorithmic_bytes": pre_bytes,
                                    "achieved": round(pre_bytes / preprocess_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                    "frac": round(pre_bytes / preprocess_ms / 1e6 / HBM_PEAK_GBS, 4)}},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "setup_s": round(setup_s, 1),
    }
    print(json.dumps(line))
    if cpu is not None and not cpu["parity_vs_gpu"]["passed"]:
        print("bench.py: PARITY FAILED: " + "; ".join(cpu["parity_vs_gpu"]["failures"]), file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
