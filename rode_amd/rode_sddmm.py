"""PyTorch-facing SDDMM op with the interface of the reference's
``RoDe_SDDMM/rode_sddmm.py``: ``RoDeCSR`` (:12-191), ``rode_sddmm`` (:194-248),
``torch_sddmm_reference`` (:251-304) and ``compare_results`` (:307-378).
"""
import math

import torch

from . import rode_sddmm_hip


class RoDeCSR:
    """CSR matrix plus its RoDe row decomposition (block segments + residues).

    Attributes (same names as the reference class): ``m, n, k, nnz, device,
    row_offsets_cpu, row_offsets, column_indices, values, block_indices,
    residue_indices, st_offsets, m1, m2``.
    """

    # The reference's table (rode_sddmm.py:35-38): its K=128 kernels handle exactly
    # one 32-slot chunk per segment, hence seg_length 32 there.
    REFERENCE_CONFIGS = {
        32: {"seg_length": 512, "k_block": 32, "vec_len": 4},
        128: {"seg_length": 32, "k_block": 32, "vec_len": 4},
    }
    # Decomposition used here, per hidden size k.  The wave64 kernels walk a segment
    # in 64-slot steps whatever its length, so one segment length serves every k;
    # 512 measured best on MI355X (short segments multiply the atomics of SpMM,
    # longer ones unbalance the waves).  Any multiple of 32 is valid, including the
    # reference's values, through the ``config`` argument; ``config="auto"`` picks the
    # length from the matrix (``auto_config``).
    CONFIGS = {
        32: {"seg_length": 512, "k_block": 32, "vec_len": 4},
        64: {"seg_length": 512, "k_block": 32, "vec_len": 4},
        128: {"seg_length": 512, "k_block": 32, "vec_len": 4},
    }

    DEFAULT_CONFIG = {"seg_length": 512, "k_block": 32, "vec_len": 4}  # for a k that is not in CONFIGS
    MAX_K = 512
    PLAN_MIN_CHUNKS = 512  # windowed chunks of 128 residue rows below which "auto" drops the plan

    def __init__(self, row_offsets, column_indices, values, device, m, n, k=128, config=None, locality="auto"):
        if not (isinstance(k, int) and 0 < k <= self.MAX_K and k % 4 == 0):
            raise ValueError(f"k must be a positive multiple of 4 up to {self.MAX_K} (the reference: 32 or 128), got {k}")
        self.m = m
        self.n = n
        self.k = k
        self.nnz = values.numel()
        self.device = torch.device(device)
        if self.device.type == "cuda" and self.device.index is None and torch.cuda.is_available():
            # "cuda" means the current GPU; tensors created there report "cuda:<index>", which is
            # what the operand checks of the ops compare with
            self.device = torch.device("cuda", torch.cuda.current_device())
        self.row_offsets_cpu = row_offsets.to(dtype=torch.int32, device="cpu").contiguous()
        if isinstance(config, str):
            if config != "auto":
                raise ValueError(f'config must be a dict, None or "auto", got {config!r}')
            config = self.auto_config(self.row_offsets_cpu)
        self.config = dict(config) if config is not None else dict(self.CONFIGS.get(k, self.DEFAULT_CONFIG))
        cfg = self.config
        if cfg.get("k_block") != 32 or cfg.get("vec_len") != 4 or cfg.get("seg_length", 0) <= 0 \
                or cfg["seg_length"] % 32 != 0:
            # the kernels process 32-slot chunks from 4-aligned offsets, as the reference's do
            raise ValueError(f"config must have k_block=32, vec_len=4 and seg_length a positive multiple of 32, got {cfg}")

        self.column_indices = column_indices.to(dtype=torch.int32, device=self.device).contiguous()
        self.values = values.to(dtype=torch.float32, device=self.device).contiguous()
        self.row_offsets = self.row_offsets_cpu.to(device=self.device)
        ro = self.row_offsets_cpu
        self.max_row_length = int((ro[1:] - ro[:-1]).max()) if ro.numel() > 1 else 0
        if locality not in (True, False, "auto"):
            raise ValueError(f'locality must be True, False or "auto", got {locality!r}')
        self.locality = locality
        self._shared = {}  # per-pattern cache (the transposed pattern); with_values() copies share it
        self._preprocess()

    @classmethod
    def auto_config(cls, row_offsets):
        """Segment length picked from the row lengths (the reference hard-codes one per k,
        rode_sddmm.py:35-38).  Measured on MI355X over the five benchmark patterns:

        * a small matrix (fewer than 16384 segments of 512 slots: not enough work items to
          fill the GPU) wants short segments, 128: more wavefronts, and the kernels merge
          what is too short;
        * otherwise a row should be a single segment where that is possible, so that one
          wavefront sums it whole: the power of two that holds 90 % of the rows that have
          block segments, between 512 and 2048 (attention masks: 1024; power-law graphs:
          512 - their hub rows are cut into many segments either way, and the block kernel
          adds the sums of neighbouring segments up before it updates the row of C).
        """
        ro = row_offsets.to(device="cpu")
        if ro.dtype not in (torch.int32, torch.int64):
            ro = ro.to(torch.int64)
        start = ro[:-1]
        aligned = (ro[1:] - start) + (start & 3)
        blocked = aligned >= 32  # rows that have block segments
        rows = int(blocked.sum())
        seg = 512
        if rows > 0:
            segments = int((((aligned + 511) >> 9) * blocked).sum())  # at 512 slots a segment (the sum is 64-bit)
            if segments < 16384:
                seg = 128
            else:
                # the smallest of 512, 1024, 2048 that at least 90 % of those rows do not exceed: the
                # order statistic torch.quantile(..., "higher") returns lies at or below a length
                # exactly when that many rows do (counting avoids quantile's 16 M element limit)
                rank = min(rows, math.ceil(0.9 * (rows - 1)) + 1)
                while seg < 2048 and int((blocked & (aligned <= seg)).sum()) < rank:
                    seg *= 2
        return {"seg_length": seg, "k_block": 32, "vec_len": 4}

    def _preprocess(self):
        """Row decomposition on the GPU; the index arrays never visit the host."""
        cfg = self.config
        blk, st, res, m1, m2 = rode_sddmm_hip.preprocess_device(
            self.row_offsets, self.nnz, cfg["seg_length"], cfg["k_block"], cfg["vec_len"])
        self.block_indices = blk
        self.st_offsets = st
        self.residue_indices = res
        self.m1 = m1
        self.m2 = m2
        # Locality plan: chunks of the residue list whose dense rows cluster in a window that
        # fits LDS (banded matrices) go to the window kernels.  Kept only when it pays:
        # "auto" wants windows on at least half of the chunks and enough of them to fill the
        # GPU twice (a few windowed chunks only add launches); True keeps any plan with a
        # window; False makes none.
        self.plan = (self._group_plan() or self._hub_plan()) if self.locality else None
        if self.plan is None and self.locality and m2 > 0:
            plan = rode_sddmm_hip.window_plan(res, m2, self.row_offsets, self.column_indices, self.n)
            enough = plan.windowed >= max(self.PLAN_MIN_CHUNKS, (plan.counts[0] + 1) // 2)
            if plan.windowed > 0 and (self.locality is True or enough):
                self.plan = rode_sddmm_hip.window_plan_rows(plan, res, m2, self.row_offsets, self.column_indices)

    # A hub plan is made when the rows of at least HUB_MIN_LEN nonzeros (and 8 per 4096
    # columns) hold a tenth of the matrix and the matrix has at least HUB_MIN_SLABS times 4096
    # columns (a smaller dense operand stays in the caches by itself).
    HUB_MIN_LEN = 4096
    HUB_MIN_SLABS = 16
    HUB_MIN_SHARE = 0.1

    # A group plan is kept when at least half of the groups of four rows share a run (or any,
    # with locality=True), and is only looked for in matrices with at least GROUP_MIN_MEAN
    # nonzeros per row (a shared run has at least 64 columns).
    GROUP_MIN_MEAN = 64

    def _group_plan(self):
        """Group plan (adjacent rows that share a long run of consecutive columns are processed
        together, each dense row of the run loaded once for all of them), or None."""
        if self.m < 4 or self.nnz < self.GROUP_MIN_MEAN * self.m:
            return None
        plan = rode_sddmm_hip.group_plan(self.row_offsets, self.column_indices, self.m)
        enough = 2 * plan.counts[1] >= plan.counts[0]
        return plan if plan.usable and (self.locality is True or enough) else None

    def _hub_plan(self):
        """Hub plan (rows with very many nonzeros are processed column slab by column slab so
        that they share the dense rows they fetch), or None when the pattern has no use for it."""
        slabs = (self.n + 4095) // 4096
        if slabs < self.HUB_MIN_SLABS or self.nnz == 0:
            return None
        min_len = max(self.HUB_MIN_LEN, 8 * slabs)
        start = self.row_offsets_cpu[:-1]
        lens = self.row_offsets_cpu[1:] - start
        hub = (lens + (start & 3)) >= min_len  # (aligned length, as the kernels count it)
        hub_nnz = int((lens * hub).sum())  # (summed in 64 bits)
        if self.locality is not True and hub_nnz < self.HUB_MIN_SHARE * self.nnz:
            return None
        if hub_nnz == 0:
            return None
        plan = rode_sddmm_hip.hub_plan(self.row_offsets, self.column_indices, self.m, self.n, int(min_len))
        return plan if plan.usable else None

    def call_plans(self, spmm_width=None, spmm_elem_bytes=4):
        """The ``rode_hip_plans`` struct of this matrix for an SDDMM call (no arguments) or an
        SpMM call of the given dense width and output element size; built once per pattern
        and kind of call (the plan and the segment length never change after construction)."""
        key = ("plans", spmm_width, spmm_elem_bytes)
        plans = self._shared.get(key)
        if plans is None:
            plans = rode_sddmm_hip.plans_struct(self.plan, spmm_width, spmm_elem_bytes, True,
                                                seg_length=self.config["seg_length"])
            self._shared[key] = plans
        return plans

    def spmm_stores_every_row(self):
        """Whether an SpMM on this matrix leaves no row of C to be cleared beforehand: every row
        has slots (rows without any are never written) and a single work item, which then stores
        its row instead of adding to it (``RODE_SPMM_OVERWRITE``).  Worked out once per pattern
        from the row lengths and ``rode_hip_spmm_overwrite_limit``."""
        cached = self._shared.get("spmm_stores_every_row")
        if cached is None:
            cached = False
            if self.m > 0 and self.nnz > 0:
                start = self.row_offsets_cpu[:-1]
                aligned = (self.row_offsets_cpu[1:] - start) + (start & 3)  # slots as the kernels count them
                shortest, longest = int(aligned.min()), int(aligned.max())
                if shortest > 0:
                    plan = self.plan
                    if isinstance(plan, rode_sddmm_hip.GroupPlan) and plan.usable and plan.counts[2] == 0:
                        cached = True  # every row is in a kept group: one wave (or workgroup) owns it
                    else:
                        import ctypes
                        from . import _lib
                        limit = _lib.load().rode_hip_spmm_overwrite_limit(self.m1, ctypes.byref(self.call_plans()))
                        cached = longest < 32 or longest <= limit
            self._shared["spmm_stores_every_row"] = cached
        return cached

    def with_values(self, values):
        """The same pattern and decomposition with other values (no preprocessing is
        repeated): how the output of one op becomes the sparse operand of the next,
        e.g. SDDMM scores -> softmax -> SpMM."""
        if values.shape != self.values.shape:
            raise ValueError(f"values shape must be {tuple(self.values.shape)}, got {tuple(values.shape)}")
        other = object.__new__(RoDeCSR)
        other.__dict__.update(self.__dict__)
        other.values = values if values.dtype == torch.float64 else values.to(torch.float32)
        other.values = other.values.to(self.device).contiguous()
        return other

    def transpose(self, with_values=True):
        """``(csr_t, perm)``: the decomposed pattern of the transposed matrix and the int32
        permutation with ``csr_t.values == self.values[perm]`` (built on the GPU once, then
        cached).  Needed by the gradients with respect to the column-side operands; a caller
        that brings its own values for ``csr_t`` passes ``with_values=False`` and gets the
        cached pattern as it is, without the gather of this instance's values."""
        cached = self._shared.get("transpose")
        if cached is None:
            row_offsets_t, rows_t, perm = rode_sddmm_hip.csr_transpose(self.row_offsets, self.column_indices,
                                                                       self.m, self.n)
            csr_t = RoDeCSR(row_offsets_t, rows_t, self._permuted_values(perm).float(), self.device, self.n, self.m,
                            self.k, config=self.config, locality=self.locality)
            cached = (csr_t, perm)
            self._shared["transpose"] = cached
        csr_t, perm = cached
        if not with_values:
            return csr_t, perm
        return csr_t.with_values(self._permuted_values(perm)), perm

    def transposed_slots(self):
        """int32 vector over the nonzeros: the index of each in the transposed pattern (the
        inverse of the ``perm`` of ``transpose``; made once per pattern)."""
        cached = self._shared.get("transposed_slots")
        if cached is None:
            _, perm = self.transpose(with_values=False)
            cached = torch.empty_like(perm)
            cached[perm.long()] = torch.arange(perm.numel(), dtype=torch.int32, device=perm.device)
            self._shared["transposed_slots"] = cached
        return cached

    def ones(self):
        """A float32 vector of ones over the nonzeros (made once per pattern): the values of an
        SDDMM that samples without weighting."""
        cached = self._shared.get("ones")
        if cached is None:
            cached = torch.ones(self.nnz, dtype=torch.float32, device=self.device)
            self._shared["ones"] = cached
        return cached

    def _permuted_values(self, perm):
        if self.values.dtype == torch.float32:
            return rode_sddmm_hip.permute(self.values.contiguous(), perm)
        return self.values[perm]

    @classmethod
    def from_random(cls, m, n, nnz_per_row, device, k=128):
        """Random pattern with about ``nnz_per_row`` entries per row (duplicates
        removed, rows not padded), N(0,1) values -- rode_sddmm.py:100-144."""
        nnz_raw = m * nnz_per_row
        coords = torch.unique(torch.randint(0, m, (nnz_raw,)) * n + torch.randint(0, n, (nnz_raw,)))
        rows = torch.div(coords, n, rounding_mode="floor")
        cols = coords % n
        vals = torch.randn(coords.numel(), dtype=torch.float32)
        row_offsets = torch.zeros(m + 1, dtype=torch.int64)
        row_offsets[1:] = torch.cumsum(torch.bincount(rows, minlength=m), 0)
        return cls(row_offsets.to(torch.int32), cols.to(torch.int32), vals, device, m, n, k)

    def to_torch_sparse_csr(self):
        """``torch.sparse_csr`` copy without the explicit zeros that pad rows in the
        reference's C++ generators (rode_sddmm.py:146-185)."""
        keep = (self.values != 0).cpu()
        ro = self.row_offsets_cpu.to(torch.int64)
        rows = torch.repeat_interleave(torch.arange(self.m), ro[1:] - ro[:-1])
        crow = torch.zeros(self.m + 1, dtype=torch.int64)
        crow[1:] = torch.cumsum(torch.bincount(rows[keep], minlength=self.m), 0)
        return torch.sparse_csr_tensor(
            crow,
            self.column_indices.cpu()[keep].to(torch.int64),
            self.values.cpu()[keep],
            size=(self.m, self.n),
            device=self.device,
        )

    def __repr__(self):
        return (f"RoDeCSR(m={self.m}, n={self.n}, nnz={self.nnz}, k={self.k}, "
                f"m1={self.m1}, m2={self.m2}, device={self.device})")


def rode_sddmm(sparse_matrix, lhs, rhs, values=None):
    """out = S (.) (lhs @ rhs^T) sampled at the nonzeros of S; returns the (nnz,)
    values in CSR order.  lhs is (m, k), rhs is (n, k); float32, or float16 with
    fp32 accumulation.  ``values`` (optional) replaces the values of S for this call.
    Differentiable with respect to lhs, rhs and values (the reference op is
    forward-only)."""
    m, n, k = sparse_matrix.m, sparse_matrix.n, sparse_matrix.k
    if tuple(lhs.shape) != (m, k):
        raise ValueError(f"lhs_matrix shape must be ({m}, {k}), got {tuple(lhs.shape)}")
    if tuple(rhs.shape) != (n, k):
        raise ValueError(f"rhs_matrix shape must be ({n}, {k}), got {tuple(rhs.shape)}")
    assert lhs.is_cuda and lhs.device == sparse_matrix.device, f"lhs must be on {sparse_matrix.device}, got {lhs.device}"
    assert rhs.is_cuda and rhs.device == sparse_matrix.device, f"rhs must be on {sparse_matrix.device}, got {rhs.device}"
    assert lhs.dtype in (torch.float32, torch.float16), f"lhs must be float32 or float16, got {lhs.dtype}"
    assert rhs.dtype == lhs.dtype, f"rhs must be {lhs.dtype}, got {rhs.dtype}"
    vals = sparse_matrix.values if values is None else values
    if torch.is_grad_enabled() and (lhs.requires_grad or rhs.requires_grad or vals.requires_grad):
        from .autograd import SddmmFunction
        return SddmmFunction.apply(sparse_matrix, vals, lhs, rhs)
    if values is not None:
        sparse_matrix = sparse_matrix.with_values(values)
    return rode_sddmm_hip.sddmm_forward(
        sparse_matrix.block_indices, sparse_matrix.residue_indices, sparse_matrix.st_offsets,
        sparse_matrix.m1, sparse_matrix.m2, sparse_matrix.row_offsets, sparse_matrix.column_indices,
        sparse_matrix.values, m, n, lhs.contiguous(), rhs.contiguous(), k, plan=sparse_matrix.plan,
        seg_length=sparse_matrix.config["seg_length"], checked_lists=True, plans=sparse_matrix.call_plans())


def torch_sddmm_reference(sparse_csr, lhs_matrix, rhs_matrix):
    """Library oracle used by the reference's tests: ``sampled_addmm`` with beta 0
    samples lhs @ rhs^T on the pattern, then the pattern's values are multiplied
    in (rode_sddmm.py:285-304)."""
    sampled = torch.sparse.sampled_addmm(sparse_csr, lhs_matrix, rhs_matrix.T, beta=0.0, alpha=1.0)
    return torch.sparse_csr_tensor(
        sampled.crow_indices(), sampled.col_indices(), sampled.values() * sparse_csr.values(),
        size=sampled.shape, device=sampled.device, dtype=sampled.dtype)


def compare_results(rode_output, torch_sparse_output, rode_csr, tolerance=1e-3):
    """Error statistics of a RoDe output against a sparse-CSR oracle; an entry is
    an error when both its absolute and its relative difference exceed
    ``tolerance`` (rode_sddmm.py:357-368).  Entries whose pattern value is exactly
    0 are padding and are skipped (:333-339)."""
    keep = (rode_csr.values != 0).cpu()
    got = rode_output.detach().cpu().to(torch.float32)[keep]
    ref = torch_sparse_output.values().detach().cpu().to(torch.float32)
    if got.numel() != ref.numel():
        inf = float("inf")
        return {"passed": False, "error": f"Size mismatch: RoDe={got.numel()}, Torch={ref.numel()}",
                "mae": inf, "mean_rel": inf, "max_abs": inf, "max_rel": inf,
                "error_count": -1, "total_count": got.numel()}
    if got.numel() == 0:
        return {"passed": True, "mae": 0.0, "mean_rel": 0.0, "max_abs": 0.0, "max_rel": 0.0,
                "error_count": 0, "total_count": 0}
    diff = (got - ref).abs()
    rel = diff / (ref.abs() + 1e-8)
    errors = int(((diff > tolerance) & (rel > tolerance)).sum())
    return {"passed": errors == 0, "mae": diff.mean().item(), "mean_rel": rel.mean().item(),
            "max_abs": diff.max().item(), "max_rel": rel.max().item(),
            "error_count": errors, "total_count": got.numel()}
