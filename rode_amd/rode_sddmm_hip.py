"""Tensor-level entry points, mirroring the reference's compiled torch module
``rode_sddmm_cuda`` (``RoDe_SDDMM/rode_sddmm_cuda.cu:254-278``): ``preprocess``
and ``sddmm_forward`` keep their argument names, order and error behaviour
(``RuntimeError`` where the reference's ``TORCH_CHECK`` throws).  PyTorch is used
for device memory and the current stream only; all work is done by
``librode_hip.so`` through its C ABI.

Additions with no counterpart in the reference module: ``preprocess_device``
(decomposition of a row pointer that already lives on the GPU, results stay on
the GPU) and ``spmm_forward``.
"""
import ctypes

import torch

from . import _lib

_VEC = {torch.float32: 4, torch.float16: 8, torch.float64: 2}  # elements per 128-bit load
_MAX_K = 512


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _check_input(x, name):
    _check(x.device.type == "cuda", f"{name} must be a CUDA tensor")
    _check(x.is_contiguous(), f"{name} must be contiguous")


def _stream_handle(device):
    """Raw handle of PyTorch's current stream on ``device`` (the direct lookup costs a
    fraction of a microsecond; building a ``torch.cuda.Stream`` object costs several)."""
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None and device.index is not None:
        return raw(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(device):
    """Context in which ``device`` is the current GPU; nothing to enter or leave when it
    already is (the usual case, and the switch costs microseconds per call)."""
    if device.index is None or torch.cuda.current_device() == device.index:
        return _NO_SWITCH
    return torch.cuda.device(device)


def preprocess_capacity(m, nnz, seg_length, vec_len):
    """Upper bound on the number of block segments (each row's aligned length is
    at most len + vec_len - 1, and it yields at most aligned/seg + 1 segments)."""
    return (nnz + (vec_len - 1) * m) // seg_length + m


def preprocess_device(row_offsets, nnz, seg_length, k_block, vec_len):
    """Row decomposition of a device-resident int32 row pointer.

    Returns ``(block_indices, st_offsets, residue_indices, n_blk, n_res)`` with
    the tensor sizes of the reference (``rode_sddmm_cuda.cu:115-117``):
    ``block_indices[max(n_blk,1)]``, ``st_offsets[n_blk+1]``,
    ``residue_indices[max(n_res,1)]``, all on ``row_offsets.device``.
    """
    _check_input(row_offsets, "row_offsets")
    _check(row_offsets.dtype == torch.int32, "row_offsets must be int32")
    _check(row_offsets.dim() == 1 and row_offsets.numel() >= 1, "row_offsets must hold m+1 entries")
    _check(seg_length > 0 and k_block > 0 and vec_len > 0, "seg_length, k_block and vec_len must be positive")
    lib = _lib.load()
    dev = row_offsets.device
    m = row_offsets.numel() - 1
    cap = preprocess_capacity(m, int(nnz), seg_length, vec_len)
    with torch.cuda.device(dev):
        blk = torch.empty(cap + 1, dtype=torch.int32, device=dev)
        st = torch.empty(cap + 2, dtype=torch.int32, device=dev)
        res = torch.empty(max(m, 1), dtype=torch.int32, device=dev)
        counts = torch.empty(2, dtype=torch.int32, device=dev)
        ws_bytes = lib.rode_hip_preprocess_workspace_bytes(m)
        ws = torch.empty((ws_bytes + 7) // 8, dtype=torch.int64, device=dev)
        code = lib.rode_hip_preprocess(seg_length, k_block, vec_len, m, row_offsets.data_ptr(), blk.data_ptr(),
                                       st.data_ptr(), res.data_ptr(), counts.data_ptr(),
                                       counts.data_ptr() + 4, cap, ws.data_ptr(), ws_bytes, _stream_handle(dev))
        _lib.check(code, "rode_hip_preprocess")
        n_blk, n_res = (int(v) for v in counts.cpu())  # stream-ordered copy: waits for the kernels
    _check(n_blk <= cap and n_res <= max(m, 1), "row decomposition larger than its capacity bound")
    # copies, so that the capacity-sized buffers are released
    return blk[: max(n_blk, 1)].clone(), st[: n_blk + 1].clone(), res[: max(n_res, 1)].clone(), n_blk, n_res


class WindowPlan:
    """Locality plan of one decomposition (``rode_hip_window_plan``): the device array and
    a host copy of its header ``[residue chunks, residue chunks with a window, 0, 0]``."""

    def __init__(self, data, counts, rows=None):
        self.data = data                                       # descriptors (device int32)
        self.rows = rows                                       # planned rows of the chunks with a window (device bytes)
        self.counts = counts                                   # list of 4 ints
        self._header = (ctypes.c_int * 4)(*counts)             # what the C ABI reads

    @property
    def windowed(self):
        return self.counts[1]

    def descriptors(self):
        """int32 array of shape (residue chunks, 4): first window row, window rows (0: none),
        nonzeros, nonzeros outside the window."""
        return self.data.cpu().numpy()[4:].reshape(-1, 4)


def window_plan(residue_indices, m2, row_offsets, column_indices, dense_rows):
    """Locality plan for the residue list of one decomposition: which chunks of 128 residue
    rows have their dense rows inside a window small enough for LDS.  ``dense_rows``: number
    of columns of the sparse matrix.  Waits for the two small kernels (it returns the chunk
    counts)."""
    for t, name in ((residue_indices, "residue_indices"), (row_offsets, "row_offsets"),
                    (column_indices, "column_indices")):
        _check_input(t, name)
        _check(t.dtype == torch.int32, f"{name} must be int32")
    lib = _lib.load()
    dev = row_offsets.device
    nbytes = lib.rode_hip_window_plan_bytes(m2)
    with torch.cuda.device(dev):
        data = torch.empty(nbytes // 4, dtype=torch.int32, device=dev)
        counts = (ctypes.c_int * 4)()
        code = lib.rode_hip_window_plan(m2, dense_rows, residue_indices.data_ptr(), row_offsets.data_ptr(),
                                        column_indices.data_ptr(), data.data_ptr(), nbytes, ctypes.addressof(counts),
                                        _stream_handle(dev))
        _lib.check(code, "rode_hip_window_plan")
    return WindowPlan(data, list(counts))


def window_plan_rows(plan, residue_indices, m2, row_offsets, column_indices):
    """Second part of a plan (``rode_hip_window_rows``): for every residue row of a chunk
    with a window, where in the window its nonzeros are.  10 KiB per 128 residue rows; made
    only for a plan that is going to be used."""
    lib = _lib.load()
    dev = row_offsets.device
    with torch.cuda.device(dev):
        rbytes = lib.rode_hip_window_rows_bytes(m2)
        plan.rows = torch.empty(rbytes // 16, 4, dtype=torch.int32, device=dev)
        code = lib.rode_hip_window_rows(m2, residue_indices.data_ptr(), row_offsets.data_ptr(),
                                        column_indices.data_ptr(), plan.data.data_ptr(), plan.rows.data_ptr(), rbytes,
                                        _stream_handle(dev))
    _lib.check(code, "rode_hip_window_rows")
    return plan


def csr_transpose(row_offsets, column_indices, m, n):
    """``(row_offsets_t, column_indices_t, perm)`` of the transposed pattern, all int32 on
    the device of the inputs: nonzero j of the transposed matrix is nonzero ``perm[j]`` of
    the input (ordered by column, then by index), its column is that nonzero's row."""
    for t, name in ((row_offsets, "row_offsets"), (column_indices, "column_indices")):
        _check_input(t, name)
        _check(t.dtype == torch.int32, f"{name} must be int32")
    _check(row_offsets.numel() == m + 1, "row_offsets must have m + 1 entries")
    nnz = column_indices.numel()
    lib = _lib.load()
    dev = row_offsets.device
    row_offsets_t = torch.empty(n + 1, dtype=torch.int32, device=dev)
    column_indices_t = torch.empty(nnz, dtype=torch.int32, device=dev)
    perm = torch.empty(nnz, dtype=torch.int32, device=dev)
    ws_bytes = lib.rode_hip_csr_transpose_workspace_bytes(nnz)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(lib.rode_hip_csr_transpose(m, n, nnz, row_offsets.data_ptr(), column_indices.data_ptr(),
                                              row_offsets_t.data_ptr(), column_indices_t.data_ptr(), perm.data_ptr(),
                                              ws.data_ptr(), ws_bytes, _stream_handle(dev)), "rode_hip_csr_transpose")
    return row_offsets_t, column_indices_t, perm


def permute(values, perm):
    """``values[perm]`` for a float32 vector and the int32 ``perm`` of ``csr_transpose``: the
    values of the transposed pattern (``rode_hip_permute_f32``)."""
    _check_input(values, "values")
    _check_input(perm, "perm")
    _check(values.dtype == torch.float32 and perm.dtype == torch.int32, "values must be float32 and perm int32")
    _check(values.dim() == 1 and perm.dim() == 1 and values.device == perm.device, "values and perm must be vectors on one device")
    out = torch.empty(perm.numel(), dtype=torch.float32, device=values.device)
    with torch.cuda.device(values.device):
        _lib.check(_lib.load().rode_hip_permute_f32(perm.numel(), values.data_ptr(), perm.data_ptr(), out.data_ptr(),
                                                     _stream_handle(values.device)), "rode_hip_permute_f32")
    return out


class HubPlan:
    """Hub plan of one pattern (``rode_hip_hub_plan``): the device array and a host copy
    of its header ``[hub rows, slabs, min_len, usable, room, 0, 0, 0]``."""

    def __init__(self, data, counts):
        self.data = data
        self.counts = counts
        self._header = (ctypes.c_int * 8)(*counts)
        self.rows = None  # (a matrix has a hub plan or a locality plan, never both)
        self._workspaces = {}

    def workspace(self, n, elem_bytes):
        """Scratch for the SpMM hub kernels at dense width ``n`` (one partial row of C per
        hub row and slab); kept for the next call.  Calls that overlap in time on different
        streams must not share it."""
        key = (n, elem_bytes)
        if key not in self._workspaces:
            nbytes = _lib.load().rode_hip_hub_workspace_bytes(ctypes.addressof(self._header), n, elem_bytes)
            self._workspaces[key] = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=self.data.device)
        return self._workspaces[key]

    @property
    def usable(self):
        return self.counts[3] != 0 and self.counts[0] > 0

    def hub_rows(self):
        return self.data[8:8 + self.counts[0]].cpu().numpy()

    def pieces(self):
        """int32 array (hub rows, slabs + 1): where every hub row's nonzeros of each column slab start."""
        first = 8 + self.counts[4]
        return self.data[first:first + self.counts[0] * (self.counts[1] + 1)].cpu().numpy().reshape(self.counts[0], -1)


def hub_plan(row_offsets, column_indices, m, n, min_len):
    """Hub plan: the rows of at least ``min_len`` aligned nonzero slots, cut into pieces by
    slab of 2048 columns.  Waits for its two kernels (it returns the counts)."""
    for t, name in ((row_offsets, "row_offsets"), (column_indices, "column_indices")):
        _check_input(t, name)
        _check(t.dtype == torch.int32, f"{name} must be int32")
    lib = _lib.load()
    dev = row_offsets.device
    nnz = column_indices.numel()
    nbytes = lib.rode_hip_hub_plan_bytes(m, n, nnz, min_len)
    _check(nbytes > 0, "min_len is too small for a hub plan")
    with torch.cuda.device(dev):
        data = torch.empty(nbytes // 4, dtype=torch.int32, device=dev)
        counts = (ctypes.c_int * 8)()
        _lib.check(lib.rode_hip_hub_plan(m, n, nnz, min_len, row_offsets.data_ptr(), column_indices.data_ptr(),
                                         data.data_ptr(), nbytes, ctypes.addressof(counts), _stream_handle(dev)),
                   "rode_hip_hub_plan")
    counts = list(counts)
    hub_rows, slabs, room = counts[0], counts[1], counts[4]
    if counts[3] != 0 and 0 < hub_rows < room:
        # the call needs room for the most hub rows a matrix of this many nonzeros can have; what it
        # found is kept in an array of its own size (header, the rows, their pieces)
        small = torch.empty(8 + hub_rows + hub_rows * (slabs + 1), dtype=torch.int32, device=dev)
        small[:8] = data[:8]
        small[4] = hub_rows
        small[8:8 + hub_rows] = data[8:8 + hub_rows]
        small[8 + hub_rows:] = data[8 + room:8 + room + hub_rows * (slabs + 1)]
        data, counts[4] = small, hub_rows
    return HubPlan(data, counts)


class GroupPlan:
    """Group plan of one pattern (``rode_hip_group_plan``): the device array and a host copy
    of its header ``[groups, groups with a shared run, rows outside those groups, 0]``."""

    def __init__(self, data, counts):
        self.data = data
        self.counts = counts
        self._header = (ctypes.c_int * 4)(*counts)
        self.rows = None  # (a matrix has one kind of plan)

    @property
    def usable(self):
        return self.counts[1] > 0

    def groups(self):
        """int32 array (groups, 8): first column and length of the range the four rows' runs
        cover (0: group not kept), the position of its own run in each row, and per row, a byte
        each, how many columns of the range lie before and after its run."""
        return self.data[4:4 + 8 * self.counts[0]].cpu().numpy().reshape(-1, 8)


def group_plan(row_offsets, column_indices, m):
    """Group plan: which groups of four adjacent rows share a long run of consecutive
    columns.  Waits for its kernels (it returns the counts)."""
    for t, name in ((row_offsets, "row_offsets"), (column_indices, "column_indices")):
        _check_input(t, name)
        _check(t.dtype == torch.int32, f"{name} must be int32")
    lib = _lib.load()
    dev = row_offsets.device
    nbytes = lib.rode_hip_group_plan_bytes(m)
    with torch.cuda.device(dev):
        data = torch.empty(nbytes // 4, dtype=torch.int32, device=dev)
        counts = (ctypes.c_int * 4)()
        _lib.check(lib.rode_hip_group_plan(m, row_offsets.data_ptr(), column_indices.data_ptr(), data.data_ptr(), nbytes,
                                           ctypes.addressof(counts), _stream_handle(dev)), "rode_hip_group_plan")
    return GroupPlan(data, list(counts))


def plans_struct(plan, spmm_width=None, spmm_elem_bytes=4, whole_lists=True, seg_length=0):
    """The ``rode_hip_plans`` struct of one call (keep it alive until the call returns; pass
    it with ``ctypes.byref``).  ``plan``: a ``WindowPlan``, a ``HubPlan``, a ``GroupPlan`` or None.
    ``spmm_width``: for an SpMM call the dense width, so that a hub plan's workspace is
    attached; a hub plan is left out of an SpMM call without the whole-lists promise.
    ``seg_length``: the segment length the lists were made with, 0 when not known."""
    p = _lib.Plans()
    p.seg_length = int(seg_length or 0)  # (the segment length of the decomposition, when the caller knows it)
    if isinstance(plan, GroupPlan):
        if plan.usable and (spmm_width is None or whole_lists):
            p.groups, p.group_counts = plan.data.data_ptr(), ctypes.addressof(plan._header)
    elif isinstance(plan, HubPlan):
        if plan.usable and (spmm_width is None or whole_lists):
            p.hub, p.hub_counts = plan.data.data_ptr(), ctypes.addressof(plan._header)
            if spmm_width is not None:
                ws = plan.workspace(spmm_width, spmm_elem_bytes)
                p.hub_workspace, p.hub_workspace_bytes = ws.data_ptr(), ws.numel()
    elif plan is not None and plan.rows is not None:
        p.window, p.window_rows = plan.data.data_ptr(), plan.rows.data_ptr()
        p.window_counts = ctypes.addressof(plan._header)
    return p


def preprocess(row_offsets, nnz, seg_length, k_block, vec_len):
    """``rode_sddmm_cuda.preprocess`` (``rode_sddmm_cuda.cu:54-131``): takes the CPU
    int32 row pointer and returns CPU tensors, as the reference does; the
    decomposition itself runs on the current GPU."""
    _check(row_offsets.device.type == "cpu", "row_offsets must be on CPU for preprocessing")
    _check(row_offsets.dtype == torch.int32, "row_offsets must be int32")
    _lib.load()
    dev = torch.device("cuda", torch.cuda.current_device())
    blk, st, res, n_blk, n_res = preprocess_device(row_offsets.contiguous().to(dev), nnz, seg_length, k_block, vec_len)
    return blk.cpu(), st.cpu(), res.cpu(), n_blk, n_res


def _dense_kind(lhs_matrix, rhs_matrix, lhs_name, rhs_name):
    if lhs_matrix.dtype == torch.float16 and rhs_matrix.dtype == torch.float16:
        return "f16"
    _check(lhs_matrix.dtype == torch.float32, f"{lhs_name} must be float32")
    _check(rhs_matrix.dtype == torch.float32, f"{rhs_name} must be float32")
    return "f32"


def sddmm_forward(block_indices, residue_indices, st_offsets, m1, m2, row_offsets, column_indices, values, m, n,
                  lhs_matrix, rhs_matrix, k_version, plan=None, seg_length=0, checked_lists=False, plans=None):
    """``rode_sddmm_cuda.sddmm_forward`` (``rode_sddmm_cuda.cu:136-249``).

    Differences from the reference, none of which changes a result: any k_version
    that is a multiple of 4 up to 512 (multiple of 8 for fp16) and fp16
    ``lhs_matrix``/``rhs_matrix`` (fp32 accumulate) are accepted too; the
    kernels are queued on PyTorch's current stream instead of two streams that
    are created, synchronised and destroyed per call (``:203-246``).  ``plan``: a
    plan made from these very lists, or None; ``seg_length``: the segment length the lists were
    made with (``preprocess``'s third argument), 0 when not known.  ``checked_lists``: the
    index tensors and values are a ``RoDeCSR``'s own (device, layout and type were settled
    when it was built); ``plans``: the ``plans_struct`` of (plan, seg_length), kept by the caller.
    """
    if not checked_lists:
        for t, name in ((block_indices, "block_indices"), (residue_indices, "residue_indices"),
                        (st_offsets, "st_offsets"), (row_offsets, "row_offsets"), (column_indices, "column_indices"),
                        (values, "values")):
            _check_input(t, name)
        for t, name in ((block_indices, "block_indices"), (residue_indices, "residue_indices"),
                        (st_offsets, "st_offsets"), (row_offsets, "row_offsets"), (column_indices, "column_indices")):
            _check(t.dtype == torch.int32, f"{name} must be int32")
        _check(values.dtype == torch.float32, "values must be float32")
    _check_input(lhs_matrix, "lhs_matrix")
    _check_input(rhs_matrix, "rhs_matrix")
    kind = _dense_kind(lhs_matrix, rhs_matrix, "lhs_matrix", "rhs_matrix")

    k = lhs_matrix.size(1)
    nnz = values.size(0)
    vec = _VEC[lhs_matrix.dtype]
    _check(0 < k_version <= _MAX_K and k_version % vec == 0,
           f"k_version must be a positive multiple of {vec} up to {_MAX_K} (the reference has 32 and 128)")
    _check(k == k_version, "k dimension must match k_version")
    _check(lhs_matrix.size(0) == m, "lhs_matrix rows must equal m")
    _check(rhs_matrix.size(0) == n, "rhs_matrix rows must equal n")
    _check(rhs_matrix.size(1) == k, "rhs_matrix cols must equal k")

    if m1 == 0 and m2 == 0:
        return torch.zeros(nnz, dtype=torch.float32, device=values.device)
    # (every nonzero is in exactly one work item and every work item stores its outputs: nothing to clear)
    out = torch.empty(nnz, dtype=torch.float32, device=values.device)
    lib = _lib.load()
    with _on_device(values.device):
        s = _stream_handle(values.device)
        if plans is None:
            plans = plans_struct(plan, seg_length=seg_length)
        code = lib.rode_hip_sddmm_planned(_lib.DENSE_CODE[kind], 0, m1, m2, n, k, block_indices.data_ptr(),
                                          residue_indices.data_ptr(), st_offsets.data_ptr(), row_offsets.data_ptr(),
                                          column_indices.data_ptr(), values.data_ptr(), lhs_matrix.data_ptr(),
                                          rhs_matrix.data_ptr(), out.data_ptr(), ctypes.byref(plans), s, s)
    _lib.check(code, "rode_hip_sddmm_planned")
    return out


def spmm_forward(block_indices, residue_indices, st_offsets, m1, m2, row_offsets, column_indices, values, m, k,
                 dense_matrix, out=None, whole_lists=True, plan=None, seg_length=0, checked_lists=False, plans=None,
                 every_row_stored=False):
    """C = A_csr @ dense_matrix through ``rode_hip_spmm_f32`` / ``_f16``
    (host API ``RoDe_SpMM/RoDeSpmm.h:4-8``).  ``dense_matrix`` is (k, n) with n a
    multiple of 4 (8 for fp16, 2 for fp64), fp32 / fp16 (fp32 ``values``) or fp64 (fp64 ``values``); the
    result is a new zero-initialised (m, n) tensor of the dtype of ``values``, or
    ``out`` accumulated in place the way the reference kernels do (long rows add,
    short rows overwrite).  ``whole_lists`` promises that the index tensors are the
    complete decomposition (always true for a ``RoDeCSR``); pass False for a slice.
    ``plan``: a ``WindowPlan`` made from these very lists, a ``HubPlan`` of this pattern
    (used only with ``whole_lists``), or None.  ``checked_lists`` / ``plans``: as for
    ``sddmm_forward`` (``plans``: of (plan, this width and element size, whole_lists, seg_length)).
    ``every_row_stored``: with ``out`` None and ``whole_lists``, the caller has checked
    (``rode_hip_spmm_overwrite_limit``) that every row of the matrix has slots and a single
    work item: the kernels then store their rows (``RODE_SPMM_OVERWRITE``) and nothing is cleared."""
    if not checked_lists:
        for t, name in ((block_indices, "block_indices"), (residue_indices, "residue_indices"),
                        (st_offsets, "st_offsets"), (row_offsets, "row_offsets"), (column_indices, "column_indices"),
                        (values, "values")):
            _check_input(t, name)
        for t, name in ((block_indices, "block_indices"), (residue_indices, "residue_indices"),
                        (st_offsets, "st_offsets"), (row_offsets, "row_offsets"), (column_indices, "column_indices")):
            _check(t.dtype == torch.int32, f"{name} must be int32")
    _check_input(dense_matrix, "dense_matrix")
    if dense_matrix.dtype == torch.float64:
        _check(values.dtype == torch.float64, "values must be float64 when dense_matrix is float64")
    else:
        _check(values.dtype == torch.float32, "values must be float32")
        _check(dense_matrix.dtype in (torch.float32, torch.float16),
               "dense_matrix must be float32, float16 or float64")
    out_dtype = values.dtype
    _check(dense_matrix.dim() == 2 and dense_matrix.size(0) == k, "dense_matrix rows must equal k")
    n = dense_matrix.size(1)
    vec = _VEC[dense_matrix.dtype]
    _check(n > 0 and n % vec == 0, f"dense_matrix cols must be a positive multiple of {vec}")
    lib = _lib.load()
    if out is None:
        if m1 == 0 and m2 == 0:
            return torch.zeros((m, n), dtype=out_dtype, device=values.device)
        # only the rows the kernels add to (or skip) need clearing, the others are overwritten
        out = torch.empty((m, n), dtype=out_dtype, device=values.device)
        every_row_stored = every_row_stored and whole_lists
        with _on_device(values.device):
            if not every_row_stored:
                _lib.check(lib.rode_hip_spmm_clear_rows(m, n, out.element_size(), row_offsets.data_ptr(), out.data_ptr(),
                                                        _stream_handle(values.device)), "rode_hip_spmm_clear_rows")
    else:
        every_row_stored = False  # (the caller's C is added to, as the kernels' contract says)
        _check_input(out, "out")
        _check(out.dtype == out_dtype and tuple(out.shape) == (m, n), f"out must be {out_dtype} of shape (m, n)")
    if m1 == 0 and m2 == 0:
        return out
    dtype = {torch.float32: 0, torch.float16: 1, torch.float64: 2}[dense_matrix.dtype]  # RODE_DENSE_*
    with _on_device(values.device):
        s = _stream_handle(values.device)
        if plans is None:
            plans = plans_struct(plan, n, out.element_size(), whole_lists, seg_length=seg_length)
        flags = (_lib.SPMM_WHOLE_LISTS if whole_lists else 0) | (_lib.SPMM_OVERWRITE if every_row_stored else 0)
        code = lib.rode_hip_spmm_planned(dtype, flags, m1, m2, k, n,
                                         values.data_ptr(), column_indices.data_ptr(), row_offsets.data_ptr(),
                                         block_indices.data_ptr(), residue_indices.data_ptr(), st_offsets.data_ptr(),
                                         dense_matrix.data_ptr(), out.data_ptr(), ctypes.byref(plans), s, s)
    _lib.check(code, "rode_hip_spmm_planned")
    return out
