"""ctypes view of the device library's C ABI (include/compressgnn_abi.h).

torch tensors supply device memory and the current stream; every computation goes
through libcgnn_hip.so.  There is no fallback: if the library is missing or a call
fails, an exception is raised.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcgnn_hip.so")

F32, F64 = 0, 1
SPMM_AUTO, SPMM_ROW, SPMM_NNZ = 0, 1, 2

EXPORTS = [
    "cgnn_last_error", "cgnn_version",
    "cgnn_spmm_schedule", "cgnn_spmm_run_length", "cgnn_spmm_run_starts", "cgnn_spmm_workspace_bytes", "cgnn_spmm", "cgnn_spmm_dual",
    "cgnn_spmm_static_scratch_bytes", "cgnn_spmm_static_init", "cgnn_spmm_static",
    "cgnn_csr_prepare_i64", "cgnn_csr_expand_rows", "cgnn_narrow_ids", "cgnn_csr_compose_columns",
    "cgnn_csr_transpose_workspace_bytes", "cgnn_csr_transpose_device",
    "cgnn_compress_batch_workspace_bytes", "cgnn_compress_csr_batch_device",
    "cgnn_lsh_scan_workspace_bytes", "cgnn_lsh_hash", "cgnn_lsh_scan", "cgnn_lsh_finish",
    "cgnn_lsh_group_workspace_bytes", "cgnn_lsh_group",
    "cgnn_cluster_members_workspace_bytes", "cgnn_cluster_members",
    "cgnn_cluster_mean_workspace_bytes", "cgnn_cluster_mean", "cgnn_cluster_mean_backward",
    "cgnn_reconstruct", "cgnn_reconstruct_backward", "cgnn_sign_words", "cgnn_reconstruct_signs",
    "cgnn_reconstruct_backward_signs", "cgnn_copy_bytes", "cgnn_read_bytes", "cgnn_fill_bytes",
    "cgnn_exclusive_sum_workspace_bytes", "cgnn_exclusive_sum_i32", "cgnn_sample_count", "cgnn_sample_fill",
    "cgnn_sample_relabel_begin", "cgnn_sample_relabel_workspace_bytes", "cgnn_sample_relabel",
]


class CsrStruct(ctypes.Structure):
    _fields_ = [
        ("rows", ctypes.c_int64), ("cols", ctypes.c_int64), ("nnz", ctypes.c_int64),
        ("rowptr", ctypes.c_void_p), ("colidx", ctypes.c_void_p), ("rowidx", ctypes.c_void_p),
        ("val", ctypes.c_void_p), ("max_row_nnz", ctypes.c_int32), ("seg_nnz", ctypes.c_int32),
        ("rowmap", ctypes.c_void_p),
        ("cut_rows", ctypes.c_void_p), ("empty_rows", ctypes.c_void_p),
        ("n_cut_rows", ctypes.c_int32), ("n_empty_rows", ctypes.c_int32),
        ("run_start", ctypes.c_void_p),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libcgnn_hip.so is not built (%s); run `python -m compressgnn_amd.build hip`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.cgnn_last_error.restype = ctypes.c_char_p
        L.cgnn_version.restype = ctypes.c_char_p
        for name in ("cgnn_spmm_workspace_bytes", "cgnn_spmm_static_scratch_bytes", "cgnn_lsh_scan_workspace_bytes", "cgnn_lsh_group_workspace_bytes",
                     "cgnn_cluster_members_workspace_bytes", "cgnn_cluster_mean_workspace_bytes",
                     "cgnn_csr_transpose_workspace_bytes", "cgnn_compress_batch_workspace_bytes",
                     "cgnn_exclusive_sum_workspace_bytes", "cgnn_sample_relabel_workspace_bytes"):
            getattr(L, name).restype = ctypes.c_size_t
        _lib = L
    return _lib


class CgnnError(RuntimeError):
    pass


def check(rc):
    if rc != 0:
        raise CgnnError("cgnn error %d: %s" % (rc, lib().cgnn_last_error().decode()))


def dtype_code(dtype):
    if dtype == torch.float32:
        return F32
    if dtype == torch.float64:
        return F64
    raise TypeError("only float32 and float64 are supported, got %s" % dtype)


def ptr(t):
    return ctypes.c_void_p(0 if t is None or t.numel() == 0 and t.data_ptr() == 0 else t.data_ptr())


def stream_of(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def i64(x):
    return ctypes.c_int64(int(x))


class DeviceCsr:
    """A CSR block on the device with int32 indices (the layout the kernels read)."""

    def __init__(self, rows, cols, rowptr, colidx, val, rowidx=None, max_row_nnz=0, seg_nnz=0, rowmap=None):
        self.rows, self.cols = int(rows), int(cols)
        self.rowptr, self.colidx, self.val, self.rowidx = rowptr, colidx, val, rowidx
        self.rowmap = rowmap  # int32 [rows] on the device: stored row g is row rowmap[g] of the output
        self.nnz = int(colidx.numel())
        self.max_row_nnz, self.seg_nnz = int(max_row_nnz), int(seg_nnz)
        self.run_start = None  # int32 on the device, see make_run_starts
        self._ws = {}

    @classmethod
    def from_host(cls, rows, cols, rowptr, colidx, val, device, with_rowidx=True, seg_nnz=0, rowmap=None):
        """rowptr/colidx: integer arrays or tensors on the host; val: float tensor/array or None;
        rowmap: the rows are given in a stored order, stored row g being output row rowmap[g]."""
        rp = torch.as_tensor(rowptr).to(torch.int64)
        ci = torch.as_tensor(colidx).to(torch.int64)
        lens = rp[1:] - rp[:-1]
        max_row = int(lens.max()) if lens.numel() else 0
        rowidx = None
        if with_rowidx:
            rowidx = torch.repeat_interleave(torch.arange(rows, dtype=torch.int32), lens).to(device)
        v = None if val is None else torch.as_tensor(val).to(device)
        rm = None if rowmap is None else torch.as_tensor(rowmap).to(torch.int32).to(device)
        return cls(rows, cols, rp.to(torch.int32).to(device), ci.to(torch.int32).to(device), v, rowidx,
                   max_row, seg_nnz, rm)

    def struct(self):
        s = CsrStruct()
        s.rows, s.cols, s.nnz = self.rows, self.cols, self.nnz
        s.rowptr = self.rowptr.data_ptr()
        s.colidx = self.colidx.data_ptr() if self.nnz else 0
        s.rowidx = self.rowidx.data_ptr() if (self.rowidx is not None and self.nnz) else 0
        s.val = self.val.data_ptr() if (self.val is not None and self.nnz) else 0
        s.max_row_nnz, s.seg_nnz = self.max_row_nnz, self.seg_nnz
        s.rowmap = self.rowmap.data_ptr() if self.rowmap is not None else 0
        s.run_start = self.run_start.data_ptr() if self.run_start is not None else 0
        return s

    def make_run_starts(self):
        """Builds the optional table of run starts through cgnn_spmm_run_starts (the block needs
        rowidx); the products that follow read it."""
        self.run_start = None
        s = self.struct()
        runs = lib().cgnn_spmm_run_length(ctypes.byref(s))
        table = torch.empty((self.nnz + runs - 1) // runs + 1, dtype=torch.int32, device=self.rowptr.device)
        check(lib().cgnn_spmm_run_starts(ctypes.byref(s), ptr(table), stream_of(table)))
        self.run_start = table
        return table

    def workspace(self, F, dtype, kernel):
        """Scratch for one (F, dtype, kernel), cached on the block (per stream use is the
        caller's business: calls on one stream are ordered)."""
        s = self.struct()
        need = lib().cgnn_spmm_workspace_bytes(ctypes.byref(s), i64(F), dtype_code(dtype), kernel)
        key = (int(F), dtype, kernel)
        ws = self._ws.get(key)
        if ws is None or ws.numel() < need:
            ws = torch.empty(max(need, 1), dtype=torch.uint8, device=self.rowptr.device)
            self._ws[key] = ws
        return ws, need


def spmm(A, X, Y=None, accumulate=False, kernel=SPMM_AUTO):
    """Y (+)= A @ X through cgnn_spmm.  Returns Y (allocated when None)."""
    F = X.shape[1]
    if Y is None:
        Y = torch.empty((A.rows, F), dtype=X.dtype, device=X.device)
        accumulate = False
    ws, need = A.workspace(F, X.dtype, kernel)
    s = A.struct()
    check(lib().cgnn_spmm(ctypes.byref(s), dtype_code(X.dtype), ptr(X), ptr(Y), i64(F),
                          ctypes.c_int(1 if accumulate else 0), ctypes.c_int(kernel), ptr(ws),
                          ctypes.c_size_t(need), stream_of(X)))
    return Y


def spmm_static(A, X, Y, accumulate=False, kernel=SPMM_AUTO):
    """Y (+)= A @ X through cgnn_spmm_static: the caller brings X and Y, the library its own
    scratch; nothing is allocated by the call."""
    s = A.struct()
    check(lib().cgnn_spmm_static(ctypes.byref(s), dtype_code(X.dtype), ptr(X), ptr(Y), i64(X.shape[1]),
                                 ctypes.c_int(1 if accumulate else 0), ctypes.c_int(kernel), stream_of(X)))
    return Y


def spmm_dual(A, split, X0, X1, Y=None, kernel=SPMM_AUTO):
    """Y = A[:, :split] @ X0 + A[:, split:] @ X1 in one pass through cgnn_spmm_dual."""
    F = X0.shape[1]
    if Y is None:
        Y = torch.empty((A.rows, F), dtype=X0.dtype, device=X0.device)
    ws, need = A.workspace(F, X0.dtype, kernel)
    s = A.struct()
    check(lib().cgnn_spmm_dual(ctypes.byref(s), i64(split), dtype_code(X0.dtype), ptr(X0), ptr(X1), ptr(Y),
                               i64(F), ctypes.c_int(kernel), ptr(ws), ctypes.c_size_t(need), stream_of(X0)))
    return Y


def lsh_assign(x, planes, bits):
    """(ids int64 [N], counts int32 [active+1], active) through the three LSH entry
    points; one host read of the active-bucket count."""
    N, F = x.shape
    dev = x.device
    L = lib()
    buckets = 1 << bits
    bucket_count = torch.empty(buckets, dtype=torch.int32, device=dev)
    prefix = torch.empty(buckets, dtype=torch.int32, device=dev)
    scan_bytes = L.cgnn_lsh_scan_workspace_bytes(bits)
    scan_ws = torch.empty(max(scan_bytes, 1), dtype=torch.uint8, device=dev)
    raw = torch.empty(N, dtype=torch.int32, device=dev)
    ids = torch.empty(N, dtype=torch.int64, device=dev)
    st = stream_of(x)
    check(L.cgnn_lsh_hash(i64(N), i64(F), bits, dtype_code(x.dtype), ptr(x), ptr(planes), ptr(raw),
                          ptr(bucket_count), st))
    check(L.cgnn_lsh_scan(bits, ptr(bucket_count), ptr(prefix), ptr(scan_ws), ctypes.c_size_t(scan_bytes), st))
    active = int(prefix[-1].item())
    counts = torch.zeros(active + 1, dtype=torch.int32, device=dev)
    check(L.cgnn_lsh_finish(i64(N), bits, ptr(raw), ptr(bucket_count), ptr(prefix), ptr(ids), ptr(counts), st))
    return ids, counts, active


def lsh_assign_grouped(x, planes, bits):
    """(ids, counts, active, (offsets, perm, sorted_id)) through cgnn_lsh_hash without
    counters and cgnn_lsh_group (sort by code); one host read of the group count."""
    N, F = x.shape
    dev = x.device
    L = lib()
    cap = min(N, 1 << bits)
    raw = torch.empty(N, dtype=torch.int32, device=dev)
    ids = torch.empty(N, dtype=torch.int64, device=dev)
    perm = torch.empty(N, dtype=torch.int32, device=dev)
    sorted_id = torch.empty(N, dtype=torch.int32, device=dev)
    offsets = torch.empty(cap + 2, dtype=torch.int32, device=dev)
    counts = torch.zeros(cap + 1, dtype=torch.int32, device=dev)
    active = torch.zeros(2, dtype=torch.int32, device=dev)  # number of groups, largest group
    st = stream_of(x)
    check(L.cgnn_lsh_hash(i64(N), i64(F), bits, dtype_code(x.dtype), ptr(x), ptr(planes), ptr(raw), None, st))
    need = L.cgnn_lsh_group_workspace_bytes(i64(N), bits)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    check(L.cgnn_lsh_group(i64(N), bits, ptr(raw), ptr(ids), ptr(offsets), ptr(perm), ptr(sorted_id), ptr(counts),
                           ptr(active), ptr(ws), ctypes.c_size_t(need), st))
    n, largest = (int(v) for v in active.cpu())
    return ids, counts[:n + 1], n, (offsets[:n + 2], perm, sorted_id, largest)


def csr_transpose(rowptr, col, value, cols):
    """(colptr, row, value) of an int64 CSR block on the GPU: the CSR of its transpose, entries
    sorted by column, ties in storage order."""
    dev = rowptr.device
    rows, nnz = rowptr.numel() - 1, col.numel()
    L = lib()
    colptr = torch.empty(cols + 1, dtype=torch.int64, device=dev)
    row = torch.empty(nnz, dtype=torch.int64, device=dev)
    tval = None if value is None else torch.empty_like(value)
    bad = torch.empty(1, dtype=torch.int32, device=dev)
    need = L.cgnn_csr_transpose_workspace_bytes(i64(nnz))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    null = ctypes.c_void_p(0)
    check(L.cgnn_csr_transpose_device(
        i64(rows), i64(cols), i64(nnz), ptr(rowptr), ptr(col) if nnz else null,
        ctypes.c_int(dtype_code(value.dtype) if value is not None else F32),
        ptr(value) if (value is not None and nnz) else null, ptr(colptr), ptr(row) if nnz else null,
        ptr(tval) if (tval is not None and nnz) else null, ptr(bad), ptr(ws), ctypes.c_size_t(need), stream_of(rowptr)))
    if int(bad.item()) != 0:
        raise CgnnError("csr_transpose: column out of range [0, %d)" % cols)
    return colptr, row, tval


def _id_flag(dev):
    return torch.zeros(1, dtype=torch.int32, device=dev)


def _check_id_flag(flag, what, groups):
    if int(flag.item()) != 0:
        raise CgnnError("%s: cluster id outside [0, %d)" % (what, groups))


def cluster_members(ids, groups):
    """(offsets int32 [groups+1], perm int32 [N], sorted_id int32 [N])."""
    N = ids.numel()
    dev = ids.device
    L = lib()
    offsets = torch.empty(groups + 1, dtype=torch.int32, device=dev)
    perm = torch.empty(N, dtype=torch.int32, device=dev)
    sorted_id = torch.empty(N, dtype=torch.int32, device=dev)
    need = L.cgnn_cluster_members_workspace_bytes(i64(N), i64(groups))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    bad = _id_flag(dev)
    check(L.cgnn_cluster_members(i64(N), i64(groups), ptr(ids), ptr(offsets), ptr(perm), ptr(sorted_id),
                                 ptr(bad), ptr(ws), ctypes.c_size_t(need), stream_of(ids)))
    _check_id_flag(bad, "cluster_members", groups)
    return offsets, perm, sorted_id


def cluster_mean(x, members, counts, max_members=0):
    offsets, perm, sorted_id = members[:3]
    N, F = x.shape
    groups = counts.numel()
    L = lib()
    reps = torch.empty((groups, F), dtype=x.dtype, device=x.device)
    need = L.cgnn_cluster_mean_workspace_bytes(i64(N), i64(F), i64(groups), dtype_code(x.dtype))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    check(L.cgnn_cluster_mean(i64(N), i64(F), i64(groups), i64(max_members), dtype_code(x.dtype), ptr(x), ptr(offsets),
                              ptr(perm), ptr(sorted_id), ptr(counts), ptr(reps), ptr(ws),
                              ctypes.c_size_t(need), stream_of(x)))
    return reps


def cluster_mean_backward(grad, ids, counts, members=None):
    N = ids.numel()
    F = grad.shape[1]
    dx = torch.empty((N, F), dtype=grad.dtype, device=grad.device)
    perm = None if members is None else members[1]
    bad = _id_flag(grad.device)
    check(lib().cgnn_cluster_mean_backward(i64(N), i64(F), i64(counts.numel()), dtype_code(grad.dtype),
                                           ptr(grad), ptr(ids), ptr(counts), ptr(perm), ptr(dx), ptr(bad),
                                           stream_of(grad)))
    _check_id_flag(bad, "cluster_mean_backward", counts.numel())
    return dx


def reconstruct(reps, ids, bias=None, relu=False, members=None):
    N = ids.numel()
    F = reps.shape[1]
    out = torch.empty((N, F), dtype=reps.dtype, device=reps.device)
    perm = None if members is None else members[1]
    bad = _id_flag(reps.device)
    check(lib().cgnn_reconstruct(i64(N), i64(F), i64(reps.shape[0]), dtype_code(reps.dtype), ptr(reps),
                                 ptr(ids), ptr(perm), ptr(bias), ctypes.c_int(1 if relu else 0), ptr(out),
                                 ptr(bad), stream_of(reps)))
    _check_id_flag(bad, "reconstruct", reps.shape[0])
    return out


def reconstruct_signs(reps, ids, bias=None, members=None):
    """(rows with ReLU, int32 [N, ceil(F / 32)] sign bits)"""
    N = ids.numel()
    F = reps.shape[1]
    L = lib()
    L.cgnn_sign_words.restype = ctypes.c_int64
    out = torch.empty((N, F), dtype=reps.dtype, device=reps.device)
    signs = torch.empty((N, L.cgnn_sign_words(i64(F))), dtype=torch.int32, device=reps.device)
    perm = None if members is None else members[1]
    bad = _id_flag(reps.device)
    check(L.cgnn_reconstruct_signs(i64(N), i64(F), i64(reps.shape[0]), dtype_code(reps.dtype), ptr(reps), ptr(ids),
                                   ptr(perm), ptr(bias), ptr(out), ptr(signs), ptr(bad), stream_of(reps)))
    _check_id_flag(bad, "reconstruct_signs", reps.shape[0])
    return out, signs


def reconstruct_backward_signs(grad, signs, members, groups, max_members=0):
    offsets, perm, sorted_id = members[:3]
    N, F = grad.shape
    L = lib()
    reps_grad = torch.empty((groups, F), dtype=grad.dtype, device=grad.device)
    need = L.cgnn_cluster_mean_workspace_bytes(i64(N), i64(F), i64(groups), dtype_code(grad.dtype))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=grad.device)
    check(L.cgnn_reconstruct_backward_signs(i64(N), i64(F), i64(groups), i64(max_members), dtype_code(grad.dtype),
                                            ptr(grad), ptr(signs), ptr(offsets), ptr(perm), ptr(sorted_id),
                                            ptr(reps_grad), ptr(ws), ctypes.c_size_t(need), stream_of(grad)))
    return reps_grad


def reconstruct_backward(grad, output, members, groups, relu=False, max_members=0):
    offsets, perm, sorted_id = members[:3]
    N, F = grad.shape
    L = lib()
    reps_grad = torch.empty((groups, F), dtype=grad.dtype, device=grad.device)
    need = L.cgnn_cluster_mean_workspace_bytes(i64(N), i64(F), i64(groups), dtype_code(grad.dtype))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=grad.device)
    check(L.cgnn_reconstruct_backward(i64(N), i64(F), i64(groups), i64(max_members), dtype_code(grad.dtype), ptr(grad),
                                      ptr(output), ptr(offsets), ptr(perm), ptr(sorted_id),
                                      ctypes.c_int(1 if relu else 0), ptr(reps_grad), ptr(ws),
                                      ctypes.c_size_t(need), stream_of(grad)))
    return reps_grad
