"""numpy front end of the CPU oracle (oracle/oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product never imports this module.

Each function names the reference code (ZhengChenCS/CompressGNN, paths relative to its
root) that it restates.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "oracle"], check=True, stdout=subprocess.PIPE,
                   stderr=subprocess.STDOUT)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_max_threads.restype = ctypes.c_int
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError("oracle supports float32/float64 only")


def max_threads():
    return lib().oracle_max_threads()


def spmm(vlist, elist, value, mat, out=None, threads=1):
    """spmm_func(..., "rowbalance", out) on CPU tensors:
    src/runtime/csrc/sparse/cpu/spmm_cpu.cpp:19-70.  Returns the accumulated array (a
    fresh zero-initialised one when out is None; `out` is updated in place otherwise,
    including when it is `mat` itself)."""
    vlist = _c(vlist, np.int64)
    elist = _c(elist, np.int64)
    rows = vlist.shape[0] - 1
    F = mat.shape[1]
    value = _c(value, mat.dtype)
    assert mat.flags.c_contiguous
    if out is None:
        out = np.zeros((rows, F), dtype=mat.dtype)
    assert out.flags.c_contiguous and out.dtype == mat.dtype and out.shape == (rows, F)
    fn = getattr(lib(), "oracle_spmm_" + _suffix(mat.dtype))
    fn(ctypes.c_int64(rows), _ptr(vlist), _ptr(elist), _ptr(value), _ptr(mat), ctypes.c_int64(F),
       _ptr(out), ctypes.c_int(threads))
    return out


def compress_spmm_forward(blocks, x, threads=1):
    """The 4-stage compressed propagation, layer/CompressgnnSPMM.py:43-62 (CPU branch).
    blocks = dict(v2v=(vlist, elist, value), v2r=..., r2v=..., r2r=[(vlist, elist, value), ...]).
    A graph without rules (r2v has no rows) yields the v2v product alone; the reference
    divides by zero there (spmm_cpu.cpp:43-45)."""
    rule_out = spmm(*blocks["r2v"], x, None, threads)
    for level in blocks["r2r"]:
        rule_out = spmm(*level, rule_out, rule_out, threads)
    out = spmm(*blocks["v2r"], rule_out, None, threads)
    out = spmm(*blocks["v2v"], x, out, threads)
    return out


def compress_spmm_backward(blocks_t, grad, threads=1):
    """Transposed propagation, layer/CompressgnnSPMM.py:65-86 (the working branch 80-85;
    the CPU branch 71-78 of the reference cannot run).  blocks_t holds the transposes:
    v2v_t, v2r_t (= csc of v2r, rows are rules), r2v_t (= csc of r2v, rows are
    vertices) and r2r_t[i] = csc of level i."""
    rule_g = spmm(*blocks_t["v2r_t"], grad, None, threads)
    for level in reversed(blocks_t["r2r_t"]):
        rule_g = spmm(*level, rule_g, rule_g, threads)
    gx = spmm(*blocks_t["v2v_t"], grad, None, threads)
    gx = spmm(*blocks_t["r2v_t"], rule_g, gx, threads)
    return gx


def lsh(x, planes, bits):
    """cluster_forward on CPU: src/runtime/csrc/cluster/cluster.cpp:12-30 and
    cpu/cluster_cpu.cpp:27-70, with the projection order fixed to an ascending fused
    multiply-add chain.  Returns (index int32 [N], active, raw_code int32 [N])."""
    if not 0 <= bits <= 30:
        raise ValueError("Hash bits must be in [0,30]")
    x = np.ascontiguousarray(x)
    planes = _c(planes, x.dtype)
    N, F = x.shape
    assert planes.shape == (F, bits)
    index = np.zeros(N, dtype=np.int32)
    raw = np.zeros(N, dtype=np.int32)
    active = ctypes.c_int32(0)
    fn = getattr(lib(), "oracle_lsh_" + _suffix(x.dtype))
    fn(ctypes.c_int64(N), ctypes.c_int64(F), ctypes.c_int(bits), _ptr(x), _ptr(planes), _ptr(index),
       ctypes.byref(active), _ptr(raw))
    return index, int(active.value), raw


def assign(x, planes, bits):
    """_assign on the CPU path, layer/CompressgnnCluster.py:41-50: ids widened to int64,
    counts = bincount(index, minlength=active+1) as int32."""
    if x.shape[0] == 0:
        return np.zeros(0, np.int64), np.zeros(1, np.int32), 0
    index, active, _ = lsh(x, planes, bits)
    index = index.astype(np.int64)
    counts = np.bincount(index, minlength=active + 1).astype(np.int32)
    return index, counts, active


def cluster_mean(x, index, counts):
    """_mean_forward, layer/CompressgnnCluster.py:16-19."""
    x = np.ascontiguousarray(x)
    index = _c(index, np.int64)
    counts = _c(counts, np.int32)
    N, F = x.shape
    groups = counts.shape[0]
    reps = np.zeros((groups, F), dtype=x.dtype)
    fn = getattr(lib(), "oracle_cluster_mean_" + _suffix(x.dtype))
    fn(ctypes.c_int64(N), ctypes.c_int64(F), ctypes.c_int64(groups), _ptr(x), _ptr(index), _ptr(counts),
       _ptr(reps))
    return reps


def cluster_mean_backward(grad, index, counts, threads=1):
    """_mean_backward, layer/CompressgnnCluster.py:22-25."""
    grad = np.ascontiguousarray(grad)
    index = _c(index, np.int64)
    counts = _c(counts, np.int32)
    N = index.shape[0]
    F = grad.shape[1]
    dx = np.empty((N, F), dtype=grad.dtype)
    fn = getattr(lib(), "oracle_cluster_mean_backward_" + _suffix(grad.dtype))
    fn(ctypes.c_int64(N), ctypes.c_int64(F), _ptr(grad), _ptr(index), _ptr(counts), _ptr(dx),
       ctypes.c_int(threads))
    return dx


def reconstruct(reps, index, bias=None, relu=False, threads=1):
    """Compressgnn_Reconstruct.forward, layer/CompressgnnReconstruct.py:34-42."""
    reps = np.ascontiguousarray(reps)
    index = _c(index, np.int64)
    if bias is not None:
        bias = _c(bias, reps.dtype)
    N = index.shape[0]
    F = reps.shape[1]
    out = np.empty((N, F), dtype=reps.dtype)
    fn = getattr(lib(), "oracle_reconstruct_" + _suffix(reps.dtype))
    fn(ctypes.c_int64(N), ctypes.c_int64(F), _ptr(reps), _ptr(index), _ptr(bias), ctypes.c_int(bool(relu)),
       _ptr(out), ctypes.c_int(threads))
    return out


def reconstruct_backward(grad, index, output, groups, relu=False):
    """cluster_reconstruct_backward, src/runtime/csrc/cluster/cuda/cluster_kernel.cu:98-108,196-208;
    bias_grad is reps_grad.sum(0) (layer/CompressgnnReconstruct.py:26)."""
    grad = np.ascontiguousarray(grad)
    output = _c(output, grad.dtype)
    index = _c(index, np.int64)
    N, F = grad.shape
    reps_grad = np.zeros((groups, F), dtype=grad.dtype)
    fn = getattr(lib(), "oracle_reconstruct_backward_" + _suffix(grad.dtype))
    fn(ctypes.c_int64(N), ctypes.c_int64(F), ctypes.c_int64(groups), _ptr(grad), _ptr(output), _ptr(index),
       ctypes.c_int(bool(relu)), _ptr(reps_grad))
    return reps_grad


# ---- neighbour sampling over a compressed graph (oracle_sample.c) -------------------------
DRAW_FN = ctypes.CFUNCTYPE(ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                           ctypes.c_void_p)


def _graph_args(blocks):
    """blocks: dict with v2v, v2r, r2v = (ptr, idx) int64 arrays, r2r = [(ptr, idx), ...],
    v_degree, r_degree (int64 arrays or None).  Returns (ctypes arguments, keep-alive list)."""
    keep = []

    def arr(a):
        a = _c(a, np.int64)
        keep.append(a)
        return _ptr(a)

    levels = len(blocks["r2r"])
    ptrs = (ctypes.c_void_p * max(levels, 1))(*[arr(p).value for p, _ in blocks["r2r"]])
    idxs = (ctypes.c_void_p * max(levels, 1))(*[arr(i).value if len(i) else None for _, i in blocks["r2r"]])
    keep += [ptrs, idxs]
    args = [arr(blocks["v2v"][0]), arr(blocks["v2v"][1]), arr(blocks["v2r"][0]), arr(blocks["v2r"][1]),
            arr(blocks["r2v"][0]), arr(blocks["r2v"][1]), ctypes.c_int(levels), ptrs, idxs]
    return args, keep


def _take64(pointer, n):
    out = np.ctypeslib.as_array(pointer, shape=(max(n, 1),))[:n].copy() if n else np.zeros(0, np.int64)
    lib().oracle_free(pointer)
    return out


def neighbor_sample(blocks, input_node, num_neighbors, draw=None, seed=0, plain=False):
    """neighbor_sample_cg_sim (src/sample/csrc/neighbor_sample.h:27-131) or, with plain=True and
    blocks["v2v"] = (colptr, row), neighbor_sample_ori_impl (:134-211).  draw(high) -> int in
    [0, high): the source of the random indices, called in the reference's order (its
    uniform_randint, :10-15); None: the counter-based generator of the HIP sampler with `seed`.
    Returns (samples, rows, cols); raises IndexError where the reference throws out_of_range."""
    L = lib()
    if plain:
        blocks = dict(v2v=blocks["v2v"], v2r=(np.zeros(len(blocks["v2v"][0]), np.int64), np.zeros(0, np.int64)),
                      r2v=(np.zeros(1, np.int64), np.zeros(0, np.int64)), r2r=[], v_degree=None, r_degree=None)
    args, keep = _graph_args(blocks)
    vdeg = _c(blocks["v_degree"] if blocks.get("v_degree") is not None else np.zeros(1), np.int64)
    rdeg = _c(blocks["r_degree"] if blocks.get("r_degree") is not None else np.zeros(1), np.int64)
    inp = _c(input_node, np.int64)
    fan = _c(num_neighbors, np.int64)
    cb = DRAW_FN(lambda high, layer, i, j, user: int(draw(high))) if draw is not None else ctypes.cast(None, DRAW_FN)
    ps, pr, pc = (ctypes.POINTER(ctypes.c_int64)() for _ in range(3))
    ns, ne = ctypes.c_int64(0), ctypes.c_int64(0)
    vertex_cnt = len(blocks["v2v"][0]) - 1
    rc = L.oracle_neighbor_sample(ctypes.c_int64(vertex_cnt), *args, _ptr(vdeg), _ptr(rdeg), _ptr(inp),
                                  ctypes.c_int64(len(inp)), _ptr(fan), ctypes.c_int(len(fan)), ctypes.c_int(1 if plain else 0),
                                  cb, None, ctypes.c_uint64(seed), ctypes.byref(ps), ctypes.byref(ns), ctypes.byref(pr),
                                  ctypes.byref(pc), ctypes.byref(ne))
    samples, rows, cols = _take64(ps, ns.value), _take64(pr, ne.value), _take64(pc, ne.value)
    if rc != 0:
        raise IndexError("Neighbor index out of range")
    return samples, rows, cols


def get_neighbors(blocks, nodes, indices):
    """get_neighbor (src/sample/csrc/storage_api.h:6-70) for (node, index) pairs; -1 where the
    reference throws out_of_range."""
    args, keep = _graph_args(blocks)
    nodes, indices = _c(nodes, np.int64), _c(indices, np.int64)
    out = np.zeros(len(nodes), np.int64)
    lib().oracle_get_neighbors(*args, _ptr(_c(blocks["v_degree"], np.int64)), _ptr(_c(blocks["r_degree"], np.int64)),
                               ctypes.c_int64(len(nodes)), _ptr(nodes), _ptr(indices), _ptr(out))
    return out


def neighbor_list(blocks, node):
    """get_neighbor_list (src/sample/csrc/storage_api.h:72-118)."""
    args, keep = _graph_args(blocks)
    p = ctypes.POINTER(ctypes.c_int64)()
    L = lib()
    L.oracle_neighbor_list.restype = ctypes.c_int64
    n = L.oracle_neighbor_list(*args, ctypes.c_int64(node), ctypes.byref(p))
    return _take64(p, n)


def counter_draw(seed, layer, i, j, high):
    L = lib()
    L.oracle_counter_draw.restype = ctypes.c_int64
    return L.oracle_counter_draw(ctypes.c_uint64(seed), ctypes.c_int64(layer), ctypes.c_int64(i), ctypes.c_int64(j),
                                 ctypes.c_int64(high))
