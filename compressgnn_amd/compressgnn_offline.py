"""`compressgnn_offline`: the graph-preparation functions the loader needs, under the
names and argument meaning of the reference's offline module
(ZhengChenCS/CompressGNN src/offline/csrc/function.cpp:25-72), implemented by
libcgnn_prep.so (C++, include/compressgnn_prep.h) and reached through ctypes.
Inputs and outputs are numpy arrays (int64 indices, float32 weights).
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcgnn_prep.so")
_lib = None

EXPORTS = [
    "cgnn_arrays_count", "cgnn_arrays_type", "cgnn_arrays_size", "cgnn_arrays_data",
    "cgnn_arrays_scalar", "cgnn_arrays_free", "cgnn_prep_last_error",
    "cgnn_add_self_loop_csr", "cgnn_get_norm_degree", "cgnn_gcn_norm_csr_compress",
    "cgnn_csr_transpose", "cgnn_hybird_partition", "cgnn_topo_partition", "cgnn_gen_degree",
    "cgnn_filter_csr", "cgnn_depth_filter_csr", "cgnn_gen_vertex_order_csr", "cgnn_gen_vertex_order_csc",
    "cgnn_compress_csr_batch", "cgnn_csr_hstack", "cgnn_csr_row_stats", "cgnn_gen_chung_lu", "cgnn_gen_copy_model",
    "cgnn_add_self_loop_coo", "cgnn_gcn_norm_coo_compress", "cgnn_gen_edge_order",
    "cgnn_csr_locality_order", "cgnn_csr_permute_rows", "cgnn_csr_fold_levels",
]

_NP_TYPES = {0: np.int64, 1: np.float32, 2: np.int32}


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libcgnn_prep.so is not built (%s); run `python -m compressgnn_amd.build prep`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.cgnn_prep_last_error.restype = ctypes.c_char_p
        L.cgnn_arrays_size.restype = ctypes.c_int64
        L.cgnn_arrays_scalar.restype = ctypes.c_int64
        L.cgnn_arrays_data.restype = ctypes.c_void_p
        for name in EXPORTS:
            if name.startswith("cgnn_") and name not in (
                    "cgnn_arrays_count", "cgnn_arrays_type", "cgnn_arrays_size", "cgnn_arrays_data",
                    "cgnn_arrays_scalar", "cgnn_arrays_free", "cgnn_prep_last_error",
                    "cgnn_get_norm_degree", "cgnn_gcn_norm_csr_compress", "cgnn_gcn_norm_coo_compress",
                    "cgnn_csr_row_stats"):
                getattr(L, name).restype = ctypes.c_void_p
        L.cgnn_arrays_free.argtypes = [ctypes.c_void_p]
        L.cgnn_arrays_count.argtypes = [ctypes.c_void_p]
        L.cgnn_arrays_type.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.cgnn_arrays_size.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.cgnn_arrays_data.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.cgnn_arrays_scalar.argtypes = [ctypes.c_void_p, ctypes.c_int]
        _lib = L
    return _lib


def _err():
    return lib().cgnn_prep_last_error().decode()


def _i64(a):
    kind = np.asarray(a).dtype.kind
    if kind not in "iu":
        raise ValueError("CSR arrays must be integer arrays")
    return np.ascontiguousarray(a, dtype=np.int64)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _take(handle, n_scalars=0):
    """Copy the arrays of a result bundle into numpy and free it."""
    L = lib()
    if not handle:
        raise RuntimeError(_err())
    try:
        out = []
        for i in range(L.cgnn_arrays_count(handle)):
            dt = np.dtype(_NP_TYPES[L.cgnn_arrays_type(handle, i)])
            n = L.cgnn_arrays_size(handle, i)
            arr = np.empty(n, dtype=dt)
            if n:
                ctypes.memmove(arr.ctypes.data, L.cgnn_arrays_data(handle, i), n * dt.itemsize)
            out.append(arr)
        scalars = [int(L.cgnn_arrays_scalar(handle, i)) for i in range(n_scalars)]
    finally:
        L.cgnn_arrays_free(handle)
    return out, scalars


def add_self_loop_csr(vlist, elist):
    vlist, elist = _i64(vlist), _i64(elist)
    (v, e), _ = _take(lib().cgnn_add_self_loop_csr(ctypes.c_int64(len(vlist) - 1), _p(vlist), _p(elist)))
    return v, e


def get_norm_degree(dst, vertex_cnt):
    dst = _i64(dst)
    out = np.empty(vertex_cnt, dtype=np.float32)
    if lib().cgnn_get_norm_degree(ctypes.c_int64(len(dst)), _p(dst), ctypes.c_int64(vertex_cnt), _p(out)):
        raise RuntimeError(_err())
    return out


def gcn_norm_csr_compress(vlist, elist, norm_degree, vertex_cnt, rule_cnt):
    vlist, elist, d = _i64(vlist), _i64(elist), _f32(norm_degree)
    w = np.empty(len(elist), dtype=np.float32)
    if lib().cgnn_gcn_norm_csr_compress(ctypes.c_int64(vertex_cnt), ctypes.c_int64(rule_cnt), _p(vlist),
                                        _p(elist), _p(d), _p(w)):
        raise RuntimeError(_err())
    return w


def csr_transpose(vlist, elist, value, cols):
    """(colptr, row, value) of the transpose; value may be None."""
    vlist, elist = _i64(vlist), _i64(elist)
    v = None if value is None else _f32(value)
    (cp, row, val), _ = _take(lib().cgnn_csr_transpose(ctypes.c_int64(len(vlist) - 1), ctypes.c_int64(cols),
                                                       _p(vlist), _p(elist), _p(v)))
    return cp, row, (None if value is None else val)


def hybird_partition(vlist, elist, value, vertex_cnt):
    vlist, elist, value = _i64(vlist), _i64(elist), _f32(value)
    arrs, _ = _take(lib().cgnn_hybird_partition(ctypes.c_int64(len(vlist) - 1), _p(vlist), _p(elist),
                                                _p(value), ctypes.c_int64(vertex_cnt)))
    return tuple(tuple(arrs[3 * i:3 * i + 3]) for i in range(4))


def topo_partition(vlist, elist, value):
    vlist, elist, value = _i64(vlist), _i64(elist), _f32(value)
    arrs, (levels,) = _take(lib().cgnn_topo_partition(ctypes.c_int64(len(vlist) - 1), _p(vlist), _p(elist),
                                                      _p(value)), 1)
    return [tuple(arrs[3 * i:3 * i + 3]) for i in range(levels)]


def gen_degree(v2v_vlist, v2v_elist, v2r_vlist, v2r_elist, r2v_vlist, r2v_elist, r2r_vlists, r2r_elists):
    a = [_i64(np.asarray(x)) for x in (v2v_vlist, v2r_vlist, v2r_elist, r2v_vlist)]
    lv = [_i64(np.asarray(x)) for x in r2r_vlists]
    le = [_i64(np.asarray(x)) for x in r2r_elists]
    n = len(lv)
    PtrArr = ctypes.c_void_p * max(n, 1)
    pv = PtrArr(*[x.ctypes.data for x in lv]) if n else PtrArr()
    pe = PtrArr(*[x.ctypes.data for x in le]) if n else PtrArr()
    (vd, rd), _ = _take(lib().cgnn_gen_degree(ctypes.c_int64(len(a[0]) - 1), ctypes.c_int64(len(a[3]) - 1),
                                              _p(a[0]), _p(a[1]), _p(a[2]), _p(a[3]), ctypes.c_int(n), pv, pe))
    return vd, rd


def filter_csr(vlist, elist, vertex_cnt, rule_cnt, threshold=16):
    vlist, elist = _i64(vlist), _i64(elist)
    (v, e), (V, R) = _take(lib().cgnn_filter_csr(ctypes.c_int64(vertex_cnt), ctypes.c_int64(rule_cnt),
                                                 _p(vlist), _p(elist), ctypes.c_int(threshold)), 2)
    return v, e, V, R


def depth_filter_csr(vlist, elist, vertex_cnt, rule_cnt, max_depth, min_edge):
    vlist, elist = _i64(vlist), _i64(elist)
    (v, e), (V, R) = _take(lib().cgnn_depth_filter_csr(ctypes.c_int64(vertex_cnt), ctypes.c_int64(rule_cnt),
                                                       _p(vlist), _p(elist), ctypes.c_int(max_depth),
                                                       ctypes.c_int(min_edge)), 2)
    return v, e, V, R


def gen_vertex_order_csr(vlist, elist, vertex_cnt, rule_cnt):
    vlist, elist = _i64(vlist), _i64(elist)
    (order,), (depth,) = _take(lib().cgnn_gen_vertex_order_csr(ctypes.c_int64(vertex_cnt),
                                                              ctypes.c_int64(rule_cnt), _p(vlist), _p(elist)), 1)
    return order, depth


def gen_vertex_order_csc(vlist, elist, vertex_cnt, rule_cnt):
    vlist, elist = _i64(vlist), _i64(elist)
    (order,), (depth,) = _take(lib().cgnn_gen_vertex_order_csc(ctypes.c_int64(vertex_cnt),
                                                              ctypes.c_int64(rule_cnt), _p(vlist), _p(elist)), 1)
    return order, depth


def compress_csr_batch(vlist, elist, threads=4, rounds=12, min_pair_frequency=16):
    """(vlist int32, elist int32, vertex_cnt, rule_cnt); ValueError on non-integer or
    out-of-range input and on min_pair_frequency < 3, as the reference's bridge
    (src/offline/bindings/batch_bridge.hpp:8-26) and tests require."""
    for arr in (vlist, elist):
        a = np.asarray(arr)
        if a.ndim != 1 or a.dtype.kind not in "iu":
            raise ValueError("CSR arrays must be one-dimensional integer arrays")
        if a.size and (int(a.max()) > np.iinfo(np.int32).max or int(a.min()) < 0):
            raise ValueError("CSR value exceeds int32 range")
    if min_pair_frequency < 3:
        raise ValueError("Batch compression needs min_pair_frequency >= 3")
    if threads < 1 or rounds < 1:
        raise ValueError("threads and rounds must be positive")
    vlist, elist = _i64(vlist), _i64(elist)
    if len(vlist) == 0:
        return np.zeros(1, np.int32), np.zeros(0, np.int32), 0, 0
    h = lib().cgnn_compress_csr_batch(ctypes.c_int64(len(vlist) - 1), _p(vlist), _p(elist), ctypes.c_int(threads),
                                      ctypes.c_int(rounds), ctypes.c_int(min_pair_frequency))
    if not h:
        raise ValueError(_err())
    (v, e), (V, R) = _take(h, 2)
    return v, e, V, R


def coo2csr(src, dst, vertex_cnt):
    """src sorted ascending (src/offline/csrc/convert.h:3-35)."""
    src, dst = _i64(src), _i64(dst)
    vlist = np.zeros(vertex_cnt + 1, dtype=np.int64)
    np.cumsum(np.bincount(src, minlength=vertex_cnt), out=vlist[1:])
    return vlist, dst.copy()


def csr2coo(vlist, elist):
    """src/offline/csrc/convert.h:37-65."""
    vlist, elist = _i64(vlist), _i64(elist)
    src = np.repeat(np.arange(len(vlist) - 1, dtype=np.int64), np.diff(vlist))
    return src, elist.copy()


def add_self_loop_coo(src, dst, vertex_cnt):
    src, dst = _i64(src), _i64(dst)
    (s, d), _ = _take(lib().cgnn_add_self_loop_coo(ctypes.c_int64(len(src)), _p(src), _p(dst),
                                                   ctypes.c_int64(vertex_cnt)))
    return s, d


def gcn_norm_coo_compress(src, dst, norm_degree, vertex_cnt, rule_cnt):
    src, dst, d = _i64(src), _i64(dst), _f32(norm_degree)
    w = np.empty(len(src), dtype=np.float32)
    if lib().cgnn_gcn_norm_coo_compress(ctypes.c_int64(len(src)), _p(src), _p(dst), _p(d),
                                        ctypes.c_int64(vertex_cnt), ctypes.c_int64(rule_cnt), _p(w)):
        raise RuntimeError(_err())
    return w


def gen_edge_order(src, dst, vertex_cnt, rule_cnt):
    """(phase of every edge int32[E], number of phases)."""
    src, dst = _i64(src), _i64(dst)
    (order,), (phases,) = _take(lib().cgnn_gen_edge_order(ctypes.c_int64(len(src)), _p(src), _p(dst),
                                                          ctypes.c_int64(vertex_cnt), ctypes.c_int64(rule_cnt)), 1)
    return order, phases


def gen_mask_edge(src, dst, vertex_cnt, rule_cnt):
    """(bool mask [phases, E], phases): mask[k] selects the edges of phase k
    (src/offline/csrc/gen_mask.h:86-108)."""
    order, phases = gen_edge_order(src, dst, vertex_cnt, rule_cnt)
    return order[None, :] == np.arange(phases, dtype=np.int32)[:, None], phases


def csr_hstack(a0, a1, col_offset):
    """[A0 | A1] for two CSR triples (vlist, elist, value) with the same number of rows."""
    v0, e0, w0 = _i64(a0[0]), _i64(a0[1]), _f32(a0[2])
    v1, e1, w1 = _i64(a1[0]), _i64(a1[1]), _f32(a1[2])
    if len(v0) != len(v1):
        raise ValueError("csr_hstack: blocks must have the same number of rows")
    (v, e, w), _ = _take(lib().cgnn_csr_hstack(ctypes.c_int64(len(v0) - 1), _p(v0), _p(e0), _p(w0), _p(v1), _p(e1),
                                               _p(w1), ctypes.c_int64(col_offset)))
    return v, e, w


def csr_fold_levels(base, levels):
    """The CSR triple `base` (R rows) after the in-place updates base[r] += sum_c L[r, c] * base[c]
    for every level L (a list of R x R CSR triples, applied in order), as one matrix."""
    v, e, w = _i64(base[0]), _i64(base[1]), _f32(base[2])
    lv = [_i64(l[0]) for l in levels]
    le = [_i64(l[1]) for l in levels]
    lw = [_f32(l[2]) for l in levels]
    n = len(levels)
    ptrs = lambda arrs: (ctypes.c_void_p * max(n, 1))(*[a.ctypes.data for a in arrs])
    (nv, ne, nw), _ = _take(lib().cgnn_csr_fold_levels(ctypes.c_int64(len(v) - 1), _p(v), _p(e), _p(w), ctypes.c_int(n),
                                                     ptrs(lv), ptrs(le), ptrs(lw)))
    return nv, ne, nw


def csr_fold_levels_bound(base, levels):
    """Upper bound on the entries of csr_fold_levels(base, levels): the entries before equal
    columns of a row are merged.  Row sizes only (a float64 per rule, one pass per level), so a
    deep hierarchy whose folded rows would be huge is seen before anything is built."""
    size = np.diff(_i64(base[0])).astype(np.float64)
    for lv, le, _ in levels:
        lv, le = _i64(lv), _i64(le)
        if len(le) == 0:
            continue
        rows = np.repeat(np.arange(len(lv) - 1), np.diff(lv))
        size = size + np.bincount(rows, weights=size[le], minlength=len(size))
    return float(size.sum())


def csr_locality_order(vlist, elist):
    """Rows sorted lexicographically by their column lists (int32 [rows])."""
    vlist, elist = _i64(vlist), _i64(elist)
    (order,), _ = _take(lib().cgnn_csr_locality_order(ctypes.c_int64(len(vlist) - 1), _p(vlist), _p(elist)))
    return order


def csr_permute_rows(vlist, elist, value, order):
    """(vlist, elist, value) with row g = row order[g] of the input; value may be None."""
    vlist, elist = _i64(vlist), _i64(elist)
    v = None if value is None else _f32(value)
    order = np.ascontiguousarray(order, dtype=np.int32)
    (nv, ne, nw), _ = _take(lib().cgnn_csr_permute_rows(ctypes.c_int64(len(vlist) - 1), _p(vlist), _p(elist), _p(v),
                                                       _p(order)))
    return nv, ne, (None if value is None else nw)


def csr_row_stats(vlist):
    """(longest row, histogram of row lengths by powers of two)."""
    vlist = _i64(vlist)
    mx = ctypes.c_int64(0)
    hist = np.zeros(40, dtype=np.int64)
    if lib().cgnn_csr_row_stats(ctypes.c_int64(len(vlist) - 1), _p(vlist), ctypes.byref(mx), _p(hist)):
        raise RuntimeError(_err())
    return int(mx.value), hist


def gen_chung_lu(vertex_cnt, target_edges, exponent=2.5, seed=0):
    (v, e), _ = _take(lib().cgnn_gen_chung_lu(ctypes.c_int64(vertex_cnt), ctypes.c_int64(target_edges),
                                              ctypes.c_double(exponent), ctypes.c_uint64(seed)))
    return v, e


def gen_copy_model(vertex_cnt, avg_degree=9.8, copy_prob=0.7, seed=0):
    (v, e), _ = _take(lib().cgnn_gen_copy_model(ctypes.c_int64(vertex_cnt), ctypes.c_double(avg_degree),
                                                ctypes.c_double(copy_prob), ctypes.c_uint64(seed)))
    return v, e
