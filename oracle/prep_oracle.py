"""Pure numpy / Python restatement of the reference's graph-format routines (small inputs).

TEST INFRASTRUCTURE ONLY (see oracle.c).  Each function cites the reference code
(ZhengChenCS/CompressGNN, paths relative to its root) whose result it restates; all of
them are pinned by tests/golden/offline_golden.npz, which holds the outputs of the
reference's own compiled routines on seeded graphs.
"""
import numpy as np


def add_self_loop_csr(vlist, elist):
    """src/offline/csrc/add_self_loop.h:17-43 (rows sorted ascending)."""
    nv, ne = [0], []
    for v in range(len(vlist) - 1):
        row = list(elist[vlist[v]:vlist[v + 1]])
        if v not in row:
            k = 0
            while k < len(row) and row[k] < v:
                k += 1
            row.insert(k, v)
        ne += row
        nv.append(len(ne))
    return np.array(nv, np.int64), np.array(ne, np.int64)


def get_norm_degree(dst, vertex_cnt):
    """src/offline/csrc/norm.h:20-45: float32 count on top of 1e-6, then 1/sqrt in float32."""
    d = np.full(vertex_cnt, np.float32(1e-6), dtype=np.float32)
    one = np.float32(1)
    for v in dst:
        d[v] = np.float32(d[v] + one)
    return (one / np.sqrt(d, dtype=np.float32)).astype(np.float32)


def gcn_norm_csr_compress(vlist, elist, d, V, R):
    """src/offline/csrc/norm.h:179-216."""
    w = np.empty(len(elist), np.float32)
    for n in range(V + R):
        for e in range(vlist[n], vlist[n + 1]):
            c = elist[e]
            if n < V:
                w[e] = np.float32(d[n] * d[c]) if c < V else d[n]
            else:
                w[e] = d[c] if c < V else np.float32(1)
    return w


def csc(vlist, elist, value, cols):
    """Entries ordered by column, then row, ties in storage order: the order of
    torch_sparse's SparseTensor.csc() that loader/CompressgnnData.py:180 relies on."""
    rows = len(vlist) - 1
    src = np.repeat(np.arange(rows), np.diff(vlist))
    key = np.lexsort((np.arange(len(elist)), src, elist))
    colptr = np.zeros(cols + 1, np.int64)
    np.cumsum(np.bincount(elist, minlength=cols), out=colptr[1:])
    return colptr, src[key].astype(np.int64), (None if value is None else np.asarray(value)[key])


def hybird_partition(vlist, elist, value, V):
    """src/offline/csrc/partition.h:14-110."""
    total = len(vlist) - 1
    blocks = [[[0], [], []] for _ in range(4)]  # v2v, v2r, r2v, r2r
    for r in range(total):
        to_vertex, to_rule = blocks[0 if r < V else 2], blocks[1 if r < V else 3]
        e, end = vlist[r], vlist[r + 1]
        while e < end and elist[e] < V:
            to_vertex[1].append(elist[e]); to_vertex[2].append(value[e]); e += 1
        while e < end:
            to_rule[1].append(elist[e] - V); to_rule[2].append(value[e]); e += 1
        to_vertex[0].append(len(to_vertex[1])); to_rule[0].append(len(to_rule[1]))
    return [(np.array(b[0], np.int64), np.array(b[1], np.int64), np.array(b[2], np.float32)) for b in blocks]


def topo_partition(vlist, elist, value):
    """src/offline/csrc/partition.h:112-216."""
    R = len(vlist) - 1
    order = [-1] * R
    left = R
    for r in range(R):
        if vlist[r + 1] == vlist[r]:
            order[r] = 0; left -= 1
    sweep = 1
    while left > 0:
        for r in range(R):
            if order[r] != -1:
                continue
            if all(order[c] != -1 for c in elist[vlist[r]:vlist[r + 1]]):
                order[r] = sweep; left -= 1
        sweep += 1
    levels = sweep - 1
    out = [[[0], [], []] for _ in range(levels)]
    for r in range(R):
        k = order[r] - 1
        if k >= 0:
            out[k][1] += list(elist[vlist[r]:vlist[r + 1]])
            out[k][2] += list(value[vlist[r]:vlist[r + 1]])
        for lv in out:
            lv[0].append(len(lv[1]))
    return [(np.array(l[0], np.int64), np.array(l[1], np.int64), np.array(l[2], np.float32)) for l in out], order


def gen_degree(v2v, v2r, r2v, levels):
    """src/offline/csrc/gen_degree.h:52-82."""
    vd = np.diff(v2v[0]).astype(np.int64)
    rd = np.diff(r2v[0]).astype(np.int64)
    for lv in reversed(levels):
        for r in range(len(rd)):
            for e in range(lv[0][r], lv[0][r + 1]):
                rd[r] += rd[lv[1][e]]
    for v in range(len(vd)):
        for e in range(v2r[0][v], v2r[0][v + 1]):
            vd[v] += rd[v2r[1][e]]
    return vd, rd


def expand(vlist, elist, node, V):
    """Ordered expansion of a node of a compressed CSR into vertex ids
    (tests/test_batch_compression.py:15-27 of the reference)."""
    stack = list(reversed([int(c) for c in elist[vlist[node]:vlist[node + 1]]]))
    out = []
    while stack:
        child = stack.pop()
        if child < V:
            out.append(child)
        else:
            children = elist[vlist[child]:vlist[child + 1]]
            assert np.all(children < child), "rule graph must be acyclic (children < rule)"
            stack.extend(reversed([int(c) for c in children]))
    return out


def add_self_loop_coo(src, dst, vertex_cnt):
    """src/offline/csrc/add_self_loop.h:55-107 (edges grouped by ascending source, targets
    ascending within a source)."""
    ns, nd = [], []
    e, E = 0, len(src)
    for v in range(vertex_cnt):
        mine = []
        while e < E and src[e] == v:
            mine.append(int(dst[e]))
            e += 1
        below = [t for t in mine if t < v]
        rest = mine[len(below):]
        if not rest or rest[0] != v:
            rest = [v] + rest
        for t in below + rest:
            ns.append(v)
            nd.append(t)
    return np.array(ns, np.int64), np.array(nd, np.int64)


def gcn_norm_coo_compress(src, dst, d, V, R):
    """src/offline/csrc/norm.h:129-166."""
    w = np.empty(len(src), np.float32)
    for e, (s, t) in enumerate(zip(src, dst)):
        if s < V:
            w[e] = np.float32(d[s] * d[t]) if t < V else d[s]
        else:
            w[e] = d[t] if t < V else np.float32(1)
    return w


def gen_edge_order(src, dst, V, R):
    """src/offline/csrc/gen_mask.h:10-84: (phase of every edge, number of phases)."""
    E = len(src)
    order = np.full(E, -1, np.int32)
    pending = np.zeros(R, np.int64)
    for e in range(E):
        if dst[e] >= V:
            pending[dst[e] - V] += 1
    for e in range(E):
        if src[e] < V:
            order[e] = 0
            if dst[e] >= V:
                pending[dst[e] - V] -= 1
    step = 1
    while (order < 0).any():
        arrived = np.zeros(R, np.int64)
        for e in range(E):
            if src[e] >= V and order[e] < 0 and pending[src[e] - V] == 0:
                order[e] = step
                if dst[e] >= V and pending[dst[e] - V] > 0:
                    arrived[dst[e] - V] += 1
        pending -= arrived
        step += 1
    return order, step


def coo_propagate(x, phases, weights, V, R):
    """layer/CompressgnnPropagation.py:68-83 with KPropagate.message (layer/KPropagate.py:30-31)
    and a sequential scatter-add in edge order: out[(V+R) x F] starts at zero, phase 0
    gathers from x, later phases from out; returns out[:V]."""
    out = np.zeros((V + R, x.shape[1]), x.dtype)
    for k, (edges, w) in enumerate(zip(phases, weights)):
        feat = x if k == 0 else out
        msg = feat[edges[0]] if w is None else (w.reshape(-1, 1) * feat[edges[0]]).astype(x.dtype)
        np.add.at(out, edges[1], msg)
    return out[:V]
