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
