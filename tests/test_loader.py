"""CompressgnnData / CompressGraph on the host: fields and repr of the reference's
loader, block shapes, the expansion invariant (the blocks reproduce the original graph
with self loops), weights along every expanded path, and level ordering."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path[:0] = [os.path.join(ROOT, "compressgnn_amd"), os.path.join(ROOT, "compressgnn_amd", "layer"),
                os.path.join(ROOT, "compressgnn_amd", "loader")]

import compressgnn_offline as off  # noqa: E402
from CompressgnnData import CompressgnnData  # noqa: E402
from compress_graph import CompressGraph  # noqa: E402
from sparse_csr import SparseCSR  # noqa: E402


def make(kind, normalize=True, freq=3, add_self_loop=True):
    if kind == "blocks":
        n = 64
        v = np.arange(n + 1, dtype=np.int32) * 32
        e = np.tile(np.arange(32, dtype=np.int32), n)
    else:
        v, e = off.gen_copy_model(1500, 9.0, 0.7, 3)
    V = len(v) - 1
    x = np.random.default_rng(0).standard_normal((V, 8))
    mask = np.ones(V, dtype=bool)
    data = CompressgnnData(x, (v, e), np.zeros(V, np.int64), mask, mask, mask, add_self_loop=add_self_loop,
                           normalize=normalize, graph_type="csr", min_pair_frequency=freq)
    return data, np.asarray(v, np.int64), np.asarray(e, np.int64)


def dense_of(graph, V, R):
    """(V+R)-square matrix M with M[child, parent] = weight, from the blocks."""
    M = np.zeros((V + R, V + R))
    def put(g, r0, c0):
        rp, ci, val = (t.numpy() for t in g.csr())
        for r in range(len(rp) - 1):
            for k in range(rp[r], rp[r + 1]):
                M[r0 + r, c0 + ci[k]] += val[k]
    put(graph.v2v_graph, 0, 0)
    put(graph.v2r_graph, 0, V)
    put(graph.r2v_graph, V, 0)
    for g in graph.r2r_graph:
        put(g, V, V)
    return M


@pytest.mark.parametrize("kind", ["blocks", "copy"])
@pytest.mark.parametrize("normalize", [False, True])
def test_blocks_expand_to_the_original_graph(kind, normalize):
    data, v, e = make(kind, normalize)
    g = data.edge_index
    V, R = data.vertex_cnt, data.rule_cnt
    assert isinstance(g, CompressGraph) and R > 0
    assert data.x.dtype == torch.float32 and data.feature_dim == 8 and data.graph_type == "csr"
    assert repr(data).startswith('CompressgnnData(vertex_cnt:"%d", rule_cnt:"%d"' % (V, R)) and repr(g) == 'CompressGraph'
    assert g.v2v_graph.sparse_sizes() == (V, V) and g.v2r_graph.sparse_sizes() == (V, R)
    assert g.r2v_graph.sparse_sizes() == (R, V) and all(l.sparse_sizes() == (R, R) for l in g.r2r_graph)
    assert g.step == len(g.r2r_graph)
    for t in g.v2v_graph.csr()[:2]:
        assert t.dtype == torch.int64
    assert g.v2v_graph.csr()[2].dtype == torch.float32
    # out = (I - N)^-1 restricted to vertices: propagate the identity through the blocks
    M = dense_of(g, V, R)
    vv, vr, rv, rr = M[:V, :V], M[:V, V:], M[V:, :V], M[V:, V:]
    closure = np.linalg.inv(np.eye(R) - rr)  # rule levels are acyclic, so this is a finite sum
    A_t = vv + vr @ closure @ rv             # A_hat^T as the compressed chain computes it
    sv, se = off.add_self_loop_csr(v, e)
    src = np.repeat(np.arange(V), np.diff(sv))
    want = np.zeros((V, V))
    if normalize:
        d = off.get_norm_degree(se, V).astype(np.float64)
        np.add.at(want, (se, src), d[src] * d[se])
    else:
        np.add.at(want, (se, src), 1.0)
    np.testing.assert_allclose(A_t, want, rtol=1e-5, atol=1e-7)
    # expanded degrees count the expanded in-edges
    indeg = np.bincount(se, minlength=V)
    assert np.array_equal(g.vertex_degree.numpy(), indeg)


def test_csc_is_the_stable_transpose():
    rng = np.random.default_rng(1)
    rp = np.array([0, 3, 3, 6, 8])
    ci = np.array([2, 0, 2, 1, 1, 0, 3, 2])  # duplicates inside rows keep their order
    val = rng.standard_normal(8).astype(np.float32)
    g = SparseCSR(rp, ci, val, (4, 4))
    cp, row, tv = g.csc()
    assert cp.tolist() == [0, 2, 4, 7, 8]
    assert row.tolist() == [0, 2, 2, 2, 0, 0, 3, 3]
    assert np.array_equal(tv.numpy(), val[[1, 5, 3, 4, 0, 2, 7, 6]])
    assert g.t().sparse_sizes() == (4, 4) and g.to("cpu").nnz() == 8


def test_unsupported_paths_fail_loudly():
    with pytest.raises(ValueError):
        CompressgnnData(np.zeros((2, 1)), (np.array([0, 1]), np.array([1, 0])), np.zeros(2), np.ones(2, bool),
                        np.ones(2, bool), np.ones(2, bool), graph_type="ell")
    with pytest.raises(ValueError):
        CompressgnnData(np.zeros((2, 1)), (np.array([0, 1, 2]), np.array([1, 0])), np.zeros(2), np.ones(2, bool),
                        np.ones(2, bool), np.ones(2, bool), graph_type="csr", compression_backend="tpu")
    data, _, _ = make("blocks")
    from KPropagate import KPropagate
    with pytest.raises(RuntimeError, match="GPU"):
        KPropagate()(data.x, data.edge_index, None, data.vertex_cnt, data.rule_cnt)
    with pytest.raises(RuntimeError, match="GPU"):
        data.edge_index.plan()


def test_backend_resolution():
    import compression_backend as dispatch
    import torch
    assert dispatch.resolve_backend('cpu') == 'cpu'
    if torch.cuda.is_available():  # the GPU compressor is picked where a GPU is usable
        assert dispatch.resolve_backend('auto') == 'cuda' and dispatch.resolve_backend('cuda') == 'cuda'
    else:
        assert dispatch.resolve_backend('auto') == 'cpu'
        with pytest.raises(RuntimeError):
            dispatch.resolve_backend('cuda')
    for bad in ['wrong', 'legacy', None]:
        with pytest.raises(ValueError):
            dispatch.resolve_backend(bad)
    with pytest.raises(ValueError):
        dispatch.compress_graph_csr(np.array([0, 0]), np.array([], np.int64), 2)
    with pytest.raises(ValueError):
        dispatch.compress_graph_csr(np.array([0, 0]), np.array([], np.int64), 16, threads=0)


def test_coo_phases_cover_the_compressed_graph():
    """graph_type="coo": the phases partition the compressed edge list, phase 0 holds the
    edges that leave vertices, and summing the phases in order (the oracle's sequential
    scatter) reproduces the uncompressed normalised product."""
    import compressgnn_offline as off
    import prep_oracle
    V = 2708
    vl, el = off.gen_chung_lu(V, 10500, 2.5, 11)
    src, dst = off.csr2coo(vl, el)
    x = np.random.default_rng(2).standard_normal((V, 8)).astype(np.float32)
    m = np.ones(V, bool)
    data = CompressgnnData(x, (src, dst), np.zeros(V, np.int64), m, m, m, graph_type="coo",
                           min_pair_frequency=3, threshold=0)
    same = CompressgnnData(x, (vl, el), np.zeros(V, np.int64), m, m, m, graph_type="csr",
                           min_pair_frequency=3, threshold=0)
    assert (data.vertex_cnt, data.rule_cnt, data.edge_cnt) == (same.vertex_cnt, same.rule_cnt, same.edge_cnt)
    assert data.rule_cnt > 0 and data.step == len(data.edge_index) == len(data.edge_weight) >= 2
    assert sum(e.size(1) for e in data.edge_index) == data.edge_cnt
    assert bool((data.edge_index[0][0] < V).all())
    for e in data.edge_index[1:]:
        assert bool((e[0] >= V).all())
    out = prep_oracle.coo_propagate(x, [e.numpy() for e in data.edge_index], [w.numpy() for w in data.edge_weight],
                                    data.vertex_cnt, data.rule_cnt)
    s2, d2 = off.add_self_loop_coo(src, dst, V)
    nd = off.get_norm_degree(d2, V).astype(np.float64)
    want = np.zeros((V, 8))
    np.add.at(want, d2, (nd[s2] * nd[d2])[:, None] * x[s2])
    np.testing.assert_allclose(out, want, rtol=1e-4, atol=1e-5)
    assert "coo" in repr(data) and data.to("cpu") is data


def test_a_prepared_dataset_survives_torch_save(tmp_path):
    """The reference stores prepared datasets with torch.save(data) (genData/createCompressDataset.py:98).
    The file written here is this test's own, so loading it with the unpickler is in order."""
    import compressgnn_offline as off
    v, e = off.gen_copy_model(2000, 9.0, 0.7, 3)
    mask = np.ones(2000, dtype=bool)
    data = CompressgnnData(np.ones((2000, 3), np.float32), (v, e), np.zeros(2000, np.int64), mask, mask, mask,
                           graph_type="csr", min_pair_frequency=3, compression_backend="cpu")
    data.edge_index._plan = lambda: None  # stands for a device plan: not part of the file
    path = str(tmp_path / "data_csr.pt")
    torch.save(data, path)
    again = torch.load(path, weights_only=False)
    assert repr(again) == repr(data) and again.edge_index._plan is None
    for name in ("v2v_graph", "v2r_graph", "r2v_graph"):
        for a, b in zip(getattr(data.edge_index, name).csr(), getattr(again.edge_index, name).csr()):
            assert torch.equal(a, b)
    assert again.edge_index.step == data.edge_index.step
    assert torch.equal(again.edge_index.vertex_degree, data.edge_index.vertex_degree)


def test_batch_data_and_its_loader(tmp_path):
    """CompressgnnBatchData / CompressgnnDataLoader (loader/CompressgnnData.py:203-222 of the
    reference): a list of prepared datasets in one file, handed out one per step as shallow
    copies, in order or shuffled by the DataLoader's own arguments."""
    import compressgnn_offline as off
    from CompressgnnData import CompressgnnBatchData, CompressgnnDataLoader
    parts = []
    for seed, n in ((1, 300), (2, 500), (3, 400)):
        v, e = off.gen_copy_model(n, 6.0, 0.7, seed)
        mask = np.ones(n, dtype=bool)
        parts.append(CompressgnnData(np.full((n, 2), float(seed), np.float32), (v, e), np.zeros(n, np.int64), mask, mask,
                                     mask, graph_type="csr", min_pair_frequency=3, compression_backend="cpu"))
    path = str(tmp_path / "batches.pt")
    torch.save(parts, path)  # this test's own file
    batches = CompressgnnBatchData(path)
    assert len(batches) == 3
    seen = list(CompressgnnDataLoader(batches))
    assert [d.vertex_cnt for d in seen] == [300, 500, 400]
    for got, want in zip(seen, batches.data):
        assert got is not want and got.x is want.x and repr(got) == repr(want)  # a shallow copy
        assert float(got.x[0, 0]) == float(want.x[0, 0])
    shuffled = list(CompressgnnDataLoader(batches, shuffle=True, generator=torch.Generator().manual_seed(0)))
    assert sorted(d.vertex_cnt for d in shuffled) == [300, 400, 500]


def _binary_hierarchy(depth, width=2):
    """A compressed graph whose rules form `depth` levels of `width` rules each; every rule
    above the lowest level has all rules of the level below as children, so the vertices a
    rule stands for multiply by `width` per level while the stored entries grow by width^2."""
    V = 2 * width + 1
    rules = depth * width
    rows = [[] for _ in range(V + rules)]
    rid = lambda level, k: V + level * width + k
    for k in range(width):
        rows[rid(0, k)] = [1 + 2 * k, 2 + 2 * k]
    for level in range(1, depth):
        for k in range(width):
            rows[rid(level, k)] = [rid(level - 1, j) for j in range(width)]
    rows[0] = [rid(depth - 1, k) for k in range(width)]  # vertex 0 points at the top rules
    for v in range(1, V):
        rows[v] = [0]
    vlist = np.concatenate([[0], np.cumsum([len(r) for r in rows])]).astype(np.int64)
    elist = np.array([c for r in rows for c in r], dtype=np.int64)
    weight = np.ones(len(elist), np.float32)
    colptr, row, value = off.csr_transpose(vlist, elist, weight, V + rules)
    return CompressGraph(colptr, row, value, V), V, rules


def test_fold_bound_and_fallback_for_deep_hierarchies():
    """plan() folds the rule levels into the rule stage only while that stays cheap: the
    size bound (row lengths only) is exact when no columns merge and an upper bound otherwise,
    and a hierarchy whose folded rows would multiply out, or that is deeper than the limit,
    keeps one launch per level."""
    host = lambda triple: tuple(t.cpu().numpy() for t in triple)
    # a shallow hierarchy folds
    shallow, V, R = _binary_hierarchy(3)
    assert shallow.step == 2 and shallow.rule_cnt == R
    folded = shallow._fold_plan(host)
    assert folded is not None
    for base, levels, widest in ((folded[0], folded[1], 1), (folded[2], folded[3], 4)):
        bound = off.csr_fold_levels_bound(base, levels)
        rp, ci, val = off.csr_fold_levels(base, levels)
        assert bound >= len(ci) and bound <= 4.0 * (len(base[1]) + sum(len(l[1]) for l in levels))
        # forward, every rule descends from vertex 0 alone; backward, a top rule stands for the
        # four vertices below the lowest rules (reached along several paths, merged by column)
        assert np.diff(rp).max() == widest
    # exponential growth: 14 levels of 2 rules would fold into rows of 2^14 entries before merging
    deep, V, R = _binary_hierarchy(14)
    assert deep.step == 13
    fwd_base, fwd_levels = host(deep.r2v_graph.csr()), [host(g.csr()) for g in deep.r2r_graph]
    stored = len(fwd_base[1]) + sum(len(l[1]) for l in fwd_levels)
    assert off.csr_fold_levels_bound(fwd_base, fwd_levels) > 4.0 * stored
    assert deep._fold_plan(host) is None
    # a chain deeper than max_fold_depth is not folded even though it would not grow
    chain, V, R = _binary_hierarchy(20, width=1)
    assert chain.step == 19 and chain.step > CompressGraph.max_fold_depth
    assert chain._fold_plan(host) is None
    chain.max_fold_depth = 32
    assert chain._fold_plan(host) is not None
    # fold_levels = False always keeps the launch-per-level form
    shallow.fold_levels = False
    assert shallow._fold_plan(host) is None
    # random levels: the bound is never below the folded size
    rng = np.random.default_rng(3)
    Rn, Vn = 50, 30

    def to_csr(m):
        rp = np.concatenate([[0], np.cumsum((m != 0).sum(1))]).astype(np.int64)
        rows, cols = np.nonzero(m)
        return rp, cols.astype(np.int64), m[rows, cols].astype(np.float32)

    dense = np.where(rng.random((Rn, Vn)) < 0.2, 1.0, 0.0).astype(np.float32)
    lv = []
    for k in range(2):
        L = np.zeros((Rn, Rn), np.float32)
        lo, hi = 10 * k + 10, 10 * k + 20
        L[lo:hi, :lo] = rng.random((hi - lo, lo)) < 0.3
        lv.append(to_csr(L))
    rp, ci, _ = off.csr_fold_levels(to_csr(dense), lv)
    assert off.csr_fold_levels_bound(to_csr(dense), lv) >= len(ci)


def test_offloaded_blocks_deliver_to_their_device():
    """SparseCSR.offload(): the arrays rest on the host, the block still answers for its
    device (here the host itself, which makes offload a no-op that must change nothing)."""
    data, v, e = make("copy")
    g = data.edge_index.v2v_graph
    before = tuple(t.clone() for t in g.csr())
    csc_before = tuple(t.clone() for t in g.csc())
    assert not g.offloaded
    g.offload()
    assert not g.offloaded and g.device.type == "cpu"
    assert all(torch.equal(a, b) for a, b in zip(g.csr(), before))
    assert all(torch.equal(a, b) for a, b in zip(g.csc(), csc_before))


def test_host_merger_and_transpose_meet_the_independent_checkers():
    """The numpy checkers the GPU tests hold the device routines to (tests/util.py), applied to
    the host routines: the contract of the compressor boundary and the stable sort by column."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from util import assert_compression_contract, closed_form_transpose
    rng = np.random.default_rng(9)
    for V, freq in ((1, 3), (300, 3), (6000, 8)):
        v, e = (off.gen_copy_model(V, 9.8, 0.7, 5) if V > 1 else (np.array([0, 0], np.int64), np.zeros(0, np.int64)))
        got = off.compress_csr_batch(v, e, 4, 12, freq)
        assert_compression_contract(v, e, got)
        if got[3]:
            broken = got[1].copy()
            broken[0] = (broken[0] + 1) % V
            with pytest.raises(AssertionError):
                assert_compression_contract(v, e, (got[0], broken, got[2], got[3]))
    for rows, cols in ((7, 3), (300, 500), (5000, 300)):
        lens = rng.poisson(4, rows)
        v = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        e = rng.integers(0, cols, int(v[-1])).astype(np.int64)
        val = rng.standard_normal(len(e)).astype(np.float32)
        for a, b in zip(off.csr_transpose(v, e, val, cols), closed_form_transpose(v, e, val, cols)):
            assert np.array_equal(a, b)
