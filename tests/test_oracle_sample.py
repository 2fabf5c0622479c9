"""Pins the sampler functions of the CPU oracle (oracle/oracle_sample.c; no GPU needed):
  * golden (samples, rows, cols) recorded from the reference's compiled module on compressed
    graphs of up to three rule levels (tests/golden/sample_golden.npz): the oracle, fed from
    the generator the reference drew from (torch's CPU generator under the recorded seed),
    reproduces them exactly, for the compressed and the plain form;
  * the compiled reference itself, where oracle/_ref is built, on larger graphs;
  * the expansion invariant: get_neighbor over all positions of a vertex and the full list
    are both the expanded in-list of the vertex (as a multiset), on graphs whose hierarchy the
    reference's degrees cover (one rule level);
  * the selection loop: distinct positions, all of them when the fan-out covers the degree,
    the counter-based generator's draws in range and reproducible."""
import os
import sys

import numpy as np
import pytest
import torch

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path[:0] = [os.path.join(ROOT, "compressgnn_amd"), os.path.join(ROOT, "compressgnn_amd", "layer"),
                os.path.join(ROOT, "compressgnn_amd", "loader")]
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def golden_blocks(g, i):
    pre = "r%d_" % i
    levels = int(g[pre + "levels"])
    pair = lambda nm: (g[pre + nm + "_vlist"].astype(np.int64), g[pre + nm + "_elist"].astype(np.int64))
    return dict(v2v=pair("v2v"), v2r=pair("v2r"), r2v=pair("r2v"),
                r2r=[(g[pre + "lv%d_vlist" % k].astype(np.int64), g[pre + "lv%d_elist" % k].astype(np.int64))
                     for k in range(levels)],
                v_degree=g[pre + "vertex_degree"].astype(np.int64), r_degree=g[pre + "rule_degree"].astype(np.int64))


def torch_draws(seed):
    """The reference's uniform_randint (src/sample/csrc/neighbor_sample.h:10-15) on the same generator."""
    torch.manual_seed(seed)
    return lambda high: int(torch.randint(0, high, (1,)))


def blocks_of(graph):
    pair = lambda b: tuple(t.cpu().numpy() for t in b.csr()[:2])
    return dict(v2v=pair(graph.v2v_graph), v2r=pair(graph.v2r_graph), r2v=pair(graph.r2v_graph),
                r2r=[pair(b) for b in graph.r2r_graph], v_degree=graph.vertex_degree.cpu().numpy(),
                r_degree=graph.rule_degree.cpu().numpy())


def compressed(kind, seed=3):
    import compressgnn_offline as off
    from CompressgnnData import CompressgnnData
    if kind == "blocks":
        n = 64
        v = np.arange(n + 1, dtype=np.int64) * 32
        e = np.tile(np.arange(32, dtype=np.int64), n)
    elif kind == "shared_lists":
        # 11 vertices with the same 32 targets: every target has 11 in-neighbours that are reached
        # through rules, and itself (the self loop)
        V = 140
        lens = np.zeros(V, np.int64)
        lens[:11] = 32
        v = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        e = np.tile(np.arange(100, 132, dtype=np.int64), 11)
    elif kind == "copy":
        v, e = off.gen_copy_model(1500, 9.0, 0.7, seed)
    else:
        v, e = off.gen_chung_lu(2708, 10500, 2.5, seed)
    V = len(v) - 1
    m = np.ones(V, bool)
    data = CompressgnnData(np.zeros((V, 1), np.float32), (v, e), np.zeros(V, np.int64), m, m, m, graph_type="csr",
                           min_pair_frequency=3)
    return data, np.asarray(v, np.int64), np.asarray(e, np.int64)


def misfit_graph():
    """A graph of two rule levels on which some expanded degrees exceed what the descent of
    get_neighbor finds (the reference's degrees do not cover every hierarchy): 500-vertex copy
    model, pairs merged from frequency 3 on, no threshold filter, depth limit 8."""
    import compressgnn_offline as off
    from CompressgnnData import CompressgnnData
    v, e = off.gen_copy_model(500, 9.8, 0.7, 1)
    m = np.ones(500, bool)
    data = CompressgnnData(np.zeros((500, 1), np.float32), (v, e), np.zeros(500, np.int64), m, m, m, add_self_loop=True,
                           normalize=False, graph_type="csr", min_pair_frequency=3, threshold=0, max_depth=8, min_edge=0,
                           verbose=False)
    return data


def test_positions_the_descent_cannot_resolve_are_out_of_range():
    """Where r_degree promises more than a rule's descent finds, storage_api.h:57-64 goes on to the next
    rule with a negative position and indexes before that rule's list (or throws when no rule
    follows).  The oracle reports every such position as out of range and never leaves the arrays."""
    data = misfit_graph()
    b = blocks_of(data.edge_index)
    assert data.edge_index.step >= 2
    lost = []
    for u in range(data.vertex_cnt):
        k = np.arange(b["v_degree"][u])
        got = oracle.get_neighbors(b, np.full(len(k), u), k)
        assert ((got >= 0) | (got == -1)).all() and (got < data.vertex_cnt).all()
        lost += [(u, int(p)) for p in k[got < 0]]
    assert len(lost) >= 5
    # the sampler raises when the selection loop draws such a position
    u, p = lost[0]
    with pytest.raises(IndexError):
        oracle.neighbor_sample(b, np.array([u], np.int64), [1], draw=lambda high: min(p, high - 1))
    # and samples as usual around it
    oracle.neighbor_sample(b, np.array([u], np.int64), [1], draw=lambda high: 0)


def test_golden_vectors_of_the_compiled_reference():
    g = np.load(os.path.join(GOLD, "sample_golden.npz"))
    off = np.load(os.path.join(GOLD, "offline_golden.npz"))
    assert int(g["n_cases"]) >= 20
    seen_levels = set()
    for c in range(int(g["n_cases"])):
        key = "s%d_" % c
        blocks = golden_blocks(off, int(g[key + "graph"]))
        seen_levels.add(len(blocks["r2r"]))
        plain = bool(g[key + "plain"])
        run = lambda: oracle.neighbor_sample(blocks, g[key + "input"], g[key + "fan"].tolist(),
                                             draw=torch_draws(int(g[key + "seed"])), plain=plain)
        if int(g[key + "raised"]):
            with pytest.raises(IndexError):
                run()
            continue
        samples, rows, cols = run()
        assert np.array_equal(samples, g[key + "samples"])
        assert np.array_equal(rows, g[key + "rows"]) and np.array_equal(cols, g[key + "cols"])
    assert {0, 1, 3} <= seen_levels


@pytest.mark.parametrize("kind", ["blocks", "copy", "chung_lu"])
def test_matches_the_compiled_reference(kind):
    ref = pytest.importorskip("compressgnn_sample_ref")
    data, v, e = compressed(kind)
    b = blocks_of(data.edge_index)
    t = torch.from_numpy
    rng = np.random.default_rng(5)
    V = data.vertex_cnt
    for fan in ([3, 2], [10 ** 6, 10 ** 6], [5, 10 ** 6, 2], [1, 1, 1, 1]):
        inp = rng.integers(0, V, size=12).astype(np.int64)
        inp[3] = inp[0]  # a vertex given twice
        seed = int(rng.integers(0, 10 ** 6))
        torch.manual_seed(seed)
        want = ref.neighbor_sample_cg_sim(t(b["v2v"][0]), t(b["v2v"][1]), t(b["v2r"][0]), t(b["v2r"][1]), t(b["r2v"][0]),
                                          t(b["r2v"][1]), [t(p) for p, _ in b["r2r"]], [t(i) for _, i in b["r2r"]],
                                          t(b["v_degree"]), t(b["r_degree"]), t(inp), fan)
        got = oracle.neighbor_sample(b, inp, fan, draw=torch_draws(seed))
        for a, w in zip(got, want):
            assert np.array_equal(a, w.numpy())
        # the plain form on the uncompressed in-lists of the same graph
        import compressgnn_offline as off
        colptr, row, _ = off.csr_transpose(v, e, None, V)
        torch.manual_seed(seed)
        want = ref.neighbor_sample_ori_impl(t(colptr), t(row), t(inp), fan)
        got = oracle.neighbor_sample(dict(v2v=(colptr, row)), inp, fan, draw=torch_draws(seed), plain=True)
        for a, w in zip(got, want):
            assert np.array_equal(a, w.numpy())


@pytest.mark.parametrize("kind", ["blocks", "copy"])
def test_expansion_invariant(kind):
    """Whatever the order, the positions 0 .. degree-1 of a vertex and its full list name the
    in-neighbours of the vertex in the graph with self loops that was compressed."""
    import compressgnn_offline as off
    data, v, e = compressed(kind)
    assert data.rule_cnt > 0 and data.edge_index.step <= 1
    b = blocks_of(data.edge_index)
    v2, e2 = off.add_self_loop_csr(v, e)
    V = data.vertex_cnt
    colptr, row, _ = off.csr_transpose(v2, e2, None, V)
    rng = np.random.default_rng(1)
    with_rules = np.nonzero(np.diff(b["v2r"][0]))[0]
    assert len(with_rules)
    for node in list(rng.integers(0, V, size=25)) + list(with_rules[:15]):
        want = np.sort(row[colptr[node]:colptr[node + 1]])
        degree = int(b["v_degree"][node])
        assert degree == len(want)
        by_position = oracle.get_neighbors(b, np.full(degree, node), np.arange(degree))
        assert np.array_equal(np.sort(by_position), want)
        assert np.array_equal(np.sort(oracle.neighbor_list(b, node)), want)
        assert oracle.get_neighbors(b, [node], [degree])[0] == -1  # one past the end: the reference throws


def test_selection_loop_properties():
    data, v, e = compressed("copy")
    b = blocks_of(data.edge_index)
    V = data.vertex_cnt
    inp = np.arange(0, V, 7, dtype=np.int64)
    for fan in (1, 3, 8):
        samples, rows, cols = oracle.neighbor_sample(b, inp, [fan], seed=9)
        again = oracle.neighbor_sample(b, inp, [fan], seed=9)
        assert all(np.array_equal(x, y) for x, y in zip((samples, rows, cols), again))
        other = oracle.neighbor_sample(b, inp, [fan], seed=10)
        assert not np.array_equal(other[2], cols)
        assert np.array_equal(samples[:len(inp)], inp) and len(np.unique(samples)) == len(samples)
        per_vertex = np.bincount(rows, minlength=len(inp))
        assert np.array_equal(per_vertex, np.minimum(b["v_degree"][inp], fan))
        # every sampled neighbour is an in-neighbour, and no position is taken twice: the
        # neighbours of a vertex without duplicate in-edges are distinct
        for i in range(0, len(inp), 17):
            mine = samples[cols[rows == i]]
            full = oracle.neighbor_list(b, inp[i])
            assert set(mine) <= set(full)
            if len(set(full)) == len(full):
                assert len(set(mine)) == len(mine)
    # a fan-out that covers every degree returns the full lists in order
    samples, rows, cols = oracle.neighbor_sample(b, inp[:20], [10 ** 9], seed=1)
    at = 0
    for i in range(20):
        full = oracle.neighbor_list(b, inp[i])
        assert np.array_equal(samples[cols[at:at + len(full)]], full) and np.all(rows[at:at + len(full)] == i)
        at += len(full)
    assert at == len(rows)
    draws = [oracle.counter_draw(5, 1, 10, j, j) for j in range(1, 200)]
    assert all(0 <= d < j for d, j in zip(draws, range(1, 200)))
    assert len(set(oracle.counter_draw(5, 1, i, 1000, 1000) for i in range(100))) > 60


def _chi2_ok(observed, expected, alpha=1e-6):
    """Pearson's statistic against the 1 - alpha quantile: a sound generator fails once in a million runs
    (the draws are a fixed function of fixed seeds, so the outcome is the same on every run)."""
    from scipy.stats import chi2
    observed, expected = np.asarray(observed, float).ravel(), np.asarray(expected, float).ravel()
    stat = float(((observed - expected) ** 2 / expected).sum())
    return stat < chi2.ppf(1 - alpha, len(observed) - 1), stat


def test_counter_draws_are_uniform_and_independent():
    """What mathematics fixes about the counter-based generator (the reference draws uniformly from
    [0, high) with a sequential generator, src/sample/csrc/neighbor_sample.h:10-15,112-118; a
    parallel sampler cannot replay that stream, but its draws must have the same law): every draw
    uniform over its range, and draws that differ in one key only (frontier position, step, layer,
    seed) independent of each other.  A biased multiply-high, a counter that ignores a key or two
    keys that collapse into one would each fail here."""
    n = 30000
    draw = oracle.counter_draw
    for high in (2, 3, 7, 10, 64, 1000, 12345, 2 ** 31 - 1, 2 ** 40 + 7):
        d = np.array([draw(11, 0, i, high, high) for i in range(n)], dtype=np.float64)
        assert d.min() >= 0 and d.max() < high
        bins = min(high, 50)
        counts = np.bincount((d * bins / high).astype(np.int64), minlength=bins)
        edges = np.floor(np.arange(bins + 1) * high / bins + 0.999999) if high > bins else np.arange(bins + 1)
        expected = n * np.diff(edges) / high if high > bins else np.full(bins, n / bins)
        ok, stat = _chi2_ok(counts, expected)
        assert ok, ("marginal", high, stat)
    high = 6
    base = np.array([draw(11, 0, i, 9, high) for i in range(n)])
    variants = {
        "next position": np.array([draw(11, 0, i + 1, 9, high) for i in range(n)]),
        "next step": np.array([draw(11, 0, i, 10, high) for i in range(n)]),
        "next layer": np.array([draw(11, 1, i, 9, high) for i in range(n)]),
        "next seed": np.array([draw(12, 0, i, 9, high) for i in range(n)]),
        "position and step exchanged": np.array([draw(11, 0, 9, i, high) for i in range(n)]),
    }
    for name, other in variants.items():
        joint = np.bincount(base * high + other, minlength=high * high)
        ok, stat = _chi2_ok(joint, np.full(high * high, n / (high * high)))
        assert ok, (name, stat)
        assert np.count_nonzero(base != other) > n // 2, name
    # steps of one vertex (the selection loop walks j upwards with high = j): no drift along j
    u = np.array([draw(3, 2, 77, j, j) / j for j in range(1, n + 1)])
    ok, stat = _chi2_ok(np.bincount((u[100:] * 20).astype(np.int64), minlength=20), np.full(20, (n - 100) / 20))
    assert ok, ("along the steps", stat)


def selection_law(d, fan):
    """Exact inclusion probabilities (single positions, pairs) of the reference's selection loop
    under independent uniform draws, by enumerating every draw sequence."""
    import itertools
    single, pair, total = np.zeros(d), np.zeros((d, d)), 0
    for draws in itertools.product(*[range(j) for j in range(d - fan, d)]):
        chosen = []
        for j, rnd in zip(range(d - fan, d), draws):
            chosen.append(j if rnd in chosen else rnd)
        single[chosen] += 1
        for a in chosen:
            pair[a, chosen] += 1
        total += 1
    return single / total, pair / total


def test_selection_loop_follows_the_law_of_the_reference_loop():
    """The selection loop (neighbor_sample.h:112-118) fed by the counter-based generator.  The loop
    draws step j from [0, j), j excluded (torch::randint's upper bound, :10-15), and takes j itself on a
    collision, so the positions are not equally likely (the last one is taken on a collision
    only).  Its exact law under independent uniform draws is enumerated here -- all 7*8*9*10*11
    draw sequences for 5 of 12 -- and the frequencies of single positions and of pairs over many
    frontier positions are held to it."""
    d, fan, n = 12, 5, 8000
    single, pair = selection_law(d, fan)
    assert abs(single.sum() - fan) < 1e-9 and single[d - 1] < single[0]
    colptr = np.array([0, d] + [d] * d, dtype=np.int64)
    row = np.arange(1, d + 1, dtype=np.int64)
    samples, rows, cols = oracle.neighbor_sample(dict(v2v=(colptr, row)), np.zeros(n, np.int64), [fan], seed=5, plain=True)
    assert len(rows) == n * fan
    picked = samples[rows].reshape(n, fan) - 1  # plain form: rows index the sampled neighbours
    assert all(len(set(p)) == fan for p in picked)
    ok, stat = _chi2_ok(np.bincount(picked.ravel(), minlength=d), n * single)
    assert ok, ("single", stat)
    member = np.zeros((n, d), bool)
    member[np.arange(n)[:, None], picked] = True
    iu = np.triu_indices(d, 1)
    seen = (member[:, :, None] & member[:, None, :]).sum(0)[iu]
    ok, stat = _chi2_ok(seen, n * pair[iu])
    assert ok, ("pairs", stat)
    # the uniform law would be rejected by the same data: the test can tell the two apart
    ok, stat = _chi2_ok(np.bincount(picked.ravel(), minlength=d), np.full(d, n * fan / d))
    assert not ok
