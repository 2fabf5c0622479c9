"""Host-side graph preparation (libcgnn_prep.so through compressgnn_offline) against
  * tests/golden/offline_golden.npz: outputs of the reference's own compiled offline
    routines on seeded graphs (bit-exact integer structure and float32 weights),
  * the numpy restatement in oracle/prep_oracle.py,
  * the compiled reference itself on fresh inputs where oracle/_ref is built,
  * the expansion invariants of the reference's tests for the compressor and filters
    (tests/test_offline_compression.py, tests/test_batch_compression.py)."""
import os
import sys
from collections import Counter

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "compressgnn_amd"))
import compressgnn_offline as off  # noqa: E402

import prep_oracle  # noqa: E402

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "offline_golden.npz"))


def eq(a, b):
    a, b = np.asarray(a), np.asarray(b)
    return a.shape == b.shape and np.array_equal(a, b)


def test_self_loop_and_norm_degree_golden():
    for i in range(int(GOLD["n_plain"])):
        p = "g%d_" % i
        v, e = GOLD[p + "vlist"], GOLD[p + "elist"]
        sv, se = off.add_self_loop_csr(v, e)
        assert eq(sv, GOLD[p + "sl_vlist"]) and eq(se, GOLD[p + "sl_elist"])
        ov, oe = prep_oracle.add_self_loop_csr(v, e)
        assert eq(ov, sv) and eq(oe, se)
        nd = off.get_norm_degree(se, len(v) - 1)
        assert nd.dtype == np.float32 and eq(nd, GOLD[p + "norm_degree"])
        assert eq(prep_oracle.get_norm_degree(se, len(v) - 1), nd)


def test_edge_list_routines_golden():
    """add_self_loop_coo, gcn_norm_coo_compress and the phase order of gen_edge_order /
    gen_mask_edge against the compiled reference's outputs."""
    for i in range(int(GOLD["n_coo"])):
        p = "c%d_" % i
        V = int(GOLD[p + "V"])
        s, d = off.add_self_loop_coo(GOLD[p + "src"], GOLD[p + "dst"], V)
        assert eq(s, GOLD[p + "sl_src"]) and eq(d, GOLD[p + "sl_dst"])
        os_, od = prep_oracle.add_self_loop_coo(GOLD[p + "src"], GOLD[p + "dst"], V)
        assert eq(os_, s) and eq(od, d)
    for i in range(int(GOLD["n_rule_graphs"])):
        p = "r%d_" % i
        V, R = int(GOLD[p + "V"]), int(GOLD[p + "R"])
        src, dst = off.csr2coo(GOLD[p + "vlist"], GOLD[p + "elist"])
        w = off.gcn_norm_coo_compress(src, dst, GOLD[p + "d"], V, R)
        assert w.dtype == np.float32 and eq(w, GOLD[p + "coo_weight"]) and eq(w, GOLD[p + "weight"])
        assert eq(prep_oracle.gcn_norm_coo_compress(src, dst, GOLD[p + "d"], V, R), w)
        order, phases = off.gen_edge_order(src, dst, V, R)
        assert phases == int(GOLD[p + "edge_phases"]) and order.dtype == np.int32 and eq(order, GOLD[p + "edge_order"])
        o2, p2 = prep_oracle.gen_edge_order(src, dst, V, R)
        assert p2 == phases and eq(o2, order)
        mask, p3 = off.gen_mask_edge(src, dst, V, R)
        assert p3 == phases and mask.dtype == bool and mask.shape == (phases, len(src))
        assert eq(mask.argmax(0), order) and int(mask.sum()) == len(src)
    with pytest.raises(RuntimeError):
        off.gen_edge_order(np.array([2, 3]), np.array([3, 2]), 2, 2)  # two rules feeding each other


@pytest.mark.parametrize("i", range(int(GOLD["n_rule_graphs"])))
def test_compressed_graph_routines_golden(i):
    p = "r%d_" % i
    V, R = int(GOLD[p + "V"]), int(GOLD[p + "R"])
    v, e, d = GOLD[p + "vlist"], GOLD[p + "elist"], GOLD[p + "d"]
    w = off.gcn_norm_csr_compress(v, e, d, V, R)
    assert eq(w, GOLD[p + "weight"]) and eq(prep_oracle.gcn_norm_csr_compress(v, e, d, V, R), w)
    order, depth = off.gen_vertex_order_csr(v, e, V, R)
    assert eq(order, GOLD[p + "order_csr"]) and depth == int(GOLD[p + "depth_csr"])
    order, depth = off.gen_vertex_order_csc(v, e, V, R)
    assert eq(order, GOLD[p + "order_csc"]) and depth == int(GOLD[p + "depth_csc"])
    for thr in (0, 2, 16):
        fv, fe, fV, fR = off.filter_csr(v, e, V, R, thr)
        assert fV == V and fR == int(GOLD[p + "filter%d_R" % thr])
        assert eq(fv, GOLD[p + "filter%d_vlist" % thr]) and eq(fe, GOLD[p + "filter%d_elist" % thr])
        for node in range(V):  # inlining keeps every vertex's ordered expansion
            assert prep_oracle.expand(fv, fe, node, V) == prep_oracle.expand(v, e, node, V)
    for md, me in ((1, 10 ** 6), (2, 10 ** 6), (2, 5), (3, 10 ** 6)):
        key = p + "depth%d_%d_" % (md, me)
        dv, de, dV, dR = off.depth_filter_csr(v, e, V, R, md, me)
        assert dR == int(GOLD[key + "R"]) and eq(dv, GOLD[key + "vlist"]) and eq(de, GOLD[key + "elist"])
    # transpose in the order the partition expects, then partition, levels, degrees
    colptr, row, val = off.csr_transpose(v, e, w, V + R)
    assert eq(colptr, GOLD[p + "t_vlist"]) and eq(row, GOLD[p + "t_elist"]) and eq(val, GOLD[p + "t_value"])
    oc, orow, oval = prep_oracle.csc(v, e, w, V + R)
    assert eq(oc, colptr) and eq(orow, row) and eq(oval, val)
    blocks = off.hybird_partition(colptr, row, val, V)
    oblocks = prep_oracle.hybird_partition(colptr, row, val, V)
    for nm, blk, oblk in zip(["v2v", "v2r", "r2v", "r2r"], blocks, oblocks):
        for part, arr, oarr in zip(("vlist", "elist", "value"), blk, oblk):
            assert eq(arr, GOLD[p + nm + "_" + part]), (nm, part)
            assert eq(oarr, arr)
    levels = off.topo_partition(*blocks[3])
    olevels, order = prep_oracle.topo_partition(*blocks[3])
    assert len(levels) == int(GOLD[p + "levels"]) == len(olevels)
    for k, (lv, olv) in enumerate(zip(levels, olevels)):
        for part, arr, oarr in zip(("vlist", "elist", "value"), lv, olv):
            assert eq(arr, GOLD[p + "lv%d_%s" % (k, part)]) and eq(oarr, arr)
        assert len(lv[0]) == R + 1  # every level carries all row pointers
        for r in range(R):  # rows of level k only read rules of earlier levels
            for c in lv[1][lv[0][r]:lv[0][r + 1]]:
                assert order[c] < k + 1 == order[r]
    vd, rd = off.gen_degree(blocks[0][0], blocks[0][1], blocks[1][0], blocks[1][1], blocks[2][0], blocks[2][1],
                            [lv[0] for lv in levels], [lv[1] for lv in levels])
    assert eq(vd, GOLD[p + "vertex_degree"]) and eq(rd, GOLD[p + "rule_degree"])
    ovd, ord_ = prep_oracle.gen_degree(blocks[0], blocks[1], blocks[2], levels)
    assert eq(ovd, vd) and eq(ord_, rd)


def test_against_compiled_reference_on_fresh_graphs():
    ref = pytest.importorskip("compressgnn_offline_ref")
    for seed in range(3):
        v, e = off.gen_copy_model(3000, 9.0, 0.7, seed)
        sv, se = off.add_self_loop_csr(v, e)
        rv, re_ = ref.add_self_loop_csr(v, e)
        assert eq(sv, rv) and eq(se, re_)
        d = off.get_norm_degree(se, 3000)
        assert eq(d, ref.get_norm_degree(se, 3000))
        cv, ce, V, R = off.compress_csr_batch(sv, se, 2, 12, 3)
        cv, ce = cv.astype(np.int64), ce.astype(np.int64)
        assert R > 0
        fv, fe, _, fR = off.filter_csr(cv, ce, V, R, 4)
        rfv, rfe, _, rfR = ref.filter_csr(cv, ce, V, R, 4)
        assert fR == rfR and eq(fv, rfv) and eq(fe, rfe)
        dv, de, _, dR = off.depth_filter_csr(fv, fe, V, fR, 2, 100000)
        rdv, rde, _, rdR = ref.depth_filter_csr(fv, fe, V, fR, 2, 100000)
        assert dR == rdR and eq(dv, rdv) and eq(de, rde)
        w = off.gcn_norm_csr_compress(dv, de, d, V, dR)
        assert eq(w, ref.gcn_norm_csr_compress(dv, de, d, V, dR))


def check_expansion(rows, packed, ordered=True):
    v, e, n, nr = packed
    assert n == len(rows) and len(v) == n + nr + 1
    assert v[0] == 0 and v[-1] == len(e) and np.all(np.diff(v) >= 0)
    if ordered:
        assert v.dtype == np.int32 and e.dtype == np.int32
    for node, row in enumerate(rows):
        actual = prep_oracle.expand(v, e, node, n)
        assert actual == list(row) if ordered else Counter(actual) == Counter(row)


def test_compressor_keeps_ordered_expansion():
    """The grid of the reference's tests/test_offline_compression.py:28-47 and
    tests/test_batch_compression.py:44-59."""
    rng = np.random.default_rng(73)
    for n in [1, 2, 17, 128]:
        fixtures = [
            [[] for _ in range(n)],
            [[i] for i in range(n)],
            [list(range(min(n, 16))) for _ in range(n)],
            [sorted(rng.choice(n, size=min(n, 20), replace=False).tolist()) for _ in range(n)],
            [sorted(rng.integers(n, size=8).tolist()) for _ in range(n)],
        ]
        for rows in fixtures:
            v = np.array([0] + list(np.cumsum([len(x) for x in rows])), dtype=np.int32)
            e = np.array([j for row in rows for j in row], dtype=np.int32)
            for freq in [3, 4, 16]:
                packed = off.compress_csr_batch(v, e, min_pair_frequency=freq)
                check_expansion(rows, packed)
                filtered = off.filter_csr(*packed, 16)
                check_expansion(rows, filtered, ordered=False)
                depth = off.depth_filter_csr(*filtered, 3, 100000)
                check_expansion(rows, depth, ordered=False)
    rng = np.random.default_rng(17)
    fixtures = [[], [[]], [[0] * 50], [list(range(32)) for _ in range(64)]]
    fixtures += [[rng.integers(32, size=20).tolist() for _ in range(32)] for _ in range(2)]
    for rows in fixtures:
        v = np.array([0] + list(np.cumsum([len(row) for row in rows])), np.int64)
        e = np.array([x for row in rows for x in row], np.int64)
        for freq in [3, 16, 256]:
            check_expansion(rows, off.compress_csr_batch(v, e, 4, 12, freq))
    # 64 identical rows of 32 entries share everything: rules must appear
    rows = [list(range(32)) for _ in range(64)]
    v = np.arange(65, dtype=np.int64) * 32
    e = np.tile(np.arange(32, dtype=np.int64), 64)
    cv, ce, V, R = off.compress_csr_batch(v, e, 4, 12, 16)
    assert R > 0 and len(ce) < len(e) // 4


def test_compressor_rejects_bad_input():
    for freq in [-1, 0, 1, 2]:
        with pytest.raises(ValueError):
            off.compress_csr_batch(np.array([0, 0], np.int32), np.array([], np.int32), min_pair_frequency=freq)
    with pytest.raises(ValueError):
        off.compress_csr_batch(np.array([0, 1], np.int64), np.array([2 ** 32], np.uint64))
    with pytest.raises(ValueError):
        off.compress_csr_batch(np.array([0, 1]), np.array([0.5]))


def test_generators_are_seeded_and_well_formed():
    for gen, args in ((off.gen_chung_lu, (2708, 10500, 2.5)), (off.gen_copy_model, (5000, 9.8, 0.7))):
        v1, e1 = gen(*args, seed=4)
        v2, e2 = gen(*args, seed=4)
        v3, e3 = gen(*args, seed=5)
        assert eq(v1, v2) and eq(e1, e2) and not eq(e1, e3)
        V = len(v1) - 1
        assert v1[0] == 0 and v1[-1] == len(e1) and e1.min() >= 0 and e1.max() < V
        for r in range(0, V, 97):
            row = e1[v1[r]:v1[r + 1]]
            assert np.all(np.diff(row) > 0) and r not in row
    v, e = off.gen_chung_lu(2708, 10500, 2.5, 0)
    assert 0.9 * 10500 < len(e) < 1.1 * 10500
    v, e = off.gen_copy_model(20000, 9.8, 0.7, 0)
    assert 8.5 < len(e) / 20000 < 11.0


def test_row_stats_and_hstack():
    v = np.array([0, 0, 1, 4, 12], np.int64)
    mx, hist = off.csr_row_stats(v)
    assert mx == 8 and hist[0] == 1 and hist[1] == 1 and hist[2] == 1 and hist[4] == 1
    a0 = (np.array([0, 1, 1, 3]), np.array([2, 0, 1]), np.array([1., 2., 3.], np.float32))
    a1 = (np.array([0, 0, 2, 2]), np.array([1, 0]), np.array([4., 5.], np.float32))
    rp, ci, val = off.csr_hstack(a0, a1, 10)
    assert rp.tolist() == [0, 1, 3, 5] and ci.tolist() == [2, 11, 10, 0, 1] and val.tolist() == [1, 4, 5, 2, 3]


def _locality_order_by_hand(vlist, elist, hub_rows=256, work=64):
    """The locality order, restated with plain Python loops: every row is tied to the row it
    shares most columns with (columns listed by more than hub_rows rows do not count; ties
    go to the lower row), ties that close no cycle are kept in row order, and the forest is
    walked depth first, closest relatives first, trees in the lexicographic order of the
    column lists."""
    rows = len(vlist) - 1
    lists = [list(elist[vlist[r]:vlist[r + 1]]) for r in range(rows)]
    users = {}
    for r, cols in enumerate(lists):
        for c in cols:
            users.setdefault(c, []).append(r)
    nnz = sum(len(x) for x in lists)
    while hub_rows > 2 and sum(len(u) ** 2 for u in users.values() if len(u) <= hub_rows) > work * max(nnz, 1):
        hub_rows //= 2
    best, shared = [-1] * rows, [0] * rows
    for r, cols in enumerate(lists):
        count = Counter()
        for c in cols:
            if len(users[c]) <= hub_rows:
                for o in users[c]:
                    if o != r:
                        count[o] += 1
        for o in sorted(count):
            if count[o] > shared[r]:
                best[r], shared[r] = o, count[o]
    root = list(range(rows))

    def find(x):
        while root[x] != x:
            x = root[x]
        return x

    adj = [[] for _ in range(rows)]
    for r in range(rows):
        if best[r] >= 0 and find(r) != find(best[r]):
            root[find(r)] = find(best[r])
            adj[r].append((-shared[r], best[r]))
            adj[best[r]].append((-shared[r], r))
    order, seen = [], [False] * rows
    for start in sorted(range(rows), key=lambda r: (lists[r], r)):
        if seen[start]:
            continue
        stack = [start]
        seen[start] = True
        order.append(start)
        while stack:
            for _, o in sorted(adj[stack[-1]]):
                if not seen[o]:
                    seen[o] = True
                    order.append(o)
                    stack.append(o)
                    break
            else:
                stack.pop()
    return order


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_locality_order_matches_restatement(seed):
    rng = np.random.default_rng(seed)
    rows, cols = [(40, 12), (300, 60), (500, 2000), (700, 90)][seed]
    lens = rng.integers(0, 9, size=rows)
    if seed == 3:
        lens[::7] = 0
    vlist = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    elist = np.concatenate([np.sort(rng.choice(cols, size=n, replace=False)) for n in lens] + [np.zeros(0, np.int64)])
    elist = elist.astype(np.int64)
    if seed == 1:  # a column that more than 256 rows list must not tie rows together
        keep = [np.union1d(elist[vlist[r]:vlist[r + 1]], [0]) for r in range(rows)]
        vlist = np.concatenate([[0], np.cumsum([len(k) for k in keep])]).astype(np.int64)
        elist = np.concatenate(keep).astype(np.int64)
    got = off.csr_locality_order(vlist, elist)
    assert got.dtype == np.int32 and sorted(got.tolist()) == list(range(rows))
    assert got.tolist() == _locality_order_by_hand(vlist, elist)
    assert off.csr_locality_order(vlist, elist).tolist() == got.tolist()


def test_locality_order_limits_its_work():
    """100 rows that all list the same 50 columns would cost 100 steps per non-zero to match:
    the limit on shared columns is halved until those columns no longer count, and the rows
    (which then share nothing but differ in one private column) come out in lexicographic order."""
    rng = np.random.default_rng(8)
    private = rng.permutation(100) + 50
    lists = [np.concatenate([np.arange(50), [private[r]]]) for r in range(100)]
    vlist = np.concatenate([[0], np.cumsum([len(x) for x in lists])]).astype(np.int64)
    elist = np.concatenate(lists).astype(np.int64)
    got = off.csr_locality_order(vlist, elist).tolist()
    assert got == _locality_order_by_hand(vlist, elist)
    assert got == np.argsort(private).tolist()


def test_locality_order_keeps_families_together():
    """Rows with the same column list follow each other when no other row shares a column
    with them; rows that share nothing are in the lexicographic order of their lists."""
    rng = np.random.default_rng(11)
    families = [np.sort(rng.choice(50, size=6, replace=False)) + 50 * k for k in range(30)]
    owner = rng.permutation(np.repeat(np.arange(30), 4))
    lists = [families[k] for k in owner]
    vlist = np.concatenate([[0], np.cumsum([len(x) for x in lists])]).astype(np.int64)
    elist = np.concatenate(lists).astype(np.int64)
    order = off.csr_locality_order(vlist, elist)
    walked = owner[order]
    assert all(len(set(walked[i:i + 4])) == 1 for i in range(0, len(walked), 4))
    firsts = [tuple(families[k]) for k in walked[::4]]
    assert firsts == sorted(firsts)
    # unrelated rows: pure lexicographic order, shorter list first on a common prefix
    vlist = np.array([0, 2, 3, 3, 5, 6], np.int64)
    elist = np.array([7, 9, 4, 6, 8, 2], np.int64)  # rows: [7,9] [4] [] [6,8] [2]
    assert off.csr_locality_order(vlist, elist).tolist() == [2, 4, 1, 3, 0]


def test_fold_levels_equals_the_level_by_level_updates():
    """csr_fold_levels against the dense in-place updates B[r] += sum_c L_k[r, c] B[c], on
    levels shaped like topo_partition's (a level reads only rows it does not write)."""
    rng = np.random.default_rng(21)
    R, Vn = 60, 40
    dense = np.where(rng.random((R, Vn)) < 0.15, rng.standard_normal((R, Vn)), 0.0).astype(np.float32)

    def to_csr(m):
        rp = np.concatenate([[0], np.cumsum((m != 0).sum(1))]).astype(np.int64)
        rows, cols = np.nonzero(m)
        return rp, cols.astype(np.int64), m[rows, cols].astype(np.float32)

    # level k writes rows [20k + 20, 20k + 40) and reads rows below 20k + 20
    levels, want = [], dense.astype(np.float64)
    for k in range(2):
        L = np.zeros((R, R), np.float32)
        lo, hi = 20 * k + 20, 20 * k + 40
        block = np.where(rng.random((hi - lo, lo)) < 0.2, rng.integers(1, 3, (hi - lo, lo)), 0)
        L[lo:hi, :lo] = block
        levels.append(to_csr(L))
        want = want + L.astype(np.float64) @ want
    rp, ci, val = off.csr_fold_levels(to_csr(dense), levels)
    got = np.zeros((R, Vn))
    got[np.repeat(np.arange(R), np.diff(rp)), ci] = val
    assert np.all(np.diff(rp) >= 0) and rp[-1] == len(ci)
    for r in range(R):
        assert np.all(np.diff(ci[rp[r]:rp[r + 1]]) > 0)  # columns ascending, merged
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    # no levels: the block itself
    rp0, ci0, val0 = off.csr_fold_levels(to_csr(dense), [])
    base = to_csr(dense)
    assert np.array_equal(rp0, base[0]) and np.array_equal(ci0, base[1]) and np.array_equal(val0, base[2])
    # a level that reads a row it writes is refused
    bad = np.zeros((R, R), np.float32)
    bad[5, 6] = bad[6, 7] = 1
    with pytest.raises(RuntimeError):
        off.csr_fold_levels(to_csr(dense), [to_csr(bad)])
