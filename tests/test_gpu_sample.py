"""The HIP neighbour sampler (module compressgnn_sample, the device form of the reference's CPU
module of that name) against the CPU oracle on the same graphs, inputs and random streams:
samples, rows and cols are compared exactly.  The oracle is pinned against the compiled
reference in tests/test_oracle_sample.py; here both sides draw from the counter-based
generator with the same seed."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path[:0] = [os.path.join(ROOT, "compressgnn_amd"), os.path.join(ROOT, "compressgnn_amd", "layer"),
                os.path.join(ROOT, "compressgnn_amd", "loader")]

import oracle
from test_oracle_sample import GOLD, _chi2_ok, blocks_of, compressed, golden_blocks, misfit_graph, selection_law

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def on_device(b):
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(DEV)
    return [t(b["v2v"][0]), t(b["v2v"][1]), t(b["v2r"][0]), t(b["v2r"][1]), t(b["r2v"][0]), t(b["r2v"][1]),
            [t(p) for p, _ in b["r2r"]], [t(i) for _, i in b["r2r"]], t(b["v_degree"]), t(b["r_degree"])]


def check(b, dev_blocks, inp, fan, seed):
    import compressgnn_sample as sampler
    want = oracle.neighbor_sample(b, inp, fan, seed=seed)
    got = sampler.neighbor_sample_cg_sim(*dev_blocks, torch.from_numpy(inp).to(DEV), fan, seed=seed)
    assert all(t.dtype == torch.int64 and t.is_cuda for t in got)
    for name, a, w in zip(("samples", "rows", "cols"), got, want):
        assert np.array_equal(a.cpu().numpy(), w), (name, fan, seed)
    return want


@pytest.mark.parametrize("kind", ["blocks", "copy", "chung_lu"])
def test_sampler_matches_oracle(kind):
    data, v, e = compressed(kind)
    b = blocks_of(data.edge_index)
    dev_blocks = on_device(b)
    rng = np.random.default_rng(3)
    V = data.vertex_cnt
    for fan in ([3, 2], [10 ** 6, 10 ** 6], [5, 10 ** 6, 2], [1, 1, 1, 1], [25, 10], [], [0, 4]):
        inp = rng.integers(0, V, size=40).astype(np.int64)
        inp[7] = inp[2]  # a vertex given twice keeps its first position
        samples, rows, cols = check(b, dev_blocks, inp, fan, seed=int(rng.integers(0, 10 ** 9)))
        assert np.array_equal(samples[:len(inp)], inp)
    # every vertex as a seed, one layer: all waves of a large launch
    check(b, dev_blocks, np.arange(V, dtype=np.int64), [4], seed=1)
    check(b, dev_blocks, np.zeros(0, np.int64), [4, 4], seed=1)
    # the CompressGraph front end gives the same result as the raw tensors
    import compressgnn_sample as sampler
    inp = rng.integers(0, V, size=16).astype(np.int64)
    data.edge_index.to(DEV)
    got = sampler.sample_compress_graph(data.edge_index, torch.from_numpy(inp).to(DEV), [6, 3], seed=4)
    want = oracle.neighbor_sample(b, inp, [6, 3], seed=4)
    assert all(np.array_equal(a.cpu().numpy(), w) for a, w in zip(got, want))


def test_sampler_on_deeper_hierarchies():
    """The compressed graphs of the golden fixtures: up to three rule levels, where the breadth-first
    order of a full list and the level-indexed descent of a random position both matter."""
    off = np.load(os.path.join(GOLD, "offline_golden.npz"))
    rng = np.random.default_rng(8)
    for i in range(int(off["n_rule_graphs"])):
        b = golden_blocks(off, i)
        dev_blocks = on_device(b)
        V = len(b["v2v"][0]) - 1
        for fan in ([10 ** 6], [2, 2], [1, 10 ** 6, 3], [4]):
            for _ in range(3):
                inp = rng.integers(0, V, size=int(rng.integers(1, 12))).astype(np.int64)
                check(b, dev_blocks, inp, fan, seed=int(rng.integers(0, 10 ** 9)))
        check(b, dev_blocks, np.arange(V, dtype=np.int64), [10 ** 6, 10 ** 6], seed=0)


def test_degrees_that_do_not_fit_the_hierarchy():
    """Expanded degrees larger than what the descent finds: a random position can then fall
    where the reference would index before a rule's list.  The kernel reports such a position as
    out of range (IndexError, as the reference's out_of_range) exactly when the oracle does and
    agrees with it otherwise; nothing is read outside the arrays."""
    import compressgnn_sample as sampler
    data = misfit_graph()
    b = blocks_of(data.edge_index)
    dev_blocks = on_device(b)
    V = data.vertex_cnt
    misfits = np.array([u for u in range(V) if len(oracle.neighbor_list(b, u)) != b["v_degree"][u]], np.int64)
    assert len(misfits) >= 4
    rng = np.random.default_rng(17)
    raised = agreed = 0
    for case in range(60):
        inp = np.concatenate([rng.choice(misfits, 6), rng.integers(0, V, 10)]).astype(np.int64)
        fan = [int(rng.choice([1, 2, 5])) for _ in range(int(rng.integers(1, 3)))]
        seed = int(rng.integers(0, 2 ** 40))
        try:
            want = oracle.neighbor_sample(b, inp, fan, seed=seed)
        except IndexError:
            want = None
        if want is None:
            with pytest.raises(IndexError, match="out of range"):
                sampler.neighbor_sample_cg_sim(*dev_blocks, torch.from_numpy(inp).to(DEV), fan, seed=seed)
            raised += 1
        else:
            got = sampler.neighbor_sample_cg_sim(*dev_blocks, torch.from_numpy(inp).to(DEV), fan, seed=seed)
            assert all(np.array_equal(a.cpu().numpy(), w) for a, w in zip(got, want)), (fan, seed)
            agreed += 1
    assert raised >= 3 and agreed >= 3, (raised, agreed)
    # full lists (fan-out beyond every degree) never descend by position: same lists as the oracle
    check(b, dev_blocks, np.arange(V, dtype=np.int64), [10 ** 6], seed=2)


def test_plain_form_and_large_fanouts():
    """neighbor_sample_ori_impl: a CSC without rules; rows and cols change roles.  A hub with 6,000
    in-neighbours takes the selection loop beyond the positions a wave keeps in LDS."""
    import compressgnn_sample as sampler
    rng = np.random.default_rng(12)
    V = 7000
    lens = rng.integers(0, 6, size=V)
    lens[5] = 6000
    lens[9] = 0
    colptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    row = rng.integers(0, V, size=int(colptr[-1])).astype(np.int64)
    row[colptr[5]:colptr[6]] = rng.permutation(V)[:6000]
    t = lambda a: torch.from_numpy(a).to(DEV)
    for fan, inp in (([2, 2], np.array([1, 2, 3, 9, 5], np.int64)), ([3000], np.array([5, 9, 5, 0], np.int64)),
                     ([1500, 1], np.array([5], np.int64)), ([10 ** 6], np.arange(0, V, 3, dtype=np.int64))):
        for seed in (0, 77):
            want = oracle.neighbor_sample(dict(v2v=(colptr, row)), inp, fan, seed=seed, plain=True)
            got = sampler.neighbor_sample_ori_impl(t(colptr), t(row), t(inp), fan, seed=seed)
            for a, w in zip(got, want):
                assert np.array_equal(a.cpu().numpy(), w)
    # positions are distinct: 3,000 of the hub's 6,000 distinct in-neighbours, no repeats
    samples, rows, cols = (x.cpu().numpy() for x in sampler.neighbor_sample_ori_impl(t(colptr), t(row), t(np.array([5])), [3000]))
    assert len(rows) == 3000 and len(set(samples[rows])) == 3000 and np.all(cols == 0)


def test_sampled_positions_follow_the_law_of_the_reference_loop():
    """The device sampler's own draws: over 8,000 frontier positions the in-neighbours of a vertex,
    and the pairs of them, are taken with the frequencies the reference's selection loop has under
    independent uniform draws (enumerated exactly, tests/test_oracle_sample.py), in the plain form
    and through the rule hierarchy of a compressed graph; and the result is the oracle's."""
    import compressgnn_sample as sampler
    d, fan, n = 12, 5, 8000
    single, pair = selection_law(d, fan)
    iu = np.triu_indices(d, 1)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(DEV)

    def held_to_the_law(picked, label):
        assert all(len(set(p)) == fan for p in picked)
        ok, stat = _chi2_ok(np.bincount(picked.ravel(), minlength=d), n * single)
        assert ok, (label, "single", stat)
        member = np.zeros((n, d), bool)
        member[np.arange(n)[:, None], picked] = True
        ok, stat = _chi2_ok((member[:, :, None] & member[:, None, :]).sum(0)[iu], n * pair[iu])
        assert ok, (label, "pairs", stat)

    colptr = np.array([0, d] + [d] * d, dtype=np.int64)
    row = np.arange(1, d + 1, dtype=np.int64)
    inp = np.zeros(n, np.int64)
    got = [x.cpu().numpy() for x in sampler.neighbor_sample_ori_impl(t(colptr), t(row), t(inp), [fan], seed=21)]
    want = oracle.neighbor_sample(dict(v2v=(colptr, row)), inp, [fan], seed=21, plain=True)
    for a, w in zip(got, want):
        assert np.array_equal(a, w)
    held_to_the_law(got[0][got[1]].reshape(n, fan) - 1, "plain")
    # a vertex of a compressed graph with 12 expanded in-neighbours: positions resolve through the rules
    data, v, e = compressed("shared_lists")
    b = blocks_of(data.edge_index)
    node = 105
    assert data.rule_cnt > 0 and int(b["v_degree"][node]) == d
    assert b["v2r"][0][node + 1] > b["v2r"][0][node], "the vertex should be reached through rules"
    full = oracle.neighbor_list(b, node)
    assert sorted(full.tolist()) == list(range(11)) + [node]
    inp = np.full(n, node, np.int64)
    got = [x.cpu().numpy() for x in sampler.neighbor_sample_cg_sim(*on_device(b), t(inp), [fan], seed=22)]
    want = oracle.neighbor_sample(b, inp, [fan], seed=22)
    for a, w in zip(got, want):
        assert np.array_equal(a, w)
    # neighbour -> its position in get_neighbor's numbering
    by_position = oracle.get_neighbors(b, np.full(d, node, np.int64), np.arange(d, dtype=np.int64))
    position_of = {int(x): k for k, x in enumerate(by_position)}
    picked = np.array([position_of[int(x)] for x in got[0][got[2]]]).reshape(n, fan)
    held_to_the_law(picked, "compressed")


def test_oversized_fanout_is_refused_not_truncated():
    """A fan-out of 2^31 or more below the degree of a vertex cannot be a count of this layer:
    the call fails (the status the kernels raise), it does not sample fanout mod 2^32."""
    import compressgnn_sample as sampler
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(DEV)
    colptr = np.array([0, 3, 3, 3, 3], dtype=np.int64)
    row = np.array([1, 2, 3], dtype=np.int64)
    # degree 3 <= fan-out: the full list, whatever the size of the fan-out
    samples, rows, cols = sampler.neighbor_sample_ori_impl(t(colptr), t(row), t(np.array([0])), [2 ** 40])
    assert samples.cpu().tolist() == [0, 1, 2, 3]
    data, v, e = compressed("blocks")
    b = blocks_of(data.edge_index)
    huge = dict(b)
    huge["v_degree"] = np.asarray(b["v_degree"]).copy()
    huge["v_degree"][0] = 2 ** 33  # claims more neighbours than any fan-out below
    with pytest.raises((RuntimeError, IndexError)):
        sampler.neighbor_sample_cg_sim(*on_device(huge), t(np.array([0])), [2 ** 32 + 1])


def test_sampler_errors():
    import compressgnn_sample as sampler
    data, v, e = compressed("blocks")
    b = blocks_of(data.edge_index)
    dev_blocks = on_device(b)
    inp = torch.tensor([1, 2, 3], device=DEV)
    with pytest.raises(RuntimeError):
        sampler.neighbor_sample_cg_sim(*dev_blocks, inp.cpu(), [2])              # CPU tensor
    with pytest.raises(RuntimeError):
        sampler.neighbor_sample_cg_sim(*dev_blocks, inp.to(torch.int32), [2])    # wrong dtype
    with pytest.raises(RuntimeError):
        sampler.neighbor_sample_cg_sim(*dev_blocks, inp, [-1])                   # negative fan-out
    with pytest.raises(RuntimeError):
        sampler.neighbor_sample_cg_sim(*dev_blocks, torch.tensor([1, data.vertex_cnt], device=DEV), [2])  # no such vertex
    with pytest.raises(RuntimeError):
        sampler.neighbor_sample_cg_sim(*dev_blocks[:6], dev_blocks[6] + [dev_blocks[4]], dev_blocks[7], *dev_blocks[8:],
                                       inp, [2])                                 # levels mismatch
    # degrees that promise more than the rules hold: the reference throws out_of_range (IndexError)
    lying = dict(b, v_degree=b["v_degree"] + 5, r_degree=b["r_degree"].copy())
    with_rules = np.nonzero(np.diff(b["v2r"][0]))[0][:4].astype(np.int64)
    worst = int(lying["v_degree"][with_rules].max())
    with pytest.raises(IndexError):
        oracle.neighbor_sample(lying, with_rules, [worst - 1], seed=2)
    with pytest.raises(IndexError):
        sampler.neighbor_sample_cg_sim(*on_device(lying), torch.from_numpy(with_rules).to(DEV), [worst - 1], seed=2)
    # the device is fine afterwards
    check(b, dev_blocks, np.array([1, 2, 3], np.int64), [2, 2], seed=3)
