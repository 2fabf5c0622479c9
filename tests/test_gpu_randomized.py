"""Seeded randomized parity sweep over the operator module.  Each case draws shapes, graph
generators, compression settings and schedules at random and compares the GPU result with the CPU
oracle (or with the host routine that is itself pinned against the compiled reference), to the bars
of the fixed-grid tests: bit-exact for integer work, for rows and clusters inside one run and across
the two forms of an operator; the float tolerance of the task (1e-5 relative, 1e-6 absolute) on
normalised weights; where sums of 10^3..10^5 terms re-associate beyond that, the bar that can fail:
no further from the float64 result than the oracle's sequential fp32 sum.  Seeds are fixed, so a
failure names a case that can be run again.  (A sweep of this kind found the out-of-range descent
that tests/test_gpu_sample.py::test_degrees_that_do_not_fit_the_hierarchy now pins.)"""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "compressgnn_amd"), os.path.join(ROOT, "compressgnn_amd", "layer"),
          os.path.join(ROOT, "compressgnn_amd", "loader"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import oracle
from compressgnn_amd import abi
from util import assert_compression_contract, closed_form_transpose

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def pick(rng, values):
    return values[int(rng.integers(0, len(values)))]


def random_csr(rng, rows, cols, mean, hubs, dtype=np.float32):
    deg = rng.poisson(mean, rows).astype(np.int64)
    for _ in range(hubs):
        deg[rng.integers(0, rows)] = rng.integers(100, 5000)
    if rng.random() < 0.3:
        deg[rng.integers(0, rows, max(1, rows // 7))] = 0
    deg = np.minimum(deg, cols * 3)
    vlist = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    elist = np.concatenate([np.sort(rng.integers(0, cols, d)) for d in deg] + [np.zeros(0, np.int64)]).astype(np.int64)
    row_len = np.repeat(deg, deg)
    value = (rng.standard_normal(len(elist)) * 0.5 / np.sqrt(np.maximum(row_len, 1))).astype(dtype)
    return vlist, elist, value


def sweep(seed, cases, one_case):
    rng = np.random.default_rng(seed)
    failures = []
    for _ in range(cases):
        one_case(rng, lambda params, msg: failures.append("%s: %s" % (params, msg)))
    assert not failures, "\n".join(failures)


# --------------------------------------------------------------------- blocks ----------

def block_case(rng, fail):
    """A block built through the operator module (row lists for the fix-up pass, optional stored row
    order, any method string, fresh or accumulating) against the oracle and against the C-ABI form
    of the same block, after the shared scratch has been filled with NaN carries."""
    import compressgnn_offline as off
    import compressgnn_runtime as rt
    rows = pick(rng, [1, 5, 63, 64, 65, 300, 2047, 2049, 9000, 30000])
    cols = pick(rng, [1, 17, 500, 5000])
    F = pick(rng, [1, 2, 4, 6, 8, 12, 16, 32, 48, 64, 100, 128, 130, 256, 300, 512])
    mean, hubs = pick(rng, [0.5, 3.0, 12.0, 40.0]), pick(rng, [0, 0, 1, 4])
    seg = pick(rng, [0, 8, 30, 32, 64, 256])
    method = pick(rng, ["row_schedule", "nnz_schedule", "auto", "rowbalance", "nnzbalance_rowcache"])
    acc, use_map = bool(rng.random() < 0.4), bool(rng.random() < 0.4)
    params = dict(rows=rows, cols=cols, F=F, mean=mean, hubs=hubs, seg=seg, method=method, acc=acc, use_map=use_map)
    vlist, elist, value = random_csr(rng, rows, cols, mean, hubs)
    x = rng.standard_normal((cols, F)).astype(np.float32)
    out0 = rng.standard_normal((rows, F)).astype(np.float32) if acc else None
    want = oracle.spmm(vlist, elist, value, x, None if out0 is None else out0.copy())
    sv, se, sval, rowmap = vlist, elist, value, None
    if use_map:
        order = rng.permutation(rows).astype(np.int32)
        sv, se, sval = off.csr_permute_rows(vlist, elist, value, order)
        rowmap = t(order)
    A = rt.DeviceCsr(t(sv), t(se), t(sval), rows, cols, DEV, seg, rowmap)
    X = t(x)
    A.spmm(torch.full_like(X, float("nan")), torch.zeros(rows, F, device=DEV) if acc else None, method)
    got = A.spmm(X, t(out0.copy()) if acc else None, method).cpu().numpy()
    if not np.isfinite(got).all():
        return fail(params, "a carry that this call did not write was read")
    err = np.abs(got - want) / np.maximum(np.abs(want), 1.0)
    if err.size and err.max() > 3e-5:
        return fail(params, "error %g" % err.max())
    plain = abi.DeviceCsr.from_host(rows, cols, sv, se, sval, DEV, seg_nnz=seg,
                                    rowmap=None if rowmap is None else rowmap.cpu())
    kern = {"row_schedule": abi.SPMM_ROW, "nnz_schedule": abi.SPMM_NNZ}.get(method, abi.SPMM_AUTO)
    got2 = abi.spmm(plain, X, t(out0.copy()) if acc else None, acc, kern).cpu().numpy()
    if not np.array_equal(got, got2):
        fail(params, "the block with row lists and the block without give different bits")


def test_blocks():
    sweep(101, 120, block_case)


def block_f64_case(rng, fail):
    rows, cols = pick(rng, [5, 300, 9000]), pick(rng, [17, 500, 5000])
    F = pick(rng, [1, 2, 3, 16, 33, 64, 128, 256])
    mean, hubs = pick(rng, [0.5, 3.0, 12.0, 40.0]), pick(rng, [0, 1, 4])
    kern, acc = pick(rng, [abi.SPMM_ROW, abi.SPMM_NNZ, abi.SPMM_AUTO]), bool(rng.random() < 0.4)
    params = dict(rows=rows, cols=cols, F=F, mean=mean, hubs=hubs, kern=kern, acc=acc)
    vlist, elist, value = random_csr(rng, rows, cols, mean, hubs, np.float64)
    x = rng.standard_normal((cols, F))
    out0 = rng.standard_normal((rows, F)) if acc else None
    want = oracle.spmm(vlist, elist, value, x, None if out0 is None else out0.copy())
    A = abi.DeviceCsr.from_host(rows, cols, vlist, elist, value, DEV, seg_nnz=pick(rng, [0, 8, 32]))
    got = abi.spmm(A, t(x), t(out0.copy()) if acc else None, acc, kern)
    if not np.allclose(got.cpu().numpy(), want, rtol=1e-12, atol=1e-12):
        return fail(params, "error %g" % np.abs(got.cpu().numpy() - want).max())
    if not acc:
        try:
            same = abi.spmm_static(A, t(x), torch.empty(rows, F, dtype=torch.float64, device=DEV), False, kern)
        except abi.CgnnError as refusal:  # a product beyond the built-in scratch is refused by name
            assert "built-in array" in str(refusal)
            return
        if not torch.equal(same, got):
            fail(params, "the entry point with built-in scratch gives different bits")


def test_blocks_in_double_precision():
    sweep(102, 60, block_f64_case)


# ------------------------------------------------------------- propagation plans -------

def plan_case(rng, fail):
    """KPropagate over a random compressed graph (generator, size, width, merging frequency, filters,
    folded or launch-per-level rule stage) against the oracle's four-stage chain, forward and gradient."""
    import compressgnn_offline as off
    from CompressgnnData import CompressgnnData
    from KPropagate import KPropagate
    from test_gpu_layers import _np_blocks
    V, kind = pick(rng, [40, 300, 2708, 6000, 15000]), pick(rng, ["copy", "chung_lu"])
    F = pick(rng, [1, 3, 16, 64, 100, 128, 256, 512])
    freq, thr, depth = pick(rng, [3, 4, 8, 16]), pick(rng, [0, 4, 16]), pick(rng, [1, 3, 8])
    params = dict(V=V, kind=kind, F=F, freq=freq, thr=thr, depth=depth)
    s = int(rng.integers(0, 1000))
    v, e = off.gen_copy_model(V, 9.8, 0.7, s) if kind == "copy" else off.gen_chung_lu(V, V * 4, 2.5, s)
    x = rng.standard_normal((V, F)).astype(np.float32)
    m = np.ones(V, bool)
    data = CompressgnnData(x, (v, e), np.zeros(V, np.int64), m, m, m, add_self_loop=True, normalize=True, graph_type="csr",
                           min_pair_frequency=freq, threshold=thr, max_depth=depth, min_edge=0, verbose=False)
    graph = data.edge_index
    fwd_blocks, bwd_blocks = _np_blocks(graph)
    want = oracle.compress_spmm_forward(fwd_blocks, x) if data.rule_cnt else oracle.spmm(*fwd_blocks["v2v"], x)
    data.to(DEV)
    graph.max_fold_growth = pick(rng, [0.0, 4.0, 100.0])
    xd = data.x.detach().clone().requires_grad_()
    out = KPropagate()(xd, graph, None, data.vertex_cnt, data.rule_cnt)
    g_np = rng.standard_normal(out.shape).astype(np.float32)
    (gx,) = torch.autograd.grad(out, xd, t(g_np))
    want_gx = (oracle.compress_spmm_backward(bwd_blocks, g_np) if data.rule_cnt
               else oracle.spmm(*bwd_blocks["v2v_t"], g_np))
    for name, got, w in (("forward", out.detach().cpu().numpy(), want), ("gradient", gx.cpu().numpy(), want_gx)):
        over = np.abs(got - w) - (1e-6 + 1e-5 * np.abs(w))
        if not np.isfinite(got).all() or over.max() > 2e-6:
            fail(dict(params, rules=data.rule_cnt, levels=graph.step, folded=graph.levels_folded),
                 "%s beyond 1e-5 / 1e-6 by %g" % (name, over.max()))


def test_propagation_plans():
    sweep(103, 50, plan_case)


def coo_case(rng, fail):
    """The multi-phase edge-list form of a graph against its CompressGraph form."""
    import compressgnn_offline as off
    from CompressgnnData import CompressgnnData
    from KPropagate import KPropagate
    V, F = pick(rng, [40, 300, 2708, 9000]), pick(rng, [1, 16, 64, 100, 128])
    freq, normalize = pick(rng, [3, 4, 16]), bool(rng.random() < 0.7)
    params = dict(V=V, F=F, freq=freq, normalize=normalize)
    s = int(rng.integers(0, 1000))
    v, e = off.gen_copy_model(V, 9.8, 0.7, s) if rng.random() < 0.5 else off.gen_chung_lu(V, V * 4, 2.5, s)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g_np = rng.standard_normal((V, F)).astype(np.float32)
    m = np.ones(V, bool)
    src, dst = off.csr2coo(v, e)
    both = []
    for form, edges in (("csr", (v, e)), ("coo", (src, dst))):
        data = CompressgnnData(x, edges, np.zeros(V, np.int64), m, m, m, add_self_loop=True, normalize=normalize,
                               graph_type=form, min_pair_frequency=freq, verbose=False).to(DEV)
        xd = data.x.detach().clone().requires_grad_()
        out = KPropagate()(xd, data.edge_index, data.edge_weight if form == "coo" else None, data.vertex_cnt, data.rule_cnt)
        (gx,) = torch.autograd.grad(out, xd, t(g_np))
        both.append((out.detach().cpu().numpy(), gx.cpu().numpy()))
    for name, a, b in (("forward", both[0][0], both[1][0]), ("gradient", both[0][1], both[1][1])):
        scale = max(1.0, float(np.abs(a).max()))
        if not np.isfinite(b).all() or np.abs(a - b).max() > (2e-5 if normalize else 2e-4) * scale:
            fail(params, "%s of the two forms differ by %g" % (name, np.abs(a - b).max()))


def test_edge_list_form_against_block_form():
    sweep(104, 30, coo_case)


# ------------------------------------------------------------- cluster operators -------

def pack_signs(out):
    n, width = out.shape
    words = (width + 31) // 32
    bits = np.zeros((n, words * 32), dtype=np.uint64)
    bits[:, :width] = ~(out <= 0)
    return (bits.reshape(n, words, 32) << np.arange(32, dtype=np.uint64)).sum(axis=2).astype(np.uint32).view(np.int32)


def cluster_case(rng, fail):
    import compressgnn_runtime as rt
    n = pick(rng, [1, 2, 63, 64, 65, 255, 1000, 4097, 30000, 120000])
    width = pick(rng, [1, 3, 4, 7, 16, 31, 32, 33, 64, 100, 128, 250, 256, 512, 602])
    bits, centres = pick(rng, [0, 1, 3, 8, 12, 16, 17, 20, 24]), pick(rng, [1, 3, 47, 1000])
    params = dict(n=n, width=width, bits=bits, centres=centres)
    c = rng.standard_normal((centres, width)).astype(np.float32) * 2
    spread = pick(rng, [0.0, 0.1, 1.0])
    x = (c[rng.integers(0, centres, n)] + rng.standard_normal((n, width)).astype(np.float32) * spread).astype(np.float32)
    w = rng.standard_normal((width, bits)).astype(np.float32)
    want_ids, want_counts, want_active = oracle.assign(x, w, bits)
    X = t(x)
    ids, counts, active, members = rt.cluster_assign_members(X, t(w), bits)
    if (active != want_active or not np.array_equal(ids.cpu().numpy(), want_ids)
            or not np.array_equal(counts.cpu().numpy(), want_counts)):
        return fail(params, "ids, counts or the number of clusters differ")
    order = np.argsort(want_ids, kind="stable")
    if not np.array_equal(members[1].cpu().numpy(), order.astype(np.int32)):
        return fail(params, "member lists are not the stable order by id")
    if not np.array_equal(members[0].cpu().numpy(), np.concatenate([[0], np.cumsum(want_counts)]).astype(np.int32)):
        return fail(params, "offsets of the member lists differ")
    groups = active + 1
    for a, b in zip(rt.cluster_members(ids, groups)[:3], members[:3]):
        if not torch.equal(a, b):
            return fail(params, "cluster_members disagrees with the lists of the assignment")
    small = want_counts <= 64
    reps = rt.cluster_mean(X, ids, counts, members).cpu().numpy()
    want_reps = oracle.cluster_mean(x, want_ids, want_counts)
    if not np.array_equal(reps[small], want_reps[small]):
        return fail(params, "means of clusters of at most 64 members are not bit-exact")
    if not np.allclose(reps, want_reps, rtol=1e-4, atol=1e-5):
        truth = oracle.cluster_mean(x.astype(np.float64), want_ids, want_counts)
        if np.abs(reps - truth).max() > 1.5 * np.abs(want_reps - truth).max() + 1e-7:
            return fail(params, "means further from float64 than the sequential sum")
    hidden = rng.standard_normal((groups, width)).astype(np.float32)
    bias = rng.standard_normal(width).astype(np.float32)
    want_out = oracle.reconstruct(hidden, want_ids, bias, True)
    H, B = t(hidden), t(bias)
    for lists in (None, members):
        rows, signs = rt.cluster_reconstruct_signs(H, ids, B, lists)
        if not np.array_equal(rows.cpu().numpy(), want_out):
            return fail(params, "reconstructed rows differ")
        if not np.array_equal(signs.cpu().numpy(), pack_signs(want_out)):
            return fail(params, "sign words differ")
        if not torch.equal(rt.cluster_reconstruct(H, ids, B, True, lists), rows):
            return fail(params, "the two forms of reconstruct differ")
    go = rng.standard_normal((n, width)).astype(np.float32)
    G = t(go)
    by_rows = rt.cluster_reconstruct_backward(G, ids, rows, groups, True, members)
    if not torch.equal(by_rows, rt.cluster_reconstruct_backward_signs(G, ids, signs, groups, members)):
        return fail(params, "the two forms of the reconstruct gradient differ")
    by_rows = by_rows.cpu().numpy()
    want_rg = oracle.reconstruct_backward(go, want_ids, want_out, groups, True)
    if not np.array_equal(by_rows[small], want_rg[small]):
        return fail(params, "reconstruct gradients of clusters of at most 64 members are not bit-exact")
    if not np.allclose(by_rows, want_rg, rtol=1e-4, atol=2e-5):
        truth = oracle.reconstruct_backward(go.astype(np.float64), want_ids, want_out.astype(np.float64), groups, True)
        if np.abs(by_rows - truth).max() > 1.5 * np.abs(want_rg - truth).max() + 1e-7:
            return fail(params, "reconstruct gradient further from float64 than the sequential sum")
    dx = rt.cluster_mean_backward(H, ids, counts, members).cpu().numpy()
    if not np.array_equal(dx, oracle.cluster_mean_backward(hidden, want_ids, want_counts)):
        fail(params, "mean gradient differs")


def test_cluster_operators():
    sweep(105, 60, cluster_case)


# ------------------------------------------------------------------- the sampler -------

def sampler_case(rng, fail):
    """Random compressed graphs (deep hierarchies included), inputs with repeats, fan-outs from 0 to
    beyond every degree: the same samples, rows and cols as the oracle, or IndexError where it raises."""
    import compressgnn_offline as off
    import compressgnn_sample as sampler
    from CompressgnnData import CompressgnnData
    from test_oracle_sample import blocks_of
    V = pick(rng, [30, 500, 6000, 20000])
    freq, thr, depth = pick(rng, [3, 4, 16]), pick(rng, [0, 4, 16]), pick(rng, [1, 3, 8])
    params = dict(V=V, freq=freq, thr=thr, depth=depth)
    v, e = off.gen_copy_model(V, pick(rng, [3.0, 9.8, 30.0]), 0.7, int(rng.integers(0, 1000)))
    m = np.ones(V, bool)
    data = CompressgnnData(np.zeros((V, 1), np.float32), (v, e), np.zeros(V, np.int64), m, m, m,
                           add_self_loop=bool(rng.random() < 0.5), normalize=False, graph_type="csr",
                           min_pair_frequency=freq, threshold=thr, max_depth=depth, min_edge=0, verbose=False)
    b = blocks_of(data.edge_index)
    i64 = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(DEV)
    dev = [i64(b["v2v"][0]), i64(b["v2v"][1]), i64(b["v2r"][0]), i64(b["v2r"][1]), i64(b["r2v"][0]), i64(b["r2v"][1]),
           [i64(p) for p, _ in b["r2r"]], [i64(i) for _, i in b["r2r"]], i64(b["v_degree"]), i64(b["r_degree"])]
    for _ in range(4):
        fan = [pick(rng, [0, 1, 2, 5, 25, 1500, 10 ** 6]) for _ in range(int(rng.integers(0, 4)))]
        inp = rng.integers(0, V, size=pick(rng, [0, 1, 7, 200, min(V, 5000)])).astype(np.int64)
        seed = int(rng.integers(0, 2 ** 40))
        case = dict(params, fan=fan, n=len(inp), seed=seed, rules=data.rule_cnt, levels=data.edge_index.step)
        try:
            want = oracle.neighbor_sample(b, inp, fan, seed=seed)
        except IndexError:
            want = None
        try:
            got = sampler.neighbor_sample_cg_sim(*dev, i64(inp), fan, seed=seed)
        except IndexError:
            got = None
        if (got is None) != (want is None):
            fail(case, "out of range for %s only" % ("the kernel" if got is None else "the oracle"))
        elif got is not None:
            for name, a, w in zip(("samples", "rows", "cols"), got, want):
                if not np.array_equal(a.cpu().numpy(), w):
                    fail(case, name + " differ")
                    break


def test_sampler():
    sweep(106, 400, sampler_case)


# ------------------------------------------------- graph preparation on the GPU --------

def merger_case(rng, fail):
    """The rule merger on the GPU against the host merger: the same arrays."""
    import compressgnn_batch_cuda as gpu
    import compressgnn_offline as off
    kind, V = pick(rng, ["copy", "chung_lu", "rows", "repeats"]), pick(rng, [1, 2, 17, 300, 5000, 40000])
    rounds, freq = pick(rng, [1, 3, 12, 20]), pick(rng, [3, 4, 8, 16])
    params = dict(kind=kind, V=V, rounds=rounds, freq=freq)
    s = int(rng.integers(0, 1000))
    if kind == "copy" and V >= 17:
        v, e = off.gen_copy_model(V, pick(rng, [3.0, 9.8, 25.0]), pick(rng, [0.3, 0.7, 0.95]), s)
    elif kind == "chung_lu" and V >= 17:
        v, e = off.gen_chung_lu(V, V * 5, 2.5, s)
    else:
        nr = min(V, 3000)
        if kind == "repeats":  # long stretches of one value: chains of overlapping pairs
            rows = [rng.integers(0, max(1, min(nr, 6)), size=int(rng.integers(0, 60))).tolist() for _ in range(nr)]
        else:
            rows = [sorted(rng.integers(0, nr, size=int(rng.integers(0, 24))).tolist()) for _ in range(nr)]
        v = np.array([0] + list(np.cumsum([len(r) for r in rows])), np.int64)
        e = np.array([j for r in rows for j in r], np.int64)
    if kind in ("copy", "chung_lu") and V >= 17 and rng.random() < 0.5:
        v, e = off.add_self_loop_csr(v, e)
    want = off.compress_csr_batch(v, e, 4, rounds, freq)
    got = gpu.compress_csr_batch(v, e, rounds=rounds, min_pair_frequency=freq)
    try:  # the reference's contract at this boundary, on the GPU's arrays directly
        assert_compression_contract(v, e, got)
    except AssertionError as exc:
        return fail(params, "contract of the compressor boundary broken: %s" % exc)
    if not (got[2] == want[2] and got[3] == want[3] and np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])):
        fail(params, "%d rules on the GPU, %d on the host" % (got[3], want[3]))


def test_rule_merger():
    sweep(107, 80, merger_case)


def transpose_case(rng, fail):
    import compressgnn_offline as off
    import compressgnn_runtime as rt
    rows, cols = pick(rng, [1, 7, 300, 5000, 70000]), pick(rng, [1, 3, 300, 5000, 70000])
    mean, dup = pick(rng, [0.3, 2.0, 9.0, 30.0]), bool(rng.random() < 0.5)
    params = dict(rows=rows, cols=cols, mean=mean, dup=dup)
    lens = rng.poisson(mean, size=rows)
    if rng.random() < 0.5:
        lens[rng.integers(0, rows)] = int(rng.integers(0, 20000))
    elist = rng.integers(0, cols, size=int(lens.sum())).astype(np.int64)
    vlist = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    if not dup:
        elist = np.concatenate([np.sort(elist[vlist[r]:vlist[r + 1]]) for r in range(rows)]
                               + [np.zeros(0, np.int64)]).astype(np.int64)
    value = rng.standard_normal(len(elist)).astype(np.float32)
    want = closed_form_transpose(vlist, elist, value, cols)  # numpy's stable sort by column: no product code
    for a, w in zip(rt.csr_transpose(t(vlist), t(elist), t(value), cols), want):
        if not np.array_equal(a.cpu().numpy(), w):
            return fail(params, "not the stable sort by column")
    for a, w in zip(off.csr_transpose(vlist, elist, value, cols), want):
        if not np.array_equal(a, w):
            return fail(params, "host transpose: not the stable sort by column")


def test_transposes():
    sweep(108, 80, transpose_case)
