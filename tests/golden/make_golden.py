#!/usr/bin/env python3
"""Writes the golden fixtures of this directory from the reference's own compiled CPU
code (oracle/_ref, built by `make -C oracle ref` where the reference checkout exists):

  spmm_golden.npz      outputs of the reference's spmm_func ("rowbalance") on seeded CSR
                       blocks: fresh output, accumulation onto an existing output, and
                       the in-place case where the output is the gathered matrix
  cluster_golden.npz   (index, active) of the reference's cluster_forward on inputs whose
                       projections are exactly representable, so that the result does
                       not depend on the order in which a dot product is summed
  offline_golden.npz   outputs of the reference's add_self_loop_csr, get_norm_degree,
                       gcn_norm_csr_compress, hybird_partition, topo_partition,
                       gen_degree, filter_csr, depth_filter_csr, gen_vertex_order_csr/csc
                       on seeded compressed graphs (inputs are stored with the outputs)

  sample_golden.npz    (samples, rows, cols) of the reference's neighbor_sample_cg_sim and
                       neighbor_sample_ori_impl on the compressed graphs of offline_golden.npz
                       (their blocks and expanded degrees are read from that file), with the
                       seed of torch's CPU generator the reference drew its random positions
                       from; also which calls raised IndexError (std::out_of_range)

Fixtures hold data only (inputs and expected outputs).  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [os.path.join(ROOT, "oracle", "_ref")]

import torch  # noqa: E402

import compressgnn_offline_ref as off  # noqa: E402
import compressgnn_runtime_ref as rt  # noqa: E402


def random_csr(rng, rows, cols, mean_deg, long_rows=0):
    deg = rng.poisson(mean_deg, size=rows)
    deg[rng.random(rows) < 0.2] = 0
    for r in rng.choice(rows, size=long_rows, replace=False):
        deg[r] = int(rng.integers(100, 400))
    vlist = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    nnz = int(vlist[-1])
    return vlist, rng.integers(0, cols, size=nnz).astype(np.int64), rng.standard_normal(nnz).astype(np.float32)


def make_spmm():
    out = {}
    rng = np.random.default_rng(20240601)
    cases = [(40, 30, 5, 3.0, 0), (64, 64, 33, 6.0, 2), (17, 50, 128, 4.0, 1), (5, 5, 1, 2.0, 0)]
    for i, (rows, cols, F, deg, long_rows) in enumerate(cases):
        vlist, elist, value = random_csr(rng, rows, cols, deg, long_rows)
        x = rng.standard_normal((cols, F)).astype(np.float32)
        t = torch.from_numpy
        fresh = rt.spmm_func(t(vlist), t(elist), t(value), t(x), "rowbalance", None).numpy()
        base = rng.standard_normal((rows, F)).astype(np.float32)
        acc = torch.from_numpy(base.copy())
        rt.spmm_func(t(vlist), t(elist), t(value), t(x), "rowbalance", acc)
        pre = "c%d_" % i
        out.update({pre + "vlist": vlist, pre + "elist": elist, pre + "value": value, pre + "x": x,
                    pre + "fresh": fresh, pre + "base": base, pre + "acc": acc.numpy()})
    # in place: rows 20.. gather rows 0..19 of the same matrix
    deg = np.concatenate([np.zeros(20, np.int64), rng.integers(1, 6, size=20)])
    vlist = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    elist = rng.integers(0, 20, size=int(vlist[-1])).astype(np.int64)
    value = rng.standard_normal(int(vlist[-1])).astype(np.float32)
    z = rng.standard_normal((40, 9)).astype(np.float32)
    zt = torch.from_numpy(z.copy())
    rt.spmm_func(torch.from_numpy(vlist), torch.from_numpy(elist), torch.from_numpy(value), zt, "rowbalance", zt)
    out.update(dict(ip_vlist=vlist, ip_elist=elist, ip_value=value, ip_z=z, ip_out=zt.numpy()))
    # float64
    vlist, elist, value = random_csr(rng, 30, 25, 4.0, 1)
    x = rng.standard_normal((25, 7))
    res = rt.spmm_func(torch.from_numpy(vlist), torch.from_numpy(elist), torch.from_numpy(value.astype(np.float64)),
                       torch.from_numpy(x), "rowbalance", None).numpy()
    out.update(dict(d_vlist=vlist, d_elist=elist, d_value=value.astype(np.float64), d_x=x, d_fresh=res))
    out["n_cases"] = np.array(len(cases))
    np.savez_compressed(os.path.join(HERE, "spmm_golden.npz"), **out)


def make_cluster():
    out = {}
    rng = np.random.default_rng(20240602)
    cases = [(200, 9, 6, 3), (513, 33, 8, 1), (67, 31, 0, 2), (1, 5, 4, 2), (300, 12, 16, 2), (64, 1, 3, 4)]
    for i, (n, width, bits, amp) in enumerate(cases):
        # small integers (and halves): every product and partial sum is exact in float32
        x = (rng.integers(-2 * amp, 2 * amp + 1, size=(n, width)) / 2.0).astype(np.float32)
        w = rng.integers(-amp, amp + 1, size=(width, bits)).astype(np.float32)
        index, active = rt.cluster_forward(torch.from_numpy(x), torch.from_numpy(w), bits)
        pre = "c%d_" % i
        out.update({pre + "x": x, pre + "w": w, pre + "bits": np.array(bits), pre + "index": index.numpy(),
                    pre + "active": np.array(active)})
    # float64 dispatch of the same routine
    x = rng.integers(-5, 6, size=(90, 11)).astype(np.float64)
    w = rng.integers(-3, 4, size=(11, 7)).astype(np.float64)
    index, active = rt.cluster_forward(torch.from_numpy(x), torch.from_numpy(w), 7)
    out.update(dict(d_x=x, d_w=w, d_bits=np.array(7), d_index=index.numpy(), d_active=np.array(active)))
    out["n_cases"] = np.array(len(cases))
    np.savez_compressed(os.path.join(HERE, "cluster_golden.npz"), **out)


def random_rule_graph(rng, V, R, deg, nest=0.3):
    """A compressed CSR over V + R nodes: vertex rows list vertices and rules, rule rows
    list vertices and smaller rules (so the rule graph is acyclic)."""
    rows = []
    for v in range(V):
        k = int(rng.integers(0, deg + 1))
        row = sorted(set(rng.integers(0, V, size=k).tolist()))
        rules = sorted(set(rng.integers(V, V + R, size=int(rng.integers(0, 3))).tolist())) if R else []
        rows.append(row + rules)
    for r in range(R):
        k = int(rng.integers(2, 5))
        row = sorted(set(rng.integers(0, V, size=k).tolist()))
        if r > 0 and rng.random() < nest:
            row += sorted(set(rng.integers(V, V + r, size=int(rng.integers(1, 3))).tolist()))
        rows.append(row)
    # every rule must be referenced at least once
    for r in range(R):
        rid = V + r
        if not any(rid in row for row in rows):
            rows[int(rng.integers(0, V))].append(rid)
    vlist = np.concatenate([[0], np.cumsum([len(x) for x in rows])]).astype(np.int64)
    elist = np.array([c for row in rows for c in row], dtype=np.int64)
    return vlist, elist


def make_offline():
    out = {}
    rng = np.random.default_rng(20240603)
    # plain graphs: self loops and norm degrees
    for i, (V, deg) in enumerate([(1, 0), (12, 3), (60, 5)]):
        rows = [sorted(set(rng.integers(0, V, size=int(rng.integers(0, deg + 1))).tolist())) for _ in range(V)]
        vlist = np.concatenate([[0], np.cumsum([len(r) for r in rows])]).astype(np.int64)
        elist = np.array([c for r in rows for c in r], dtype=np.int64)
        sv, se = off.add_self_loop_csr(vlist, elist)
        nd = off.get_norm_degree(se, V)
        pre = "g%d_" % i
        out.update({pre + "vlist": vlist, pre + "elist": elist, pre + "sl_vlist": sv, pre + "sl_elist": se,
                    pre + "norm_degree": nd})
    out["n_plain"] = np.array(3)
    # compressed graphs: weights, partition, levels, degrees, orders, filters
    graphs = [(20, 0, 4), (30, 6, 4), (50, 14, 5), (80, 25, 6)]
    for i, (V, R, deg) in enumerate(graphs):
        vlist, elist = random_rule_graph(rng, V, R, deg, nest=0.5)
        pre = "r%d_" % i
        out.update({pre + "V": np.array(V), pre + "R": np.array(R), pre + "vlist": vlist, pre + "elist": elist})
        d = (1.0 / np.sqrt(1e-6 + rng.integers(1, 9, size=V))).astype(np.float32)
        w = off.gcn_norm_csr_compress(vlist, elist, d, V, R)
        out.update({pre + "d": d, pre + "weight": w})
        order, depth = off.gen_vertex_order_csr(vlist, elist, V, R)
        out.update({pre + "order_csr": np.asarray(order), pre + "depth_csr": np.array(depth)})
        order, depth = off.gen_vertex_order_csc(vlist, elist, V, R)
        out.update({pre + "order_csc": np.asarray(order), pre + "depth_csc": np.array(depth)})
        for thr in (0, 2, 16):
            fv, fe, fV, fR = off.filter_csr(vlist, elist, V, R, thr)
            out.update({pre + "filter%d_vlist" % thr: np.asarray(fv, np.int64),
                        pre + "filter%d_elist" % thr: np.asarray(fe, np.int64), pre + "filter%d_R" % thr: np.array(fR)})
        for md, me in ((1, 10 ** 6), (2, 10 ** 6), (2, 5), (3, 10 ** 6)):
            dv, de, dV, dR = off.depth_filter_csr(vlist, elist, V, R, md, me)
            key = pre + "depth%d_%d_" % (md, me)
            out.update({key + "vlist": np.asarray(dv, np.int64), key + "elist": np.asarray(de, np.int64),
                        key + "R": np.array(dR)})
        # transpose by (column, row), the order the loader feeds to hybird_partition
        total = V + R
        src = np.repeat(np.arange(total), np.diff(vlist))
        key = np.lexsort((src, elist))
        t_rows = src[key].astype(np.int64)
        t_val = w[key]
        colptr = np.zeros(total + 1, np.int64)
        np.cumsum(np.bincount(elist, minlength=total), out=colptr[1:])
        out.update({pre + "t_vlist": colptr, pre + "t_elist": t_rows, pre + "t_value": t_val})
        blocks = off.hybird_partition(colptr, t_rows, t_val, V)
        names = ["v2v", "v2r", "r2v", "r2r"]
        for nm, blk in zip(names, blocks):
            for part, arr in zip(("vlist", "elist", "value"), blk):
                out[pre + nm + "_" + part] = np.asarray(arr)
        levels = off.topo_partition(*blocks[3])
        out[pre + "levels"] = np.array(len(levels))
        for k, lv in enumerate(levels):
            for part, arr in zip(("vlist", "elist", "value"), lv):
                out[pre + "lv%d_%s" % (k, part)] = np.asarray(arr)
        vd, rd = off.gen_degree(blocks[0][0], blocks[0][1], blocks[1][0], blocks[1][1], blocks[2][0], blocks[2][1],
                                [lv[0] for lv in levels], [lv[1] for lv in levels])
        out.update({pre + "vertex_degree": np.asarray(vd), pre + "rule_degree": np.asarray(rd)})
    out["n_rule_graphs"] = np.array(len(graphs))
    # edge-list (COO) forms: weights and phase order of the compressed graphs above, and
    # self loops on plain sorted edge lists.  (The reference's add_self_loop_coo reads one
    # element past its inputs; the arrays passed are views with a -1 behind the last edge.)
    for i in range(len(graphs)):
        pre = "r%d_" % i
        V, R = int(out[pre + "V"]), int(out[pre + "R"])
        src, dst = off.csr2coo(out[pre + "vlist"], out[pre + "elist"])
        out[pre + "coo_weight"] = np.asarray(off.gcn_norm_coo_compress(src, dst, out[pre + "d"], V, R))
        order, phases = off.gen_edge_order(src, dst, V, R)
        out.update({pre + "edge_order": np.asarray(order), pre + "edge_phases": np.array(phases)})
        mask, phases2 = off.gen_mask_edge(src, dst, V, R)
        assert phases2 == phases and np.array_equal(np.asarray(mask), np.asarray(order)[None, :] == np.arange(phases)[:, None])
    for i, (V, deg) in enumerate([(1, 0), (9, 2), (40, 4), (33, 6)]):
        rows = [sorted(set(rng.integers(0, V, size=int(rng.integers(0, deg + 1))).tolist())) for _ in range(V)]
        src = np.full(sum(len(r) for r in rows) + 1, -1, np.int64)
        dst = src.copy()
        src[:-1] = [v for v, r in enumerate(rows) for _ in r]
        dst[:-1] = [c for r in rows for c in r]
        s, d = off.add_self_loop_coo(src[:-1], dst[:-1], V)
        pre = "c%d_" % i
        out.update({pre + "V": np.array(V), pre + "src": src[:-1].copy(), pre + "dst": dst[:-1].copy(),
                    pre + "sl_src": np.asarray(s), pre + "sl_dst": np.asarray(d)})
    out["n_coo"] = np.array(4)
    np.savez_compressed(os.path.join(HERE, "offline_golden.npz"), **out)


def make_sample():
    import compressgnn_sample_ref as sampler
    g = np.load(os.path.join(HERE, "offline_golden.npz"))
    t = torch.from_numpy
    out, case = {}, 0
    rng = np.random.default_rng(77)
    for i in range(int(g["n_rule_graphs"])):
        pre = "r%d_" % i
        V, levels = int(g[pre + "V"]), int(g[pre + "levels"])
        blocks = [t(g[pre + nm + "_" + part].astype(np.int64)) for nm in ("v2v", "v2r", "r2v") for part in ("vlist", "elist")]
        lv_ptr = [t(g[pre + "lv%d_vlist" % k].astype(np.int64)) for k in range(levels)]
        lv_idx = [t(g[pre + "lv%d_elist" % k].astype(np.int64)) for k in range(levels)]
        vdeg, rdeg = t(g[pre + "vertex_degree"].astype(np.int64)), t(g[pre + "rule_degree"].astype(np.int64))
        for fan in ([2, 2], [10 ** 6], [3, 10 ** 6, 1], [1], []):
            inp = rng.integers(0, V, size=int(rng.integers(1, 9))).astype(np.int64)
            seed = int(rng.integers(0, 10 ** 6))
            key = "s%d_" % case
            out.update({key + "graph": np.array(i), key + "input": inp, key + "fan": np.array(fan, np.int64),
                        key + "seed": np.array(seed), key + "plain": np.array(0)})
            torch.manual_seed(seed)
            try:
                res = sampler.neighbor_sample_cg_sim(*blocks, lv_ptr, lv_idx, vdeg, rdeg, t(inp), fan)
                out.update({key + "raised": np.array(0), key + "samples": res[0].numpy(), key + "rows": res[1].numpy(),
                            key + "cols": res[2].numpy()})
            except IndexError:
                out[key + "raised"] = np.array(1)
            case += 1
        # the plain form on the v2v block alone (a CSC of some graph over the same vertices)
        for fan in ([2, 3], [10 ** 6, 1]):
            inp = rng.integers(0, V, size=5).astype(np.int64)
            seed = int(rng.integers(0, 10 ** 6))
            key = "s%d_" % case
            torch.manual_seed(seed)
            res = sampler.neighbor_sample_ori_impl(blocks[0], blocks[1], t(inp), fan)
            out.update({key + "graph": np.array(i), key + "input": inp, key + "fan": np.array(fan, np.int64),
                        key + "seed": np.array(seed), key + "plain": np.array(1), key + "raised": np.array(0),
                        key + "samples": res[0].numpy(), key + "rows": res[1].numpy(), key + "cols": res[2].numpy()})
            case += 1
    out["n_cases"] = np.array(case)
    np.savez_compressed(os.path.join(HERE, "sample_golden.npz"), **out)


if __name__ == "__main__":
    make_spmm()
    make_cluster()
    make_offline()
    make_sample()
    for f in ("spmm_golden.npz", "cluster_golden.npz", "offline_golden.npz", "sample_golden.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
