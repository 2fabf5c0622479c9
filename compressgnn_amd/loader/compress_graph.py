"""CompressGraph: the on-device format of a compressed graph -- three CSR blocks
(vertex->vertex, vertex->rule, rule->vertex), the rule->rule levels, and expanded
degrees.  Same fields, constructor and to() as the reference's
loader/compress_graph.py:6-57; on a GPU it additionally carries the propagation plan
(int32 index arrays, rows of non-zeros, transposes) that the HIP kernels read."""
from concurrent.futures import ThreadPoolExecutor

import _paths  # noqa: F401
import numpy as np
import torch

from compressgnn_offline import (csr_fold_levels, csr_fold_levels_bound, csr_hstack, csr_locality_order, csr_permute_rows, gen_degree,
                                 hybird_partition, topo_partition)
from sparse_csr import SparseCSR


class CompressGraph():
    def __init__(self, vlist, elist, value, vertex_cnt):
        """vlist/elist/value: CSC of the (vertex_cnt + rule_cnt)-square compressed matrix,
        i.e. row i lists the parents of node i, vertex parents first."""
        as_np = lambda t: t.detach().cpu().numpy() if torch.is_tensor(t) else t
        v2v, v2r, r2v, r2r = hybird_partition(as_np(vlist), as_np(elist), as_np(value), vertex_cnt)
        r2r_list = topo_partition(r2r[0], r2r[1], r2r[2])
        rule_cnt = len(r2v[0]) - 1
        t = torch.from_numpy
        self.vertex_cnt, self.rule_cnt = int(vertex_cnt), int(rule_cnt)
        self.v2v_graph = SparseCSR(t(v2v[0]), t(v2v[1]), t(v2v[2]), (vertex_cnt, vertex_cnt))
        self.v2r_graph = SparseCSR(t(v2r[0]), t(v2r[1]), t(v2r[2]), (vertex_cnt, rule_cnt))
        self.r2v_graph = SparseCSR(t(r2v[0]), t(r2v[1]), t(r2v[2]), (rule_cnt, vertex_cnt))
        self.step = len(r2r_list)
        self.r2r_graph = [SparseCSR(t(lv[0]), t(lv[1]), t(lv[2]), (rule_cnt, rule_cnt)) for lv in r2r_list]
        vertex_degree, rule_degree = gen_degree(v2v[0], v2v[1], v2r[0], v2r[1], r2v[0], r2v[1],
                                                [lv[0] for lv in r2r_list], [lv[1] for lv in r2r_list])
        self.vertex_degree = t(vertex_degree)
        self.rule_degree = t(rule_degree)
        # The rule levels are folded into the rule stage when the device plan is built: the
        # rules then aggregate all the vertices they stand for in one launch, forward and
        # backward, instead of one more launch per level (the same sums in another order).
        # Set to False before plan() for the launch-per-level form of the reference.
        self.fold_levels = True
        self.levels_folded = False       # what plan() decided
        self.keep_split_blocks = False   # plan(): also build the four vertex-stage blocks on their own
        self.keep_device_blocks = False  # plan(): leave the int64 blocks on the device
        self._plan = None
        self._stage_orders = None        # the locality orders of the two vertex stages, once a plan has found them

    def __repr__(self):
        return 'CompressGraph'

    # torch.save(data) of a prepared dataset, as the reference's genData scripts do
    # (genData/createCompressDataset.py:98): the blocks are saved, the device plan is not
    # (it is rebuilt on first use after loading).
    def __getstate__(self):
        state = dict(self.__dict__)
        state['_plan'] = None
        state.pop('_sampler_blocks', None)
        return state

    def __setstate__(self, state):
        self.__dict__.update(state)
        self._plan = None

    def blocks(self):
        return [self.v2v_graph, self.v2r_graph, self.r2v_graph] + list(self.r2r_graph)

    def to(self, device):
        device = torch.device(device)
        # the transposes for the backward pass are built where the blocks live: on the GPU
        # after a move there (plan()), by the host library otherwise
        self.v2v_graph = self.v2v_graph.to(device)
        self.v2r_graph = self.v2r_graph.to(device)
        self.r2v_graph = self.r2v_graph.to(device)
        for s in range(self.step):
            self.r2r_graph[s] = self.r2r_graph[s].to(device)
        self.vertex_degree = self.vertex_degree.to(device)
        self.rule_degree = self.rule_degree.to(device)
        self._plan = None
        self._sampler_blocks = None
        return self

    @property
    def device(self):
        return self.v2v_graph.device

    # Folding the levels multiplies out the rule hierarchy: a rule row grows to all the vertices
    # it stands for, which a deep hierarchy can make exponentially many.  The levels are folded
    # only while the folded rule stage stays within this multiple of the entries of the blocks
    # it replaces (r2v or v2r plus the levels) and the hierarchy is no deeper than max_fold_depth;
    # beyond that the plan keeps one launch per level, the reference's form.
    max_fold_growth = 4.0
    max_fold_depth = 16

    def _fold_plan(self, host):
        """(forward base, forward levels, backward base, backward levels) on the host when the
        levels are to be folded into the rule stage, else None."""
        if not getattr(self, "fold_levels", True) or self.step == 0:
            return None
        if self.step > self.max_fold_depth:
            return None
        fwd_base, fwd_levels = host(self.r2v_graph.csr()), [host(g.csr()) for g in self.r2r_graph]
        bwd_base, bwd_levels = host(self.v2r_graph.csc()), [host(g.csc()) for g in reversed(self.r2r_graph)]
        for base, levels in ((fwd_base, fwd_levels), (bwd_base, bwd_levels)):
            stored = len(base[1]) + sum(len(lv[1]) for lv in levels)
            if csr_fold_levels_bound(base, levels) > self.max_fold_growth * max(stored, 1):
                return None
        return fwd_base, fwd_levels, bwd_base, bwd_levels

    def plan(self):
        """The device-side propagation plan (built on first use after to(device))."""
        if self._plan is None:
            import compressgnn_runtime as rt
            dev = self.device
            if dev.type != "cuda":
                raise RuntimeError("CompressGraph.plan(): move the graph to a GPU first (graph.to('cuda'))")

            # Runs of 32 non-zeros for the graph blocks (the nnz schedule's default of 64 is
            # tuned for the member lists of clusters): measured 2 % faster on the web graph.
            seg = 32
            # The rule stage is a small launch (a few waves per SIMD) whose time is the chain of loads of
            # a run, not its traffic: runs of 16 shorten the chain (16 features: 20 -> 16 us, 128: 32 -> 31).
            rule_seg = 16

            def fwd(g):
                rp, ci, val = g.csr()
                return rt.DeviceCsr(rp, ci, val, g.sparse_size(0), g.sparse_size(1), dev, seg)

            def bwd(g):
                cp, row, val = g.csc()
                return rt.DeviceCsr(cp, row, val, g.sparse_size(1), g.sparse_size(0), dev, seg)

            def level(rp, ci, val, rows, cols):
                """A rule level as the device reads it: only the rows that have entries (the rules
                of that level; the reference pads every level to all R rule rows,
                src/offline/csrc/partition.h:175-203), each with the rule row it updates."""
                rp = rp.cpu()
                lens = rp[1:] - rp[:-1]
                live = torch.nonzero(lens).flatten()
                packed = torch.zeros(live.numel() + 1, dtype=rp.dtype)
                packed[1:] = torch.cumsum(lens[live], 0)
                return rt.DeviceCsr(packed, ci, val, live.numel(), cols, dev, seg, live, rows)

            V, R = self.vertex_cnt, self.rule_cnt
            host = lambda triple: tuple(t.cpu().numpy() for t in triple)
            t = torch.from_numpy
            folded = self._fold_plan(host)
            self.levels_folded = folded is not None
            if folded is not None:
                # forward: rule_out = (I + L_last) ... (I + L_0) r2v x; backward, with the
                # transposed levels in reverse order: rule_g = (I + L_0^T) ... (I + L_last^T) v2r^T g
                rp, ci, val = csr_fold_levels(folded[0], folded[1])
                rules_fwd = rt.DeviceCsr(t(rp), t(ci), t(val), R, V, dev, rule_seg)
                rp, ci, val = csr_fold_levels(folded[2], folded[3])
                rules_bwd = rt.DeviceCsr(t(rp), t(ci), t(val), R, V, dev, seg)
                plan = rt.PropagationPlan(V, R, rules_fwd, [], rules_bwd, [])
            else:
                plan = rt.PropagationPlan(V, R, fwd(self.r2v_graph), [level(*g.csr(), R, R) for g in self.r2r_graph],
                                          bwd(self.v2r_graph), [level(*g.csc(), R, R) for g in self.r2r_graph])
            if getattr(self, "keep_split_blocks", False):
                # the vertex stages as two launches each (plan.fuse_final = False)
                plan.set_split_blocks(fwd(self.v2v_graph), fwd(self.v2r_graph), bwd(self.v2v_graph), bwd(self.r2v_graph))
            # the vertex stage reads [v2v | v2r] (forward) and [v2v^T | r2v^T] (backward) in one pass
            # Both vertex stages store their rows in a locality order (rows that gather the same
            # rows of the input follow each other and are processed on one XCD), which cuts
            # the misses in the per-XCD L2 caches; results do not depend on the order in the
            # row schedule, and in the nnz schedule only where a long row is cut into runs.
            # The search for an order is the expensive part of a plan (most of 22 s at 18.5 M vertices)
            # and depends on the blocks alone, so the graph keeps the two orders: a later plan() -- after
            # another to(device), or after the dataset was saved and loaded -- only applies them.
            kept = getattr(self, "_stage_orders", None) or {}

            def ordered(which, first, second):
                rp, ci, val = csr_hstack(first, second, V)
                order = kept.get(which)
                if order is None or len(order) != len(rp) - 1:
                    order = np.ascontiguousarray(csr_locality_order(rp, ci), dtype=np.int32)
                return csr_permute_rows(rp, ci, val, order) + (order,)

            def stage(rp, ci, val, order):
                return rt.DeviceCsr(t(rp), t(ci), t(val), V, V + R, dev, seg, t(order))

            # The two orders are host work with serial stretches (the host library releases the
            # interpreter lock while it runs), so they are computed side by side.
            forward_blocks = (host(self.v2v_graph.csr()), host(self.v2r_graph.csr()))
            backward_blocks = (host(self.v2v_graph.csc()), host(self.r2v_graph.csc()))
            # From here on the kernels read the plan's own int32 arrays: the int64 blocks go
            # back to host memory (csr()/csc() still deliver device tensors, as copies), so the
            # device holds the graph once.  keep_device_blocks = True keeps them resident.
            if not getattr(self, "keep_device_blocks", False):
                for block in self.blocks():
                    block.offload()
            with ThreadPoolExecutor(max_workers=2) as pool:
                forward_job = pool.submit(ordered, "forward", *forward_blocks)
                backward_job = pool.submit(ordered, "backward", *backward_blocks)
                forward_stage, backward_stage = forward_job.result(), backward_job.result()
                self._stage_orders = {"forward": forward_stage[3], "backward": backward_stage[3]}
                plan.set_vertex_stages(stage(*forward_stage), stage(*backward_stage))
            self._plan = plan
        return self._plan
