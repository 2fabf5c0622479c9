"""Multi-phase propagation over an edge-list (graph_type="coo") compressed graph.

The reference runs one gather + scatter-add per phase (layer/CompressgnnPropagation.py:68-83,
phases from loader/CompressgnnData.py:86-139): out[(V+R) x F] starts at zero, phase 0
gathers from x, phase k >= 1 from out, every phase adds weight * feature[src] into
out[dst]; the result is out[:V].  Here every phase is one CSR product of the HIP kernels:
the edges of a phase are grouped by destination once (stable, so a destination sums its
messages in edge order), and the gradient runs the transposed phases in reverse order.
In the phases the loader makes, a source of phase k receives nothing in phase k, so the
product of a phase k >= 1 accumulates in place.  A phase list from elsewhere may break that;
such a phase (found when the plan is built, on the host) runs as a fresh product followed by
an addition, which is what the reference's gather-then-scatter computes for any phase list.
"""
import _paths  # noqa: F401
import numpy as np
import torch

import compressgnn_runtime as _native
from compressgnn_offline import csr_transpose


class CooPhasePlan:
    """Device CSR blocks of the phases: by destination (forward) and by source (gradient)."""

    def __init__(self, edge_index, edge_weight, vertex_cnt, rule_cnt):
        if len(edge_index) == 0:
            raise ValueError("expected at least one phase")
        if edge_weight is not None and len(edge_weight) != len(edge_index):
            raise ValueError("edge_weight must hold one tensor per phase")
        self.V, self.R = int(vertex_cnt), int(rule_cnt)
        total = self.V + self.R
        device = edge_index[0].device
        if device.type != "cuda":
            raise RuntimeError("multi-phase propagation runs on the GPU only: move the data to a GPU")
        self.device = device
        self.forward_blocks, self.backward_blocks = [], []
        self.in_place = []  # per phase: no node is both a source and a destination of the phase
        # keeps the tensors (and so their addresses) alive for as long as the plan is cached
        self.sources = (list(edge_index), None if edge_weight is None else list(edge_weight))
        t = torch.from_numpy
        for k, edges in enumerate(edge_index):
            if edges.dim() != 2 or edges.size(0) != 2:
                raise ValueError("every phase must be a [2, E] edge tensor")
            src = edges[0].detach().cpu().numpy().astype(np.int64)
            dst = edges[1].detach().cpu().numpy().astype(np.int64)
            w = None
            if edge_weight is not None and edge_weight[k] is not None:
                w = edge_weight[k].detach().cpu().numpy().astype(np.float32)
                if w.shape != src.shape:
                    raise ValueError("edge_weight[%d] must have one value per edge" % k)
            cols = self.V if k == 0 else total  # phase 0 gathers from x
            rows_back = cols
            if src.size and (src.min() < 0 or src.max() >= cols or dst.min() < 0 or dst.max() >= total):
                raise ValueError("phase %d: node id out of range" % k)
            is_src = np.zeros(total, bool)
            is_src[src] = True
            self.in_place.append(not bool(is_src[dst].any()))
            # by source (stable): the transposed block used by the gradient
            by_src = np.argsort(src, kind="stable")
            sp = np.zeros(rows_back + 1, np.int64)
            np.cumsum(np.bincount(src, minlength=rows_back), out=sp[1:])
            s_col, s_val = dst[by_src], None if w is None else w[by_src]
            # by destination, ties in edge order: the forward block
            dp, d_col, d_val = csr_transpose(sp, s_col, s_val, total)
            wt = lambda a: None if a is None else t(np.ascontiguousarray(a))
            self.forward_blocks.append(_native.DeviceCsr(t(dp), t(d_col), wt(d_val), total, cols, device))
            self.backward_blocks.append(_native.DeviceCsr(t(sp), t(np.ascontiguousarray(s_col)), wt(s_val),
                                                          rows_back, total, device))

    def forward(self, x):
        x = x.contiguous()
        if x.dim() != 2 or x.size(0) != self.V:
            raise ValueError("x must be [vertex_cnt, F]")
        out = self.forward_blocks[0].spmm(x)
        for block, in_place in zip(self.forward_blocks[1:], self.in_place[1:]):
            out = block.spmm(out, out) if in_place else out + block.spmm(out)
        return out[:self.V]

    def backward(self, grad):
        grad = grad.contiguous()
        if len(self.backward_blocks) == 1:
            full = grad if self.R == 0 else torch.cat([grad, grad.new_zeros((self.R, grad.size(1)))])
            return self.backward_blocks[0].spmm(full)
        full = torch.cat([grad, grad.new_zeros((self.R, grad.size(1)))])
        for block, in_place in zip(reversed(self.backward_blocks[1:]), reversed(self.in_place[1:])):
            full = block.spmm(full, full) if in_place else full + block.spmm(full)
        return self.backward_blocks[0].spmm(full)


class CooPropagateFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, plan, x):
        ctx.plan = plan
        return plan.forward(x)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad):
        return None, ctx.plan.backward(grad)


class CooPlanCache:
    """Plans keyed by the identity of the phase tensors (addresses, versions, shapes)."""

    def __init__(self, limit=4):
        self.limit = limit
        self.entries = {}

    @staticmethod
    def _key(edge_index, edge_weight, vertex_cnt, rule_cnt):
        sig = lambda t: None if t is None else (t.data_ptr(), t._version, tuple(t.shape), str(t.device))
        weights = () if edge_weight is None else tuple(sig(w) for w in edge_weight)
        return (tuple(sig(e) for e in edge_index), weights, int(vertex_cnt), int(rule_cnt))

    def get(self, edge_index, edge_weight, vertex_cnt, rule_cnt):
        key = self._key(edge_index, edge_weight, vertex_cnt, rule_cnt)
        plan = self.entries.get(key)
        if plan is None:
            if len(self.entries) >= self.limit:
                self.entries.pop(next(iter(self.entries)))
            plan = self.entries[key] = CooPhasePlan(edge_index, edge_weight, vertex_cnt, rule_cnt)
        return plan
