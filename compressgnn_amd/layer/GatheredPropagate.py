"""Propagation of rows that are gathered from cluster representatives.

In the reference's models a layer ends with Compressgnn_Reconstruct, which writes
rows[i] = reps[index[i]] + bias (layer/CompressgnnReconstruct.py:34-42), and the next layer
begins with a propagation that gathers those rows (layer/CompressgnnPropagation.py:62-67,
model/compressgnn/gcn.py:27-31,53-58).  An element-wise activation in between commutes with
the gather: relu(reps[index] + bias) = relu(reps + bias)[index].  GatheredPropagate takes the
small matrix and the index instead of the [N, F] rows and propagates as if the rows had been
written: the column numbers of the graph blocks are sent through the index once per
assignment, and the kernels then gather from the representatives (a few MB that stay in the
caches) instead of an N x F matrix that would be written once and gathered with most of its
accesses missing.  Same sums in the same order as KPropagate on the written rows: same bits,
forward and gradient.  This layer has no counterpart in the reference (its layers hand each
other dense tensors); models that keep the reference's layer sequence do not need it.

    reps, index = cluster(x)                       # Compressgnn_Cluster
    hidden = F.linear(reps, weight, None)
    small = (hidden + bias).relu()                 # the rows Reconstruct + relu would give, per cluster
    out = GatheredPropagate()(small, index, graph) # = KPropagate()(small[index], graph, ...)
"""
import _paths  # noqa: F401
import torch
from torch.autograd.function import once_differentiable

import compressgnn_runtime as _native
from CompressgnnCluster import members_of
from compress_graph import CompressGraph


class _PropagateGathered(torch.autograd.Function):
    """(graph, representatives [C, F], index [V]) -> A * representatives[index]  [V, F]"""

    @staticmethod
    def forward(ctx, graph, reps, index):
        out = graph.plan().forward_gathered(reps.contiguous(), index)
        ctx.graph, ctx.groups = graph, reps.size(0)
        ctx.save_for_backward(index)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        (index,) = ctx.saved_tensors
        # the gradient of the rows, then its sum over the members of every cluster: the backward
        # passes of the propagation and of the gather, one after the other
        d_rows = ctx.graph.plan().backward(grad.contiguous())
        d_reps = _native.cluster_reconstruct_backward(d_rows, index, d_rows, ctx.groups, False,
                                                      members_of(index, ctx.groups))
        return None, d_reps, None


class GatheredPropagate(torch.nn.Module):
    def forward(self, reps, index, edge_index):
        if not isinstance(edge_index, CompressGraph):
            raise TypeError("GatheredPropagate runs over a CompressGraph")
        if reps.dim() != 2 or not reps.is_cuda:
            raise RuntimeError("the representatives must be a [clusters, F] matrix on the GPU")
        if index.dim() != 1 or index.numel() != edge_index.vertex_cnt:
            raise ValueError("the index must name a cluster for every vertex of the graph")
        return _PropagateGathered.apply(edge_index, reps, index)
