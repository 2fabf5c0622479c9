"""Compressed-graph propagation out = A^T-style SpMM over a CompressGraph:
rule aggregation (r2v), rule levels in place (r2r), vertex aggregation (v2r + v2v),
and the transposed chain for the gradient.  Same names and call signatures as the
reference's layer/CompressgnnSPMM.py; every product runs in the HIP kernels behind
compressgnn_runtime (there is no CPU path here: CPU tensors raise)."""
import _paths  # noqa: F401
import torch
from torch import Tensor

from compressgnn_runtime import spmm_func
from compress_graph import CompressGraph


def _gpu_spmm(vlist, elist, value, x, out, prefer_row=False):
    """One CSR product on int64 CSR tensors (reference layer/CompressgnnSPMM.py:14-19).
    The schedule is chosen from the block's row lengths instead of from
    (prefer_row, nnz, width); prefer_row is accepted and ignored."""
    return spmm_func(vlist, elist, value, x, "auto", out)


def _check(graph, x):
    if not isinstance(graph, CompressGraph):
        raise TypeError("expected a CompressGraph")
    if not x.is_cuda:
        raise RuntimeError("compressed propagation runs on the GPU only: move the features and the graph "
                           "to a GPU (data.to('cuda'))")
    if graph.device != x.device:
        raise RuntimeError("graph is on %s but features are on %s" % (graph.device, x.device))


def compress_spmm(graph, x_j):
    """Forward propagation without autograd (reference layer/CompressgnnSPMM.py:21-39)."""
    _check(graph, x_j)
    return graph.plan().forward(x_j)


class Compressgnn_SPMM_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, graph, x_j):
        _check(graph, x_j)
        out = graph.plan().forward(x_j)
        ctx.graph = graph
        return out

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        graph = ctx.graph
        grad_output = grad_output.contiguous()
        return None, graph.plan().backward(grad_output)


class Compressgnn_SPMM(torch.nn.Module):
    def __init__(self):
        super(Compressgnn_SPMM, self).__init__()

    def forward(self, edge_index: CompressGraph, x_j: Tensor) -> Tensor:
        return Compressgnn_SPMM_Function.apply(edge_index, x_j)
