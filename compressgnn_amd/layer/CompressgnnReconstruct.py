"""Reconstruct node features from representatives, optionally fusing the shared bias
and ReLU (reference layer/CompressgnnReconstruct.py:11-42).  The gradient with respect
to the representatives is a per-cluster sum; it runs on the member lists recorded by
Compressgnn_Cluster for the index tensor when they are available, and builds them on the
fly otherwise."""
import _paths  # noqa: F401
import torch
from torch.autograd.function import once_differentiable

import compressgnn_runtime as _native
from CompressgnnCluster import members_of


class _Reconstruct(torch.autograd.Function):
    @staticmethod
    def forward(ctx, src, index, bias, relu):
        index = index.contiguous()
        ctx.members = members_of(index, src.size(0))
        output = _native.cluster_reconstruct(src.contiguous(), index, None if bias is None else bias.contiguous(),
                                             relu, ctx.members)
        ctx.save_for_backward(index, output)
        ctx.groups, ctx.relu, ctx.has_bias = src.size(0), relu, bias is not None
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        index, output = ctx.saved_tensors
        reps_grad = _native.cluster_reconstruct_backward(grad.contiguous(), index, output, ctx.groups, ctx.relu,
                                                         ctx.members)
        return reps_grad, None, reps_grad.sum(0) if ctx.has_bias else None, None


class Compressgnn_Reconstruct(torch.nn.Module):
    def __init__(self, node_dim=-2):
        super().__init__()
        self.node_dim = node_dim

    def forward(self, src, index, bias=None, activation=None):
        if activation not in (None, 'relu'):
            raise ValueError('Supported activations: None, relu')
        if src.is_cuda and src.dim() == 2 and self.node_dim in (0, -2):
            # the reference takes its fused kernel only when there is a bias or an
            # activation to fuse (layer/CompressgnnReconstruct.py:37); the plain gather
            # is the same kernel here
            return _Reconstruct.apply(src, index, bias, activation == 'relu')
        output = src.index_select(self.node_dim, index)
        if bias is not None:
            output = output + bias
        return output.relu() if activation == 'relu' else output
