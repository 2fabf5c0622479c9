"""Node features from cluster representatives: out[i] = act(src[index[i]] + bias).

Module Compressgnn_Reconstruct with the call signature of the reference's
layer/CompressgnnReconstruct.py:29-42.  On the GPU the gather, the bias and the ReLU are
one kernel; the gradient for the representatives is a per-cluster sum of the (masked)
output gradient, taken over the member lists that Compressgnn_Cluster recorded for the
index tensor, or over lists built on the spot for an index from elsewhere.  The bias
gradient is the column sum of that (layer/CompressgnnReconstruct.py:26).
"""
import _paths  # noqa: F401
import torch
from torch.autograd.function import once_differentiable

import compressgnn_runtime as _native
from CompressgnnCluster import members_of

_ACTIVATIONS = (None, 'relu')


def _dense(t):
    return None if t is None else t.contiguous()


class _GatherBiasAct(torch.autograd.Function):
    """(representatives[C, F], ids[N], bias[F] or None, relu) -> rows[N, F]"""

    @staticmethod
    def forward(ctx, reps, ids, bias, relu):
        ids = _dense(ids)
        lists = members_of(ids, reps.size(0))
        # The ReLU mask of the gradient is kept as one bit per element, written by the kernel that
        # produces the rows (the reference keeps the rows themselves, :16-22); without a ReLU
        # nothing of the [N, F] output is needed again.  Either way none of it is kept.
        if relu:
            rows, signs = _native.cluster_reconstruct_signs(_dense(reps), ids, _dense(bias), lists)
            ctx.save_for_backward(ids, signs)
        else:
            rows = _native.cluster_reconstruct(_dense(reps), ids, _dense(bias), False, lists)
            ctx.save_for_backward(ids)
        ctx.plan = (reps.size(0), relu, bias is not None, lists)
        return rows

    @staticmethod
    @once_differentiable
    def backward(ctx, d_rows):
        clusters, relu, with_bias, lists = ctx.plan
        d_rows = _dense(d_rows)
        if relu:
            ids, signs = ctx.saved_tensors
            d_reps = _native.cluster_reconstruct_backward_signs(d_rows, ids, signs, clusters, lists)
        else:
            (ids,) = ctx.saved_tensors
            # the operator wants a tensor of the shape of the output; without a ReLU it is not read
            d_reps = _native.cluster_reconstruct_backward(d_rows, ids, d_rows, clusters, False, lists)
        return d_reps, None, (d_reps.sum(0) if with_bias else None), None


class Compressgnn_Reconstruct(torch.nn.Module):
    def __init__(self, node_dim=-2):
        super().__init__()
        self.node_dim = node_dim

    def _kernel_applies(self, src):
        # rows along the first axis of a matrix that lives on the GPU
        return src.is_cuda and src.dim() == 2 and self.node_dim in (0, -2)

    def forward(self, src, index, bias=None, activation=None):
        if activation not in _ACTIVATIONS:
            raise ValueError("activation must be None or 'relu'")
        relu = activation is not None
        if self._kernel_applies(src):
            # one kernel with or without bias / activation (the reference switches to its
            # fused kernel only when there is something to fuse, :37)
            return _GatherBiasAct.apply(src, index, bias, relu)
        # anything else (other layouts, host tensors) is plain tensor algebra
        rows = src.index_select(self.node_dim, index)
        rows = rows if bias is None else rows + bias
        return rows.relu() if relu else rows
