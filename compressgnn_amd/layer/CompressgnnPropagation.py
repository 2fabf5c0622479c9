"""Propagate: one propagation step, chosen by what edge_index is.

A CompressGraph (graph_type="csr") goes through the compressed CSR chain; a list of
[2, E] edge tensors, one per phase (graph_type="coo"), goes through the multi-phase form.
Both end in the HIP SpMM kernels.  Class name, constructor and the signatures of
compressgnn_propagate / message / update follow the reference's
layer/CompressgnnPropagation.py:26-99, which its KPropagate and KPUPropagate subclass.
"""
from typing import List, Optional, Union

import _paths  # noqa: F401
import torch
from torch import Tensor

from CompressgnnSPMM import Compressgnn_SPMM
from CooPhases import CooPlanCache, CooPropagateFunction
from compress_graph import CompressGraph
from type import Size

# the names the reference accepts for `aggr`; the kernels here sum
AGGRS = frozenset(('add', 'sum', 'mean', 'min', 'max', 'mul'))
_SUMS = ('add', 'sum')


def _is_phase_list(edge_index):
    return isinstance(edge_index, (list, tuple)) and len(edge_index) > 0 and isinstance(edge_index[0], Tensor)


class Propagate(torch.nn.Module):
    def __init__(self, aggr: Optional[Union[str, List[str]]] = 'add', node_dim: int = -2):
        super().__init__()
        if aggr is not None and not isinstance(aggr, str):
            raise ValueError("aggr must be a string or None, got %s" % type(aggr).__name__)
        assert aggr is None or aggr in AGGRS, "unknown aggregation %r" % (aggr,)
        self.aggr, self.aggrs = aggr, []
        self.node_dim = node_dim
        self.rule_out = self.out = None  # attributes of the reference's class; nothing is parked here
        self.SPMM = Compressgnn_SPMM()
        self._coo_plans = CooPlanCache()

    def compressgnn_propagate(self, x: Tensor, edge_index, edge_weight: Optional[List[Tensor]] = None,
                              size: Size = None, vertex_cnt: int = None, rule_cnt: int = None):
        if isinstance(edge_index, CompressGraph):
            return self.update(self.SPMM(edge_index=edge_index, x_j=x))
        if not _is_phase_list(edge_index):
            raise TypeError("edge_index must be a CompressGraph or a list of [2, E] edge tensors")
        # The phases of layer/CompressgnnPropagation.py:68-83: gather, weight, scatter-add per
        # phase.  The reference has this form for sums of weighted copies only; so has this.
        if self.aggr not in _SUMS:
            raise ValueError("multi-phase propagation supports aggr='add' only")
        if vertex_cnt is None or rule_cnt is None:
            raise ValueError("multi-phase propagation needs vertex_cnt and rule_cnt")
        plan = self._coo_plans.get(edge_index, edge_weight, vertex_cnt, rule_cnt)
        return self.update(CooPropagateFunction.apply(plan, x))

    def propagate(self, edge_index, x: Tensor, edge_weight: Optional[Tensor] = None, size: Size = None):
        """One hop over an uncompressed graph given as a [2, E] edge tensor: out[dst] += weight * x[src]
        (the edge-tensor branch of layer/CompressgnnPropagation.py:50-60: gather, message, scatter-add,
        update), as one product of the HIP kernels over the edges grouped by destination, ties in edge
        order.  The reference's other branch takes a torch_sparse SparseTensor, which this build
        does not depend on."""
        if not isinstance(edge_index, Tensor):
            raise TypeError("propagate() takes a [2, E] edge tensor; compressed graphs go through compressgnn_propagate()")
        if self.aggr not in _SUMS:
            raise ValueError("propagate() supports aggr='add' only")
        weights = None if edge_weight is None else [edge_weight]
        plan = self._coo_plans.get([edge_index], weights, x.size(0), 0)
        return self.update(CooPropagateFunction.apply(plan, x))

    def message(self, x_j: Tensor) -> Tensor:
        return x_j

    def update(self, out: Tensor) -> Tensor:
        return out
