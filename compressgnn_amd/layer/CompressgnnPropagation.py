"""Propagate: dispatches a propagation step on the type of edge_index.  Same class,
constructor and method signatures as the reference's layer/CompressgnnPropagation.py:
a CompressGraph runs the compressed CSR chain, a list of [2, E] edge tensors (one per
phase, graph_type="coo") runs the multi-phase form; both end in the HIP SpMM kernels."""
from typing import List, Optional, Union

import _paths  # noqa: F401
import torch
from torch import Tensor

from CompressgnnSPMM import Compressgnn_SPMM
from CooPhases import CooPlanCache, CooPropagateFunction
from compress_graph import CompressGraph
from type import Adj, Size

AGGRS = {'add', 'sum', 'mean', 'min', 'max', 'mul'}


class Propagate(torch.nn.Module):
    def __init__(self, aggr: Optional[Union[str, List[str]]] = 'add', node_dim: int = -2):
        super().__init__()
        if aggr is None or isinstance(aggr, str):
            assert aggr is None or aggr in AGGRS
            self.aggr: Optional[str] = aggr
            self.aggrs: List[str] = []
        else:
            raise ValueError(f"Only strings are vaild aggregation schemes (got '{type(aggr)}')")
        self.node_dim = node_dim
        self.rule_out = None
        self.out = None
        self.SPMM = Compressgnn_SPMM()
        self._coo_plans = CooPlanCache()

    def compressgnn_propagate(self, x: Tensor, edge_index, edge_weight: Optional[List[Tensor]] = None,
                              size: Size = None, vertex_cnt: int = None, rule_cnt: int = None):
        if isinstance(edge_index, CompressGraph):
            out = self.SPMM(edge_index=edge_index, x_j=x)
        elif isinstance(edge_index, (list, tuple)) and len(edge_index) and isinstance(edge_index[0], Tensor):
            # reference layer/CompressgnnPropagation.py:68-83; only sum aggregation with the
            # weighted-copy message of KPropagate exists there and here
            if self.aggr not in ('add', 'sum'):
                raise ValueError("multi-phase propagation supports aggr='add' only")
            if vertex_cnt is None or rule_cnt is None:
                raise ValueError("multi-phase propagation needs vertex_cnt and rule_cnt")
            plan = self._coo_plans.get(edge_index, edge_weight, vertex_cnt, rule_cnt)
            out = CooPropagateFunction.apply(plan, x)
        else:
            raise TypeError("edge_index must be a CompressGraph or a list of [2, E] edge tensors")
        out = self.update(out)
        return out

    def message(self, x_j: Tensor) -> Tensor:
        return x_j

    def update(self, out: Tensor) -> Tensor:
        return out
