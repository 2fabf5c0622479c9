"""Propagate: dispatches a propagation step on the type of edge_index.  Same class,
constructor and method signatures as the reference's layer/CompressgnnPropagation.py;
the CompressGraph (CSR) branch is the one this build implements."""
from typing import List, Optional, Union

import _paths  # noqa: F401
import torch
from torch import Tensor

from CompressgnnSPMM import Compressgnn_SPMM
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

    def compressgnn_propagate(self, x: Tensor, edge_index, edge_weight: Optional[List[Tensor]] = None,
                              size: Size = None, vertex_cnt: int = None, rule_cnt: int = None):
        if isinstance(edge_index, CompressGraph):
            out = self.SPMM(edge_index=edge_index, x_j=x)
        else:
            raise NotImplementedError(
                "multi-phase COO propagation (a list of edge_index tensors) is not part of this build; "
                "build the data with graph_type='csr'")
        out = self.update(out)
        return out

    def message(self, x_j: Tensor) -> Tensor:
        return x_j

    def update(self, out: Tensor) -> Tensor:
        return out
