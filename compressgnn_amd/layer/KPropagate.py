"""One propagation hop (reference layer/KPropagate.py:15-31)."""
import _paths  # noqa: F401
from torch import Tensor

from CompressgnnPropagation import Propagate
from type import OptTensor


class KPropagate(Propagate):
    def __init__(self, spmm_impl: str = "inplace", **kwargs):
        kwargs.setdefault('aggr', 'add')
        super().__init__(**kwargs)

    def forward(self, x: Tensor, edge_index, edge_weight=None, vertex_cnt=None, rule_cnt=None) -> Tensor:
        return self.compressgnn_propagate(edge_index=edge_index, x=x, edge_weight=edge_weight,
                                          vertex_cnt=vertex_cnt, rule_cnt=rule_cnt, size=None)

    def message(self, x_j: Tensor, edge_weight: OptTensor) -> Tensor:
        return x_j if edge_weight is None else edge_weight.view(-1, 1) * x_j
