"""KPropagate: a single hop over a compressed graph (layer/KPropagate.py:15-31 of the
reference; `spmm_impl` is accepted as there and selects nothing).

HopLayer, the common part of KPropagate and KPUPropagate, lives here: both are Propagate
modules that sum weighted copies of the source rows, and differ only in how many hops one
call makes and whether the result is kept.
"""
import _paths  # noqa: F401
from torch import Tensor

from CompressgnnPropagation import Propagate


class HopLayer(Propagate):
    def __init__(self, **kwargs):
        super().__init__(**dict({'aggr': 'add'}, **kwargs))

    def hops(self, count, x, edge_index, edge_weight, vertex_cnt, rule_cnt):
        """`count` propagation steps, each on the output of the one before."""
        for _ in range(count):
            x = self.compressgnn_propagate(x, edge_index, edge_weight, None, vertex_cnt, rule_cnt)
        return x


class KPropagate(HopLayer):
    def __init__(self, spmm_impl: str = "inplace", **kwargs):
        super().__init__(**kwargs)

    def forward(self, x: Tensor, edge_index, edge_weight=None, vertex_cnt=None, rule_cnt=None) -> Tensor:
        return self.hops(1, x, edge_index, edge_weight, vertex_cnt, rule_cnt)
