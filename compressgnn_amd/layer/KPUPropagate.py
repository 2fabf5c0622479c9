"""KPUPropagate: K hops per call, optionally remembered.

Constructor (K, cached, keyword arguments of Propagate), reset_cache() and the forward
signature are those of the reference's layer/KPUPropagate.py:9-44.  With cached=True the
features that the first call produces are stored on the module, and every later call
returns that tensor detached from the graph that made it, whatever its arguments, until
reset_cache() is called: meant for models that propagate fixed input features once
(precomputed K-hop features) and train only what comes after.  With cached=False every
call propagates.  The hop itself is Propagate.compressgnn_propagate, so both graph forms
(CompressGraph, per-phase edge lists) work.
"""
import _paths  # noqa: F401
from torch import Tensor

from KPropagate import HopLayer


class KPUPropagate(HopLayer):
    def __init__(self, K: int = 1, cached: bool = False, **kwargs):
        super().__init__(**kwargs)
        self.K, self.cached = K, cached
        self._cached_x = None

    def reset_cache(self):
        self._cached_x = None

    def forward(self, x: Tensor, edge_index, edge_weight=None, vertex_cnt=None, rule_cnt=None) -> Tensor:
        kept = self._cached_x
        if kept is not None:
            return kept.detach()
        out = self.hops(self.K, x, edge_index, edge_weight, vertex_cnt, rule_cnt)
        if self.cached:
            self._cached_x = out
        return out

    def __repr__(self) -> str:
        return '%s(K=%d)' % (type(self).__name__, self.K)
