"""Typing aliases used by the layer modules (the subset of the reference's layer/type.py
that its propagation layers import)."""
from typing import List, Optional, Tuple, Union

import _paths  # noqa: F401
from torch import Tensor

from sparse_csr import SparseCSR

Adj = Union[Tensor, SparseCSR]
OptTensor = Optional[Tensor]
Size = Optional[Tuple[int, int]]
__all__ = ["Adj", "OptTensor", "Size", "List"]
