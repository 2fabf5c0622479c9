"""SparseCSR: the small part of torch_sparse.SparseTensor that the CompressGNN loader and
layers use (reference loader/compress_graph.py:21-35, layer/CompressgnnSPMM.py:22-24,68-70):
a CSR container with csr(), csc(), to() and sparse_sizes().  csc() orders entries by
column, then row, ties in storage order -- the order SparseTensor.csc() produces.  A block
that lives on a GPU is transposed there (stable radix sort by column); a block on the
host by the host library.  Both give the same arrays.

offload(): a block that belongs to a GPU can keep its int64 arrays in host memory; csr() and
csc() then upload a copy per call.  CompressGraph does that once its propagation plan (int32
arrays of its own) is built, so that the device holds the graph once."""
import _paths  # noqa: F401
import numpy as np
import torch

import compressgnn_offline as offline


class SparseCSR:
    def __init__(self, rowptr, col, value=None, sparse_sizes=None):
        self._rowptr = torch.as_tensor(rowptr).to(torch.int64)
        self._col = torch.as_tensor(col).to(torch.int64)
        self._value = None if value is None else torch.as_tensor(value)
        rows = self._rowptr.numel() - 1
        if sparse_sizes is None:
            cols = int(self._col.max()) + 1 if self._col.numel() else 0
            sparse_sizes = (rows, cols)
        if sparse_sizes[0] != rows:
            raise ValueError("rowptr does not match sparse_sizes")
        self._sizes = (int(sparse_sizes[0]), int(sparse_sizes[1]))
        self._csc = None
        self._device = self._rowptr.device  # where csr()/csc() deliver; the arrays may rest on the host

    def sparse_sizes(self):
        return self._sizes

    def sparse_size(self, dim):
        return self._sizes[dim]

    def nnz(self):
        return self._col.numel()

    @property
    def device(self):
        return self._device

    @property
    def offloaded(self):
        return self._rowptr.device != self._device

    def _deliver(self, triple):
        return tuple(None if t is None else t.to(self._device) for t in triple)

    def csr(self):
        return self._deliver((self._rowptr, self._col, self._value))

    def offload(self):
        """Keep the arrays (and the transpose, once made) in host memory; the block still
        belongs to its device and csr()/csc() deliver there."""
        host = lambda t: None if t is None else t.cpu()
        self._rowptr, self._col, self._value = host(self._rowptr), host(self._col), host(self._value)
        if self._csc is not None:
            self._csc = tuple(host(t) for t in self._csc)
        return self

    def csc(self):
        """(colptr, row, value) of the same matrix, i.e. the CSR of its transpose."""
        if self._csc is None and self._rowptr.device.type == "cuda":
            import compressgnn_runtime as rt
            value = self._value
            if value is not None and value.dtype not in (torch.float32, torch.float64):
                value = value.to(torch.float32)
            colptr, row, tval = rt.csr_transpose(self._rowptr, self._col, value, self._sizes[1])
            if tval is not None and tval.dtype != self._value.dtype:
                tval = tval.to(self._value.dtype)
            self._csc = (colptr, row, tval)
        if self._csc is None:
            dev = self._rowptr.device
            rp = self._rowptr.cpu().numpy()
            ci = self._col.cpu().numpy()
            val = None if self._value is None else self._value.detach().cpu().numpy().astype(np.float32)
            colptr, row, tval = offline.csr_transpose(rp, ci, val, self._sizes[1])
            tv = None
            if tval is not None:
                tv = torch.from_numpy(tval).to(self._value.dtype).to(dev)
            self._csc = (torch.from_numpy(colptr).to(dev), torch.from_numpy(row).to(dev), tv)
        return self._deliver(self._csc)

    def t(self):
        colptr, row, value = self.csc()
        return SparseCSR(colptr, row, value, (self._sizes[1], self._sizes[0]))

    def to(self, device):
        out = SparseCSR.__new__(SparseCSR)
        out._rowptr = self._rowptr.to(device)
        out._col = self._col.to(device)
        out._value = None if self._value is None else self._value.to(device)
        out._sizes = self._sizes
        out._device = out._rowptr.device
        out._csc = None if self._csc is None else tuple(None if t is None else t.to(device) for t in self._csc)
        return out

    def __repr__(self):
        return "SparseCSR(sizes=%s, nnz=%d, device=%s)" % (self._sizes, self.nnz(), self.device)
