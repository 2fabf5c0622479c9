"""The on-GPU CSR -> CSC transpose against the order mathematics fixes (a stable sort of the
entries by column: what SparseTensor.csc() gives, reference layer/CompressgnnSPMM.py:68-70),
computed here with numpy alone, and against the host library's transpose beside it."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "compressgnn_amd"))
sys.path.insert(0, os.path.join(ROOT, "compressgnn_amd", "loader"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def random_block(rng, rows, cols, mean, duplicates=False):
    lens = rng.poisson(mean, size=rows)
    if rows > 3:
        lens[rows // 2] = 0
        lens[0] = min(cols, 40) if not duplicates else 40
    vlist = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    if duplicates:  # unsorted rows with repeated columns: ties must keep storage order
        elist = rng.integers(0, max(cols, 1), size=int(vlist[-1])).astype(np.int64)
    else:
        elist = np.concatenate([np.sort(rng.choice(cols, size=min(n, cols), replace=False)) for n in lens]
                               + [np.zeros(0, np.int64)]).astype(np.int64)
        vlist = np.concatenate([[0], np.cumsum([min(n, cols) for n in lens])]).astype(np.int64)
    value = rng.standard_normal(len(elist)).astype(np.float32)
    return vlist, elist, value


@pytest.mark.parametrize("rows,cols,mean,dup", [(1, 1, 1.0, False), (7, 3, 2.0, True), (300, 5000, 6.0, False),
                                                (5000, 300, 4.0, True), (40000, 40000, 9.0, False)])
def test_device_transpose_matches_host(rows, cols, mean, dup):
    import compressgnn_runtime as rt
    from compressgnn_amd import abi
    from compressgnn_amd import compressgnn_offline as off
    rng = np.random.default_rng(rows * 7 + cols)
    vlist, elist, value = random_block(rng, rows, cols, mean, dup)
    from util import closed_form_transpose
    want = closed_form_transpose(vlist, elist, value, cols)
    for a, b in zip(off.csr_transpose(vlist, elist, value, cols), want):  # the host routine, beside it
        assert np.array_equal(a, b)
    t = lambda a: torch.from_numpy(a).to(DEV)
    for impl in (rt.csr_transpose, abi.csr_transpose):
        colptr, row, tval = impl(t(vlist), t(elist), t(value), cols)
        assert colptr.dtype == torch.int64 and row.dtype == torch.int64 and tval.dtype == torch.float32
        assert np.array_equal(colptr.cpu().numpy(), want[0])
        assert np.array_equal(row.cpu().numpy(), want[1])
        assert np.array_equal(tval.cpu().numpy(), want[2])
        colptr, row, none = impl(t(vlist), t(elist), None, cols)
        assert none is None and np.array_equal(row.cpu().numpy(), want[1])
    # 8-byte values travel as they are
    colptr, row, tval = rt.csr_transpose(t(vlist), t(elist), t(value.astype(np.float64)), cols)
    assert tval.dtype == torch.float64 and np.array_equal(tval.cpu().numpy(), want[2].astype(np.float64))


def test_device_transpose_edge_cases():
    import compressgnn_runtime as rt
    z = torch.zeros(0, dtype=torch.int64, device=DEV)
    colptr, row, val = rt.csr_transpose(torch.zeros(5, dtype=torch.int64, device=DEV), z, None, 3)
    assert colptr.tolist() == [0, 0, 0, 0] and row.numel() == 0 and val is None
    colptr, row, val = rt.csr_transpose(torch.zeros(1, dtype=torch.int64, device=DEV), z, None, 0)
    assert colptr.tolist() == [0]
    rp = torch.tensor([0, 2], dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError, match="out of range"):
        rt.csr_transpose(rp, torch.tensor([0, 5], dtype=torch.int64, device=DEV), None, 5)
    with pytest.raises(RuntimeError, match="out of range"):
        rt.csr_transpose(rp, torch.tensor([-1, 2], dtype=torch.int64, device=DEV), None, 5)
    with pytest.raises(RuntimeError, match="int64"):
        rt.csr_transpose(rp.to(torch.int32), torch.tensor([0, 1], dtype=torch.int64, device=DEV), None, 5)


def test_sparse_block_transposes_where_it_lives():
    """SparseCSR.csc() of a block on the GPU equals the csc() of the same block on the host,
    and a graph moved to the GPU propagates backward through transposes built there."""
    from sparse_csr import SparseCSR
    rng = np.random.default_rng(5)
    vlist, elist, value = random_block(rng, 900, 700, 5.0)
    host = SparseCSR(torch.from_numpy(vlist), torch.from_numpy(elist), torch.from_numpy(value), (900, 700))
    dev = host.to(DEV)
    assert dev._csc is None
    from util import closed_form_transpose
    for a, b, c in zip(host.csc(), dev.csc(), closed_form_transpose(vlist, elist, value, 700)):
        assert b.device.type == "cuda" and torch.equal(a, b.cpu()) and np.array_equal(b.cpu().numpy(), c)
    tt = dev.t()
    assert tt.sparse_sizes() == (700, 900) and torch.equal(tt.csr()[1].cpu(), host.csc()[1])
