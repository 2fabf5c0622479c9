"""cgnn_spmm_static, the entry point that allocates nothing: same bits as cgnn_spmm on the same
block and inputs, on two calls in a row that share the library's built-in scratch (the second
with a smaller input, so what the first call left behind in the scratch lies around it), for
rows that are cut into runs, carried across workgroups and reduced level by level, fresh and
accumulating, in both precisions; sizes beyond the scratch are refused with an error."""
import ctypes

import numpy as np
import pytest
import torch

from compressgnn_amd import abi
from util import random_csr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(seed, rows, cols, F, giant, dtype=np.float32, seg=0):
    rng = np.random.default_rng(seed)
    lens = rng.poisson(6.0, rows)
    lens[rng.random(rows) < 0.2] = 0
    for r in rng.choice(rows, size=max(1, rows // 40), replace=False):
        lens[r] = int(rng.integers(200, 3000))
    lens[rows // 2] = giant  # carries on several reduction levels
    vlist = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    elist = rng.integers(0, cols, int(vlist[-1])).astype(np.int64)
    value = (rng.standard_normal(len(elist)) / np.sqrt(np.repeat(np.maximum(lens, 1), lens))).astype(dtype)
    x = rng.standard_normal((cols, F)).astype(dtype)
    A = abi.DeviceCsr.from_host(rows, cols, vlist, elist, value, DEV, seg_nnz=seg)
    return A, torch.from_numpy(x).to(DEV), torch.from_numpy(rng.standard_normal((rows, F)).astype(dtype)).to(DEV)


def _both(A, X, Y0, kernel):
    """(cgnn_spmm, cgnn_spmm_static) results, fresh and accumulating."""
    want = abi.spmm(A, X, None, False, kernel)
    want_acc = abi.spmm(A, X, Y0.clone(), True, kernel)
    got = abi.spmm_static(A, X, torch.full_like(Y0, float("nan")), False, kernel)
    got_acc = abi.spmm_static(A, X, Y0.clone(), True, kernel)
    torch.cuda.synchronize()
    return (want, got), (want_acc, got_acc)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_static_scratch_matches_the_workspace_entry(dtype):
    capacity = abi.lib().cgnn_spmm_static_scratch_bytes()
    assert capacity == 64 << 20
    big = _case(1, 30000, 20000, 128 if dtype == np.float32 else 24, giant=400_000, dtype=dtype)
    small = _case(2, 900, 700, 20, giant=30_000, dtype=dtype, seg=8)
    for A, X, Y0 in (big, small, big):  # large, then smaller, then large again over the leftovers
        for kernel in (abi.SPMM_NNZ, abi.SPMM_AUTO, abi.SPMM_ROW):
            need = abi.lib().cgnn_spmm_workspace_bytes(ctypes.byref(A.struct()), abi.i64(X.shape[1]),
                                                       abi.dtype_code(X.dtype), kernel)
            assert need <= capacity
            for want, got in _both(A, X, Y0, kernel):
                assert torch.equal(got, want)
    # no entries, no rows, zero width: nothing to do, nothing touched
    empty = abi.DeviceCsr.from_host(5, 10, np.zeros(6, np.int64), np.zeros(0, np.int64), np.zeros(0, dtype), DEV)
    X = torch.ones(10, 8, device=DEV, dtype=torch.from_numpy(np.zeros(1, dtype)).dtype)
    out = abi.spmm_static(empty, X, torch.full((5, 8), 3.0, device=DEV, dtype=X.dtype), False, abi.SPMM_NNZ)
    assert not out.any()
    kept = abi.spmm_static(empty, X, torch.full((5, 8), 3.0, device=DEV, dtype=X.dtype), True, abi.SPMM_NNZ)
    assert bool((kept == 3).all())


def test_static_scratch_refuses_what_does_not_fit():
    """The limit is checked on the host from the sizes alone: no launch, no access."""
    s = abi.CsrStruct()
    rowptr = torch.zeros(2, dtype=torch.int32, device=DEV)
    s.rows, s.cols, s.nnz = 1, 1, 40_000_000
    s.rowptr, s.colidx, s.rowidx, s.val = rowptr.data_ptr(), rowptr.data_ptr(), rowptr.data_ptr(), 0
    s.max_row_nnz, s.seg_nnz = 40_000_000, 0
    L = abi.lib()
    need = L.cgnn_spmm_workspace_bytes(ctypes.byref(s), abi.i64(128), abi.F32, abi.SPMM_NNZ)
    assert need > L.cgnn_spmm_static_scratch_bytes()
    rc = L.cgnn_spmm_static(ctypes.byref(s), abi.F32, abi.ptr(rowptr), abi.ptr(rowptr), abi.i64(128), 0, abi.SPMM_NNZ,
                            abi.stream_of(rowptr))
    assert rc == 2 and b"built-in" in L.cgnn_last_error()  # CGNN_EWORKSPACE
    torch.cuda.synchronize()


def test_static_entry_leaves_device_memory_as_it_found_it():
    """'Allocates nothing', measured: once the array's address is known on the device
    (cgnn_spmm_static_init, outside any capture), calls leave the free memory of the device where
    it was -- the driver's own figure (hipMemGetInfo), which no caching allocator hides."""
    assert abi.lib().cgnn_spmm_static_init() == 0
    A, X, Y0 = _case(3, 20000, 15000, 128, giant=200_000)
    Y = torch.empty_like(Y0)
    abi.spmm_static(A, X, Y, False, abi.SPMM_NNZ)  # warmed: kernels loaded
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for kernel in (abi.SPMM_NNZ, abi.SPMM_ROW, abi.SPMM_AUTO):
        abi.spmm_static(A, X, Y, False, kernel)
        abi.spmm_static(A, X, Y, True, kernel)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    assert torch.equal(abi.spmm_static(A, X, Y, False, abi.SPMM_NNZ), abi.spmm(A, X, None, False, abi.SPMM_NNZ))
