"""The shared libraries load and export every entry point their headers declare (no
compute calls, so no GPU is needed), and the Python-visible operator module exposes
the reference's operator names."""
import ctypes
import os
import re
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "compressgnn_amd")
sys.path.insert(0, PKG)


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cgnn_[a-z0-9_]+)\s*\(", text)))


def test_device_library_exports_every_declared_symbol():
    names = declared("compressgnn_abi.h")
    assert len(names) >= 18
    lib = ctypes.CDLL(os.path.join(PKG, "lib", "libcgnn_hip.so"))
    for n in names:
        assert hasattr(lib, n), n
    lib.cgnn_version.restype = ctypes.c_char_p
    assert b"gfx950" in lib.cgnn_version()
    from compressgnn_amd import abi
    assert sorted(abi.EXPORTS) == names


def test_prep_library_exports_every_declared_symbol():
    names = declared("compressgnn_prep.h")
    lib = ctypes.CDLL(os.path.join(PKG, "lib", "libcgnn_prep.so"))
    for n in names:
        assert hasattr(lib, n), n
    import compressgnn_offline as off
    assert sorted(off.EXPORTS) == names


def test_argument_checks_without_a_gpu():
    """Entry points validate their arguments before touching the device."""
    from compressgnn_amd import abi
    lib = abi.lib()
    s = abi.CsrStruct()
    s.rows, s.cols, s.nnz = 4, 4, 1 << 40
    rc = lib.cgnn_spmm(ctypes.byref(s), 0, None, None, ctypes.c_int64(8), 0, 0, None, ctypes.c_size_t(0), None)
    assert rc == 1 and b"2^31" in lib.cgnn_last_error()
    assert lib.cgnn_spmm(None, 0, None, None, ctypes.c_int64(8), 0, 0, None, ctypes.c_size_t(0), None) == 1
    rc = lib.cgnn_lsh_hash(ctypes.c_int64(4), ctypes.c_int64(4), 31, 0, None, None, None, None, None)
    assert rc == 1 and b"[0,30]" in lib.cgnn_last_error()
    assert lib.cgnn_copy_bytes(None, None, ctypes.c_size_t(7), None) == 1
    assert lib.cgnn_lsh_scan_workspace_bytes(16) >= 64


def test_runtime_module_has_the_reference_operator_names():
    import compressgnn_runtime as rt
    for name in ["spmm_func", "cluster_forward", "cluster_workspace", "cluster_assign", "cluster_mean",
                 "cluster_mean_backward", "cluster_reconstruct", "cluster_reconstruct_backward"]:
        assert hasattr(rt, name), name
    import torch
    with pytest.raises(RuntimeError, match="GPU"):
        rt.spmm_func(torch.zeros(2, dtype=torch.long), torch.zeros(0, dtype=torch.long), torch.zeros(0),
                     torch.zeros(1, 3), "rowbalance", None)
    with pytest.raises(RuntimeError):
        rt.cluster_assign(torch.zeros(3, 4), torch.zeros(4, 2), 2, [])


def test_sampler_module_has_the_reference_names():
    """compressgnn_sample, the module name the reference builds from src/sample
    (function.cpp:7-9): both functions, GPU tensors only."""
    import torch
    import compressgnn_sample as sampler
    for name in ["neighbor_sample_cg_sim", "neighbor_sample_ori_impl"]:
        assert callable(getattr(sampler, name)), name
    ptr = torch.zeros(3, dtype=torch.long)
    with pytest.raises(RuntimeError, match="GPU"):
        sampler.neighbor_sample_ori_impl(ptr, torch.zeros(0, dtype=torch.long), torch.zeros(1, dtype=torch.long), [2])
