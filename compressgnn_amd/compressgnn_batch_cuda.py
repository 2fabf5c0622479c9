"""GPU batch compressor behind the reference's optional module name
(src/offline/bindings/batch_cuda.cpp:3-9: `is_available()` and
`compress_csr_batch(vlist, elist, rounds=12, min_pair_frequency=16)`), which
loader/compression_backend.py:6-40 picks when `compression_backend` is 'auto' or 'cuda'.

The rounds run as HIP kernels (csrc/merger.hip) on the current GPU and return the same
arrays as the host compressor compressgnn_offline.compress_csr_batch: (vlist int32,
elist int32, vertex_cnt, rule_cnt).  Input checks and errors follow the reference's bridge
(src/offline/bindings/batch_bridge.hpp:8-26): ValueError for non-integer, negative or
too large values and for min_pair_frequency < 3."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


def is_available():
    if not os.path.exists(os.path.join(_HERE, "lib", "libcgnn_hip.so")):
        return False
    import torch
    return torch.cuda.is_available()


def compress_csr_batch(vlist, elist, rounds=12, min_pair_frequency=16, release_cache=False):
    """release_cache=True hands the workspace (about 70 bytes per edge) back to the device
    afterwards with torch.cuda.empty_cache(), which also flushes whatever else the caller's
    allocator holds cached: for a preparation script that goes on to build a large model."""
    import torch
    try:
        from compressgnn_amd import abi
    except ImportError:  # used with compressgnn_amd/ itself on sys.path
        import abi
    arrays = []
    for arr in (vlist, elist):
        a = np.asarray(arr)
        if a.ndim != 1 or a.dtype.kind not in "iu":
            raise ValueError("CSR arrays must be one-dimensional integer arrays")
        if a.size and (int(a.max()) > np.iinfo(np.int32).max or int(a.min()) < 0):
            raise ValueError("CSR value exceeds int32 range")
        arrays.append(np.ascontiguousarray(a, dtype=np.int64))
    if min_pair_frequency < 3:
        raise ValueError("Batch compression needs min_pair_frequency >= 3")
    if rounds < 1:
        raise ValueError("rounds must be positive")
    vl, el = arrays
    if len(vl) == 0:
        return np.zeros(1, np.int32), np.zeros(0, np.int32), 0, 0
    if not torch.cuda.is_available():
        raise RuntimeError("GPU compression requested but no usable device is available")
    dev = torch.device("cuda", torch.cuda.current_device())
    V, E = len(vl) - 1, len(el)
    L = abi.lib()
    L.cgnn_compress_batch_workspace_bytes.restype = ctypes.c_size_t
    need = L.cgnn_compress_batch_workspace_bytes(abi.i64(V), abi.i64(E))
    dv, de = torch.from_numpy(vl).to(dev), torch.from_numpy(el).to(dev)
    out_ptr = torch.empty(V + E // 2 + 2, dtype=torch.int32, device=dev)
    out_col = torch.empty(max(E, 1), dtype=torch.int32, device=dev)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    summary = (ctypes.c_int64 * 2)()
    rc = L.cgnn_compress_csr_batch_device(abi.i64(V), abi.i64(E), abi.ptr(dv), abi.ptr(de), ctypes.c_int(rounds),
                                          ctypes.c_int(min_pair_frequency), abi.ptr(out_ptr), abi.ptr(out_col),
                                          summary, abi.ptr(ws), ctypes.c_size_t(need), abi.stream_of(dv))
    if rc != 0:
        msg = L.cgnn_last_error().decode()
        if rc == 1:  # CGNN_EINVAL: malformed input
            raise ValueError(msg)
        raise RuntimeError(msg)
    R, n = int(summary[0]), int(summary[1])
    result = out_ptr[:V + R + 1].cpu().numpy(), out_col[:n].cpu().numpy(), V, R
    del dv, de, out_ptr, out_col, ws
    if release_cache:
        torch.cuda.empty_cache()
    return result
