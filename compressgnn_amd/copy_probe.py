"""Memory probes: the library's plain copy kernel (cgnn_copy_bytes), streaming-read kernel
(cgnn_read_bytes) and streaming-write kernel (cgnn_fill_bytes) over a buffer of known size.

Profiler byte counters (FETCH_SIZE, WRITE_SIZE) read under `rocprofv3 --pmc` for the copy
give the factor that converts the counters' units into bytes for the other kernels:

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out -- python -m compressgnn_amd.copy_probe [MiB] [repeats]

With `read` as third argument the program times the streaming read with HIP events and
prints the rate; a buffer that fits the 256 MB last-level cache shows what that cache
delivers, a larger one what HBM delivers:

    python -m compressgnn_amd.copy_probe 1024 20 read

With `write` it times the streaming write of zeros the same way.
"""
import ctypes
import sys

import torch

from compressgnn_amd import abi


def main():
    mib = int(sys.argv[1]) if len(sys.argv) > 1 else 1024
    reps = int(sys.argv[2]) if len(sys.argv) > 2 else 3
    mode = sys.argv[3] if len(sys.argv) > 3 else "copy"
    n = mib << 20
    src = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    L = abi.lib()
    if mode == "read":
        sink = torch.zeros(1, dtype=torch.int32, device="cuda:0")
        run = lambda: abi.check(L.cgnn_read_bytes(abi.ptr(src), ctypes.c_size_t(n), abi.ptr(sink), abi.stream_of(src)))
    elif mode == "write":
        run = lambda: abi.check(L.cgnn_fill_bytes(abi.ptr(src), ctypes.c_size_t(n), abi.stream_of(src)))
    else:
        dst = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
        run = lambda: abi.check(L.cgnn_copy_bytes(abi.ptr(src), abi.ptr(dst), ctypes.c_size_t(n), abi.stream_of(src)))
    run()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        run()
    end.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / reps
    moved = n if mode in ("read", "write") else 2 * n
    print("%s: %d bytes per launch x %d launches, %.1f us per launch, %.0f GB/s (%s)"
          % (mode, n, reps, ms * 1e3, moved / ms / 1e6, mode if mode in ("read", "write") else "read + write"))


if __name__ == "__main__":
    main()
