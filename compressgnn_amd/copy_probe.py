"""Copy-kernel probe: runs the library's plain copy kernel (cgnn_copy_bytes) over a
buffer of known size a few times.  Profiler byte counters (FETCH_SIZE, WRITE_SIZE) read
under `rocprofv3 --pmc` for this program give the factor that converts the counters'
units into bytes for the other kernels.

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out -- python -m compressgnn_amd.copy_probe [MiB] [repeats]
"""
import ctypes
import sys

import torch

from compressgnn_amd import abi


def main():
    mib = int(sys.argv[1]) if len(sys.argv) > 1 else 1024
    reps = int(sys.argv[2]) if len(sys.argv) > 2 else 3
    n = mib << 20
    src = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    dst = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    for _ in range(reps):
        abi.check(abi.lib().cgnn_copy_bytes(abi.ptr(src), abi.ptr(dst), ctypes.c_size_t(n), abi.stream_of(src)))
    torch.cuda.synchronize()
    print("copied %d bytes x %d (reads %d, writes %d per launch)" % (n, reps, n, n))


if __name__ == "__main__":
    main()
