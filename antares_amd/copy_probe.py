"""Runs the library's plain copy kernel on a buffer of known size.

    python -m antares_amd.copy_probe [MiB] [launches]

Used to calibrate memory-traffic counters (FETCH_SIZE / WRITE_SIZE): the copy
reads and writes exactly MiB * 2^20 bytes per launch, so the ratio of the
counter to that figure is the scale to apply to other kernels' readings.
"""
import sys
from ctypes import c_void_p

import torch

from .runtime import capi


def main():
    mib = int(sys.argv[1]) if len(sys.argv) > 1 else 256
    launches = int(sys.argv[2]) if len(sys.argv) > 2 else 5
    capi.init(0)
    n = mib << 20
    src = torch.full((n,), 7, dtype=torch.uint8, device='cuda')
    dst = torch.empty_like(src)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(launches):
        capi.check(capi.lib().art_copy_bytes(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), n, c_void_p(stream)))
    torch.cuda.synchronize()
    assert bool((dst == 7).all())
    print(f'copied {n} bytes x {launches} launches')


if __name__ == '__main__':
    main()
