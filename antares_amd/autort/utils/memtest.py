"""``python -m autort.utils.memtest`` (README.md:43-47): device memory bandwidth of a plain copy."""
from __future__ import annotations

import argparse
import sys


def theoretical_gbps(props: dict) -> float:
    """Peak of the memory interface from what the device reports: HBM3 moves four transfers per reported memory clock
    over the bus width (MI355X: 2.0 GHz x 4 x 8192 bits = 8.2 TB/s)."""
    return 4.0 * props['memory_clock_khz'] * 1e3 * props['memory_bus_width_bits'] / 8 / 1e9


def run(rounds: int = 100, mib: int = 1024, out=sys.stdout) -> float:
    import torch
    from ctypes import c_void_p
    from ...runtime import capi
    from ..op import current_stream_handle
    capi.init(0)
    props = capi.device_props()
    n = mib << 20
    src = torch.zeros(n, dtype=torch.uint8, device='cuda')
    dst = torch.empty_like(src)
    stream = current_stream_handle()
    lib = capi.lib()
    capi.check(lib.art_copy_bytes(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), n, c_void_p(stream)))
    best = 0.0
    for i in range(1, rounds + 1):
        start, stop = capi.Event(), capi.Event()
        start.record(stream)
        capi.check(lib.art_copy_bytes(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), n, c_void_p(stream)))
        stop.record(stream)
        gbps = 2.0 * n / (start.elapsed_ms(stop) * 1e-3) / 1e9          # bytes read + bytes written
        best = max(best, gbps)
        if i % max(1, rounds // 10) == 0 or i == rounds:
            print(f'  [{i}/{rounds}] AutoRT Device Memory Bandwidth: (Actual ~= {best:.2f} GB/s) '
                  f'(Theoretical ~= {theoretical_gbps(props):.2f} GB/s)', file=out, flush=True)
    return best


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog='autort.utils.memtest')
    ap.add_argument('-n', '--rounds', type=int, default=100)
    ap.add_argument('--mib', type=int, default=1024, help='size of the copied buffer')
    args = ap.parse_args(argv)
    run(args.rounds, args.mib)
    return 0


if __name__ == '__main__':
    sys.exit(main())
