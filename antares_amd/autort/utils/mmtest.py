"""``python -m autort.utils.mmtest`` (README.md:128-150): the fp32 matrix product `gemm_f32` through autort.export."""
from __future__ import annotations

import argparse
import sys

from . import GEMM_F32_INPUTS, GEMM_F32_IR


def gemm_f32_op(config=None):
    """`autort.ops.gemm_f32`: the module file of an earlier `autort.utils.export` run when there is one (it carries the
    tuned launch configuration), else a fresh export."""
    from .. import export, ops
    if config is None:
        try:
            return getattr(ops, 'gemm_f32')
        except AttributeError:
            pass
    return export(ir=GEMM_F32_IR, inputs=GEMM_F32_INPUTS, config=config, name='gemm_f32')


def run(size: int = 4096, runs: int = 5, out=sys.stdout) -> float:
    import torch
    from ...runtime import capi
    from ..op import current_stream_handle
    op = gemm_f32_op()
    dev = torch.device('cuda')
    a = torch.randn(size, size, device=dev)
    b = torch.randn(size, size, device=dev)
    c = op(a, b)                                    # first call: compiles / loads, tunes when the configuration asks for it
    stream = current_stream_handle()
    start, stop = capi.Event(), capi.Event()
    start.record(stream)
    for _ in range(runs):
        c = op(a, b)
    stop.record(stream)
    tflops = 2.0 * size ** 3 * runs / (start.elapsed_ms(stop) * 1e-3) / 1e12
    ref = a[:64].double() @ b.double()
    assert torch.allclose(c[:64].double(), ref, rtol=1e-4, atol=1e-2), 'gemm_f32 result is off'
    print('\n  >> Performance of your device:\n', file=out)
    print(f'     `MM-Perf` (current) = {tflops:.2f} TFLOPS', file=out)
    print('    ~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~', file=out, flush=True)
    return tflops


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog='autort.utils.mmtest')
    ap.add_argument('--size', type=int, default=4096)
    args = ap.parse_args(argv)
    run(args.size)
    return 0


if __name__ == '__main__':
    sys.exit(main())
