"""``python -m autort.utils.fp32test`` (README.md:49-55): fp32 multiply-add rate of the vector units."""
from __future__ import annotations

import argparse
import sys

CHAINS, STEPS = 16, 4096
SOURCE = f"""
extern "C" __global__ __launch_bounds__(256) void fp32test(float* __restrict__ out, float a, float b) {{
  float acc[{CHAINS}];
#pragma unroll
  for (int c = 0; c < {CHAINS}; ++c) acc[c] = (float)(threadIdx.x + c);
  for (int s = 0; s < {STEPS}; ++s) {{
#pragma unroll
    for (int c = 0; c < {CHAINS}; ++c) acc[c] = __builtin_fmaf(acc[c], a, b);      // independent chains: one multiply-add each
  }}
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < {CHAINS}; ++c) sum += acc[c];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = sum;
}}
"""


def theoretical_tflops(props: dict) -> float:
    """128 fp32 lanes per compute unit and clock (four SIMDs of 16 lanes, two-wide packed issue), two flops per lane."""
    return props['compute_units'] * 128 * 2 * props['clock_khz'] * 1e3 / 1e12


def run(rounds: int = 50, out=sys.stdout) -> float:
    import torch
    from ...runtime import capi
    from ..op import compile_cached, current_stream_handle
    capi.init(0)
    props = capi.device_props()
    module = capi.Module(compile_cached(SOURCE))
    fn = module.function('fp32test')
    blocks = props['compute_units'] * 32
    buf = torch.empty(blocks * 256, dtype=torch.float32, device='cuda')
    stream = current_stream_handle()
    import struct
    fbits = lambda v: struct.unpack('<I', struct.pack('<f', v))[0]
    args = [buf.data_ptr(), fbits(0.999), fbits(0.001)]
    capi.launch(fn, (blocks, 1, 1), (256, 1, 1), stream, args)
    flops = 2.0 * CHAINS * STEPS * blocks * 256
    best = 0.0
    for i in range(1, rounds + 1):
        start, stop = capi.Event(), capi.Event()
        start.record(stream)
        capi.launch(fn, (blocks, 1, 1), (256, 1, 1), stream, args)
        stop.record(stream)
        best = max(best, flops / (start.elapsed_ms(stop) * 1e-3) / 1e12)
        if i % max(1, rounds // 10) == 0 or i == rounds:
            print(f'  [{i}/{rounds}] AutoRT FP32 TFLOPS: (Actual ~= {best:.2f} TFLOPS) (Theoretical ~= {theoretical_tflops(props):.2f} TFLOPS)',
                  file=out, flush=True)
    assert bool(torch.isfinite(buf).all())
    return best


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog='autort.utils.fp32test')
    ap.add_argument('-n', '--rounds', type=int, default=50)
    args = ap.parse_args(argv)
    run(args.rounds)
    return 0


if __name__ == '__main__':
    sys.exit(main())
