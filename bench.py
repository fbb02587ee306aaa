#!/usr/bin/env python
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra] [--no-decode]
    python bench.py --calibrate-copy MIB LAUNCHES     # plain copy of known size, for scaling memory-traffic counters
    python bench.py --read-floor                      # only the read-only launch over the headline's weight bytes
    python bench.py --stream-floors                   # read-only, store-only and copy launches over 22.5 / 67 MB
    python bench.py --phase-chain                     # phases that meet inside ONE launch against dependent launches
    python bench.py --attention                       # only the decode attention at positions 0 / 127 / 255 / 383
    python bench.py --gemv-knobs                      # only the split-K int4 GEMV with each of its launch shapes

Headline workload (BASELINE.json: "int4-GEMV HBM GB/s"): the int4 group-128
GEMV y[1,11008] = x[1,4096] @ dequant(W), through ``autort.export`` and the
C-ABI library.  One step is one pass over LAYERS distinct weight sets
(LAYERS * 22.5 MB is larger than every cache of the chip, so each launch
streams its weights from HBM, as a decode step does); all inputs are resident
in HBM before the timed region.  The pass is recorded once in a HIP graph so
that the timed region contains kernels, not Python.

Prints ONE JSON line.  ``roofline`` is for the GEMV kernel: algorithmic bytes
per launch / mean time per launch inside the timed region (HIP events on the
launch stream) against the 8 TB/s HBM peak.  ``cpu_baseline`` is the CPU
oracle's loop-nest restatement of the reference's c-mcpu backend for the same
program, timed on this host on a bounded sample.  ``extra`` carries the other
configurations (sigmoid, partition, other GEMV shapes) measured the same way.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_F32_PEAK_TFLOPS = 157.3
LAYERS = 32
# HBM bytes per launch of the headline GEMV kernel come from the committed counter summary (FETCH_SIZE / WRITE_SIZE
# scaled by the copy-kernel calibration), which states them on a line `traffic_bytes_per_launch: <integer>`.
TRAFFIC_SUMMARY = os.path.join(ROOT, 'profiles', 'gemv_w4a16_4096x11008_traffic_pmc.md')


def traffic_from_summary(path=TRAFFIC_SUMMARY):
    """Measured HBM bytes per launch as recorded in the counter summary, or None when there is none."""
    try:
        with open(path) as f:
            for line in f:
                if line.strip().startswith('traffic_bytes_per_launch:'):
                    return int(line.split(':', 1)[1].strip().replace('_', ''))
    except (OSError, ValueError):
        pass
    return None


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--no-extra', action='store_true', help='headline workload only')
    ap.add_argument('--no-decode', action='store_true', help='skip the 32-layer decode leg')
    ap.add_argument('--decode-cpu-steps', type=int, default=4, help='decode steps timed on the CPU oracle (0 = skip)')
    ap.add_argument('--att-parts', type=int, default=8, help='blocks per head of the decode attention (1 = unsplit)')
    ap.add_argument('--seed', type=int, default=0)
    ap.add_argument('--calibrate-copy', nargs=2, type=int, metavar=('MIB', 'LAUNCHES'),
                    help='run only the plain copy kernel on MIB MiB, LAUNCHES times (counter calibration), and exit')
    ap.add_argument('--read-floor', action='store_true',
                    help='run only the read-only launch over 32 distinct buffers of the headline weight size, and exit')
    ap.add_argument('--stream-floors', action='store_true',
                    help='run only the read-only, store-only and copy launches (what one launch needs to move bytes), and exit')
    ap.add_argument('--lowering', action='store_true',
                    help='run only the generic lowering on a set of programs (products, convolutions, reductions, rows, copies), one JSON line each, and exit')
    ap.add_argument('--attention', action='store_true',
                    help='run only the decode attention (rotary + cache write + attention over 8 blocks per head) at several positions, and exit')
    ap.add_argument('--gemv-knobs', action='store_true',
                    help='run only the split-K int4 GEMV at the four benchmark shapes with every (rows per lane, wavefronts per block), and exit')
    ap.add_argument('--phase-chain', action='store_true',
                    help='run only the probe of phases meeting inside one launch (a persistent kernel against dependent launches), and exit')
    return ap.parse_args()


def calibrate_copy(torch, capi, mib, launches):
    """The library's plain copy kernel on a buffer of known size: it reads and writes exactly mib * 2^20 bytes per
    launch, so the ratio of a memory-traffic counter to that figure is the scale to apply to other kernels' readings."""
    from ctypes import c_void_p
    n = mib << 20
    src = torch.full((n,), 7, dtype=torch.uint8, device='cuda')
    dst = torch.empty_like(src)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(launches):
        capi.check(capi.lib().art_copy_bytes(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), n, c_void_p(stream)))
    torch.cuda.synchronize()
    assert bool((dst == 7).all())
    return {'copied_bytes_per_launch': n, 'launches': launches}


def bench_read_floor(torch, capi, steps, warmup, nbytes=2048 * 11008, layers=LAYERS):
    """What one dependent launch needs to bring the headline GEMV's weight bytes on chip with no arithmetic behind
    them: `art_read_bytes` (same blocks, same loads as the GEMV's weight stream) over `layers` distinct buffers
    recorded in one HIP graph, exactly as the GEMV itself is timed."""
    from ctypes import c_void_p
    bufs = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device='cuda') for _ in range(layers)]
    sink = torch.zeros(4096, dtype=torch.int32, device='cuda')

    def one_pass():
        stream = torch.cuda.current_stream().cuda_stream
        for b in bufs:
            capi.check(capi.lib().art_read_bytes(c_void_p(b.data_ptr()), nbytes, c_void_p(sink.data_ptr()), c_void_p(stream)))
    sec = time_graph(torch, capi, one_pass, steps, warmup) / layers

    # the same launch over 32 KiB (one block): what a dependent kernel node costs before it has moved any bytes
    small = [b[:32768] for b in bufs]

    def tiny_pass():
        stream = torch.cuda.current_stream().cuda_stream
        for b in small:
            capi.check(capi.lib().art_read_bytes(c_void_p(b.data_ptr()), 32768, c_void_p(sink.data_ptr()), c_void_p(stream)))
    tiny = time_graph(torch, capi, tiny_pass, steps, warmup) / layers
    return {'kernel': 'art_read_kernel', 'bytes_per_launch': nbytes, 'us_per_launch': round(sec * 1e6, 3),
            'gbps': round(nbytes / sec / 1e9, 1), 'frac_of_peak': round(nbytes / sec / 1e9 / HBM_PEAK_GBPS, 4),
            'us_per_launch_of_one_block': round(tiny * 1e6, 3)}


def bench_stream_floors(torch, capi, steps, warmup, layers=16):
    """What one dependent launch needs to read, to write, and to read and write bytes with nothing else to do:
    `art_read_bytes`, `art_fill_bytes` and `art_copy_bytes` over `layers` distinct buffers in one HIP graph."""
    from ctypes import c_void_p
    lib = capi.lib()
    out = []
    sink = torch.zeros(4096, dtype=torch.int32, device='cuda')
    for nbytes in (2048 * 11008, 6144 * 11008):
        bufs = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device='cuda') for _ in range(layers)]
        dsts = [torch.empty_like(b) for b in bufs]

        def reads():
            st = torch.cuda.current_stream().cuda_stream
            for b in bufs:
                capi.check(lib.art_read_bytes(c_void_p(b.data_ptr()), nbytes, c_void_p(sink.data_ptr()), c_void_p(st)))

        def fills():
            st = torch.cuda.current_stream().cuda_stream
            for d in dsts:
                capi.check(lib.art_fill_bytes(c_void_p(d.data_ptr()), nbytes, 7, c_void_p(st)))

        def copies():
            st = torch.cuda.current_stream().cuda_stream
            for b, d in zip(bufs, dsts):
                capi.check(lib.art_copy_bytes(c_void_p(d.data_ptr()), c_void_p(b.data_ptr()), nbytes, c_void_p(st)))
        row = {'bytes': nbytes}
        for name, fn, moved in (('read_only', reads, nbytes), ('store_only', fills, nbytes), ('copy', copies, 2 * nbytes)):
            sec = time_graph(torch, capi, fn, steps, warmup) / layers
            row[name] = {'us_per_launch': round(sec * 1e6, 3), 'gbps_moved': round(moved / sec / 1e9, 1)}
        assert bool((dsts[0] == bufs[0]).all())
        out.append(row)
        del bufs, dsts
    return out


def _conv(n, c, f, hw, dt='float32', pad=False):
    cast = '.to(`float32`)' if dt == 'float16' else ''
    if pad:
        ir = (f'output0[N, F, HO, WO] +=! input0[N, C, HO + KH - 1, WO + KW - 1]{cast}.when([HO + KH - 1 >= 0, HO + KH - 1 < {hw}, '
              f'WO + KW - 1 >= 0, WO + KW - 1 < {hw}], 0.0) * input1[F, C, KH, KW]{cast} where HO in {hw}, WO in {hw}')
    else:
        ir = f'output0[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW]{cast} * input1[F, C, KH, KW]{cast} where HO in {hw - 2}, WO in {hw - 2}'
    ho = hw if pad else hw - 2
    return (f'{"padded " if pad else ""}3x3 convolution {dt} {n}x{c}x{hw}x{hw} -> {f} channels', ir,
            [f'input0={dt}[N:{n}, C:{c}, H:{hw}, W:{hw}]', f'input1={dt}[F:{f}, C:{c}, KH:3, KW:3]'], [(n, c, hw, hw), (f, c, 3, 3)],
            ('flop', 2 * n * f * ho * ho * c * 9))


# Programs of the reference's IR documentation (AntaresIR.md:108-256) and of common networks at sizes that fill the chip,
# for the generic lowering: (name, program, inputs, shapes, ('flop', count) or ('bytes', count or None = inputs + output)).
LOWERING_CASES = [
    ('fp32 product 4096x4096x1024, A stored [K, N]', 'output0[N, M] +=! input0[K, N] * input1[K, M]',
     ['input0=float32[K:1024, N:4096]', 'input1=float32[K:1024, M:4096]'], [(1024, 4096), (1024, 4096)], ('flop', 2 * 4096 * 4096 * 1024)),
    ('fp16 A B^T into float32 4096x4096x1024', 'output0[N, M] +=! input0[N, K].to(`float32`) * input1[M, K].to(`float32`)',
     ['input0=float16[N:4096, K:1024]', 'input1=float16[M:4096, K:1024]'], [(4096, 1024), (4096, 1024)], ('flop', 2 * 4096 * 4096 * 1024)),
    ('fp16 product 2048^3 (float16 statement)', 'output0[N, M] +=! input0[N, K] * input1[K, M]',
     ['input0=float16[N:2048, K:2048]', 'input1=float16[K:2048, M:2048]'], [(2048, 2048), (2048, 2048)], ('flop', 2 * 2048 ** 3)),
    ('int8 A B^T into int32 4096^3', 'output0[N, M] +=! input0[N, K].cast(`int32`) * input1[M, K].cast(`int32`)',
     ['input0=int8[N:4096, K:4096]', 'input1=int8[M:4096, K:4096]'], [(4096, 4096), (4096, 4096)], ('flop', 2 * 4096 ** 3)),
    ('attention scores: 256 fp16 products of 1024 x 1024 x 128 into float32 (a 1 GiB result)',
     'output0[B, H, S, T] +=! input0[B, H, S, D].to(`float32`) * input1[B, H, T, D].to(`float32`)',
     ['input0=float16[B:8, H:32, S:1024, D:128]', 'input1=float16[B:8, H:32, T:1024, D:128]'], [(8, 32, 1024, 128), (8, 32, 1024, 128)],
     ('bytes', None)),
    ('batched fp32 product 8 x 512^3', 'output0[B, N, M] +=! input0[B, N, K] * input1[B, K, M]',
     ['input0=float32[B:8, N:512, K:512]', 'input1=float32[B:8, K:512, M:512]'], [(8, 512, 512), (8, 512, 512)], ('flop', 2 * 8 * 512 ** 3)),
    ('fp32 A B^T 512x512x8192 (sliced along k)', 'output0[N, M] +=! input0[N, K] * input1[M, K]',
     ['input0=float32[N:512, K:8192]', 'input1=float32[M:512, K:8192]'], [(512, 8192), (512, 8192)], ('flop', 2 * 512 * 512 * 8192)),
    _conv(8, 64, 64, 56), _conv(32, 128, 128, 30), _conv(32, 128, 128, 28, pad=True), _conv(32, 128, 128, 28, 'float16'),
    _conv(32, 128, 128, 28, 'float16', pad=True), _conv(8, 512, 512, 9),
    ('3x3 convolution float32, channels last, 32x30x30x128 -> 128 channels',
     'output0[N, HO, WO, F] +=! input0[N, HO + KH, WO + KW, C] * input1[KH, KW, C, F] where HO in 28, WO in 28',
     ['input0=float32[N:32, H:30, W:30, C:128]', 'input1=float32[KH:3, KW:3, C:128, F:128]'], [(32, 30, 30, 128), (3, 3, 128, 128)],
     ('flop', 2 * 32 * 128 * 28 * 28 * 128 * 9)),
    ('3x3 convolution float16, channels last, 32x30x30x128 -> 128 channels',
     'output0[N, HO, WO, F] +=! input0[N, HO + KH, WO + KW, C].to(`float32`) * input1[KH, KW, C, F].to(`float32`) where HO in 28, WO in 28',
     ['input0=float16[N:32, H:30, W:30, C:128]', 'input1=float16[KH:3, KW:3, C:128, F:128]'], [(32, 30, 30, 128), (3, 3, 128, 128)],
     ('flop', 2 * 32 * 128 * 28 * 28 * 128 * 9)),
    ('depthwise 3x3 convolution 32x128x56x56', 'output0[N, C, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[C, KH, KW] where HO in 54, WO in 54',
     ['input0=float32[N:32, C:128, H:56, W:56]', 'input1=float32[C:128, KH:3, KW:3]'], [(32, 128, 56, 56), (128, 3, 3)], ('bytes', None)),
    ('2x2 max pooling 32x64x112x112', 'output0[N, C, HO, WO] >=! input0[N, C, HO * 2 + KH, WO * 2 + KW] where HO in 56, WO in 56, KH in 2, KW in 2',
     ['input0=float32[N:32, C:64, H:112, W:112]'], [(32, 64, 112, 112)], ('bytes', None)),
    ('channel sums of 32x256x56x56', 'output0[C] +=! input0[N, C, H, W]', ['input0=float32[N:32, C:256, H:56, W:56]'], [(32, 256, 56, 56)], ('bytes', None)),
    ('column sums of 16384x4096', 'output0[C] +=! input0[N, C]', ['input0=float32[N:16384, C:4096]'], [(16384, 4096)], ('bytes', None)),
    ('sum of 67108864 fp32', 'output0[] +=! input0[N]', ['input0=float32[N:67108864]'], [(67108864,)], ('bytes', None)),
    ('softmax of 65536 rows of 1024 (AntaresIR.md:226)', 'temp0[N] >=! input0[N, C]; temp1[N] +=! (input0[N, C] - temp0[N]).call(`exp`); '
     'output0[N, C] = (input0[N, C] - temp0[N]).call(`exp`) / temp1[N]', ['input0=float32[N:65536, C:1024]'], [(65536, 1024)], ('bytes', 65536 * 1024 * 8)),
    ('layer normalisation of 4096 rows of 4096 (AntaresIR.md:232)', 'temp0[N] +=! input0[N, C]; temp1[N] +=! input0[N, C] * input0[N, C]; '
     'output0[N, C] = (input0[N, C] * C.val() - temp0[N]) * (temp1[N] * C.val() - temp0[N] * temp0[N] + 1e-5).call(`rsqrt`)',
     ['input0=float32[N:4096, C:4096]'], [(4096, 4096)], ('bytes', 4096 * 4096 * 8)),
    ('fp32 transpose 4096x4096', 'output0[C, N] = input0[N, C]', ['input0=float32[N:4096, C:4096]'], [(4096, 4096)], ('bytes', None)),
    ('fp16 NCHW -> NHWC 8x256x64x64', 'output0[N, H, W, C] = input0[N, C, H, W]', ['input0=float16[N:8, C:256, H:64, W:64]'], [(8, 256, 64, 64)], ('bytes', None)),
    ('bias add over 32x256x56x56', 'output0[N, C, H, W] = input0[N, C, H, W] + input1[C]',
     ['input0=float32[N:32, C:256, H:56, W:56]', 'input1=float32[C:256]'], [(32, 256, 56, 56), (256,)], ('bytes', None)),
    ('gathered rows: 8192 of 32000 x 4096 fp16', 'output0[N, C] = input0[input1[N], C]',
     ['input0=float16[V:32000, C:4096]', 'input1=int32[N:8192]'], [(32000, 4096), (8192,)], ('bytes', 8192 * 4096 * 2 * 2)),
    ('convolution + bias + ReLU 32x128x30x30 -> 128 (AntaresIR.md:250, one launch)',
     'conv_out[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[F, C, KH, KW] where HO in 28, WO in 28; '
     'output0[N, F, HO, WO] = (conv_out[N, F, HO, WO] + input2[F]).call(`max`, [0.0])',
     ['input0=float32[N:32, C:128, H:30, W:30]', 'input1=float32[F:128, C:128, KH:3, KW:3]', 'input2=float32[F:128]'],
     [(32, 128, 30, 30), (128, 128, 3, 3), (128,)], ('flop', 2 * 32 * 128 * 28 * 28 * 128 * 9)),
]


def bench_lowering(torch, autort, capi, steps, warmup):
    """The generic lowering on LOWERING_CASES: each program exported as a user would, the hand-written kernels switched
    off, timed as a graph replay (eight calls on eight copies of the inputs) at the sustained clock; rate in TFLOP/s,
    or in TB/s of the bytes a single pass over inputs and output moves."""
    dev = autort.device()
    out = []
    for name, ir, inputs, shapes, (kind, count) in LOWERING_CASES:
        op = autort.export(ir=ir, inputs=inputs, name='bench_lowering_' + ''.join(c for c in name if c.isalnum())[:40])
        op.fast_path = None
        g = torch.Generator('cpu').manual_seed(len(name))
        ts = [torch.randint(0, 32000, shp, generator=g, dtype=torch.int32).to(dev) if 'int32' in spec else
              (torch.randint(-128, 128, shp, generator=g, dtype=torch.int8).to(dev) if 'int8' in spec else
               torch.randn(shp, generator=g).to(torch.float16 if 'float16' in spec else torch.float32).to(dev)) for spec, shp in zip(inputs, shapes)]
        res = op(*ts)
        # eight calls per replayed graph, each on its own copy of the inputs: a graph of one short kernel would time
        # the replay itself (about 17 us), and the same tensors every time would be served by the caches
        sets = [ts] + [[t.clone() for t in ts] for _ in range(7)]

        def one_pass():
            for tensors in sets:
                op(*tensors)
        sec = time_graph(torch, capi, one_pass, steps, warmup, warm_ms=20.0) / len(sets)
        row = {'program': name, 'us': round(sec * 1e6, 1), 'launches': sum(1 for _ in _launched(op, inputs, shapes))}
        if kind == 'flop':
            row['tflops'] = round(count / sec / 1e12, 1)
        else:
            nbytes = count if count is not None else sum(t.numel() * t.element_size() for t in ts) + res.numel() * res.element_size()
            row['tb_per_s'] = round(nbytes / sec / 1e12, 2)
        out.append(row)
        print(json.dumps(row), flush=True)
        del ts, res, sets
    return out


def _launched(op, inputs, shapes):
    """The plans a call with these shapes launches from (a plan that covers the statement behind it counts once)."""
    env = {}
    for spec, shape in zip(inputs, shapes):
        for d, v in zip(spec.split('[', 1)[1].rstrip(']').split(','), shape):
            if ':' in d:
                env[d.split(':')[0].strip()] = v
    skip = 0
    for plan in op.plans_for(env):
        if skip:
            skip -= 1
            continue
        group = plan.row_group
        if group is not None and group.choose(env, {n: 0 for n in group.args})[1]:
            skip = group.count - 1
        else:
            skip = plan.covers - 1
        yield plan


def bench_phase_chain(torch, capi, phases=32, nbytes=2048 * 11008, runs=5):
    """`phases` phases of `nbytes` each inside ONE launch, all blocks meeting after every phase
    (`art_phase_chain_probe`), against the same reads as `phases` dependent launches."""
    from ctypes import c_void_p
    lib = capi.lib()
    src = torch.randint(0, 256, (phases * nbytes,), dtype=torch.uint8, device='cuda')
    sink = torch.zeros(4096, dtype=torch.int32, device='cuda')
    status = torch.zeros(1, dtype=torch.int32, device='cuda')
    stream = side_stream(torch)
    out = {'phases': phases, 'bytes_per_phase': nbytes}
    with torch.cuda.stream(stream):
        for mode, name in ((0, 'meeting_only'), (1, 'loads_after_the_meeting'), (2, 'next_loads_before_the_meeting')):
            best = None
            for _ in range(runs + 1):
                start, stop = capi.Event(), capi.Event()
                start.record(stream.cuda_stream)
                capi.check(lib.art_phase_chain_probe(c_void_p(src.data_ptr()), src.numel(), nbytes, phases, mode, c_void_p(sink.data_ptr()),
                                                     c_void_p(status.data_ptr()), c_void_p(stream.cuda_stream)))
                stop.record(stream.cuda_stream)
                us = start.elapsed_ms(stop) * 1e3 / phases
                best = us if best is None else min(best, us)
            stream.synchronize()
            if int(status.item()) != 0:
                raise RuntimeError('art_phase_chain_probe: a block gave up waiting (the chip was not free)')
            out[name + '_us_per_phase'] = round(best, 3)

    def launches():
        st = torch.cuda.current_stream().cuda_stream
        for i in range(phases):
            capi.check(lib.art_read_bytes(c_void_p(src.data_ptr() + i * nbytes), nbytes, c_void_p(sink.data_ptr()), c_void_p(st)))
    out['dependent_launches_us_per_phase'] = round(time_graph(torch, capi, launches, 20, 3) / phases * 1e6, 3)
    return out


def bench_attention(torch, autort, capi, steps, warmup, layers=LAYERS, heads=32, head_dim=128, max_seq=384, parts=8):
    """The decode attention of one step by itself: `attention_rope_split_f16` (rotary of q and k, both cache writes,
    attention over rows 0..pos in `parts` blocks per head) on `layers` distinct caches per replayed graph, at several
    positions.  Bytes per launch: the K and V rows it reads (2 * (pos + 1) * heads * head_dim fp16) plus q|k|v."""
    dev = autort.device()
    d = heads * head_dim
    g = torch.Generator().manual_seed(3)
    keys = (torch.randn(layers, max_seq, d, generator=g) * 0.5).half().to(dev)
    vals = (torch.randn(layers, max_seq, d, generator=g) * 0.5).half().to(dev)
    qkv = [(torch.randn(3 * d, generator=g)).half().to(dev) for _ in range(layers)]
    inv = (1.0 / (10000.0 ** (torch.arange(0, head_dim, 2).float() / head_dim))).half()
    inv_freq = torch.cat([inv, inv]).to(dev)
    att_f = torch.tensor([head_dim ** -0.5], dtype=torch.float32, device=dev)
    partial = [torch.zeros(heads, parts, 132, dtype=torch.float32, device=dev) for _ in range(layers)]
    pos = torch.zeros(1, dtype=torch.int32, device=dev)
    out = []
    for p in (0, 127, 255, 383):
        pos.fill_(p)

        def one_pass():
            for l in range(layers):
                autort.ops.attention_rope_split_f16(qkv[l], inv_freq, keys[l], vals[l], att_f, partial[l], extra=[pos])
        sec = time_graph(torch, capi, one_pass, steps, warmup) / layers
        nbytes = 2 * (p + 1) * d * 2 + 3 * d * 2
        out.append({'pos': p, 'us_per_launch': round(sec * 1e6, 3), 'kv_bytes_per_launch': nbytes, 'gbps': round(nbytes / sec / 1e9, 1)})
    return {'kernel': 'attention_kernel<f16, rotary + cache write>', 'blocks_per_head': parts, 'heads': heads, 'positions': out}


def bench_gemv_knobs(torch, autort, capi, workloads, steps, warmup, layers=16):
    """The split-K int4 GEMV (M = 1, benchmark layout) through `art_gemv_w4a16_knobs` with each of its four launch
    shapes - (rows per lane, wavefronts per block) in (8, 4), (4, 4), (8, 8), (4, 8) - and with the library's own
    choice (0, 0), `layers` rotating weight sets per replayed graph: what `tune:N` searches, and what the library's
    rule is set by."""
    from ctypes import c_void_p
    dev = autort.device()
    lib = capi.lib()
    rows = []
    for K, N in ((4096, 4096), (4096, 11008), (11008, 4096), (4096, 32000)):
        sets = [{k: v.to(dev) for k, v in workloads.w4_problem(100 + i, 1, K, N).items()} for i in range(layers)]
        y = torch.empty(1, N, dtype=torch.float16, device=dev)
        row = {'workload': f'int4 g128 GEMV M=1 K={K} N={N}, benchmark layout', 'us_per_launch': {}}
        for n_th, (r, w) in enumerate(((8, 4), (8, 4), (4, 4), (8, 8), (4, 8), (0, 0))):      # the first pass is not reported
            def one_pass():
                st = c_void_p(torch.cuda.current_stream().cuda_stream)
                for d in sets:
                    capi.check(lib.art_gemv_w4a16_knobs(c_void_p(d['x'].data_ptr()), c_void_p(d['qweight'].data_ptr()),
                                                        c_void_p(d['scales'].data_ptr()), c_void_p(d['qzeros'].data_ptr()),
                                                        c_void_p(y.data_ptr()), 1, K, N, r, w, st))
            sec = time_graph(torch, capi, one_pass, steps, warmup) / layers
            if n_th > 0:
                row['us_per_launch']["library's choice" if r == 0 else f'{r} x {w}'] = round(sec * 1e6, 2)
        rows.append(row)
        del sets
    return {'kernel': 'gemv_w4a16_kernel<M=1, plain>', 'launch_shapes': 'rows per lane x wavefronts per block', 'shapes': rows}


_SIDE_STREAM = None


def side_stream(torch):
    """One non-default stream for every recording and timed region of this run."""
    global _SIDE_STREAM
    if _SIDE_STREAM is None:
        _SIDE_STREAM = torch.cuda.Stream()
    return _SIDE_STREAM


def time_graph(torch, capi, fn, steps, warmup, warm_ms=0.0):
    """Records ``fn`` (which enqueues kernels on the current stream) in a HIP
    graph, replays it warmup + steps times, returns mean seconds per replay of
    the timed ones, measured with events on the replay stream.  ``warm_ms`` > 0
    keeps replaying until that much time has gone by: a kernel that loads the
    matrix cores for a millisecond at a time only settles at its sustained
    clock after some tens of milliseconds."""
    stream = side_stream(torch)
    with torch.cuda.stream(stream):
        fn()                                   # first call: compiles / loads modules, outside capture
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            fn()
        for _ in range(warmup):
            graph.replay()
        stream.synchronize()
        t_end = time.perf_counter() + warm_ms * 1e-3
        while warm_ms > 0 and time.perf_counter() < t_end:
            for _ in range(4):
                graph.replay()
            stream.synchronize()
        torch.cuda.synchronize()
        start, stop = capi.Event(), capi.Event()
        start.record(stream.cuda_stream)
        for _ in range(steps):
            graph.replay()
        stop.record(stream.cuda_stream)
        ms = start.elapsed_ms(stop)
        torch.cuda.synchronize()
    return ms * 1e-3 / steps


def bench_gemv(torch, autort, capi, workloads, K, N, M, steps, warmup, seed, layers=LAYERS, distinct=None):
    from antares_amd.autort import patterns
    dev = autort.device()
    op = autort.export(ir=patterns.W4A16_IR, inputs=patterns.W4A16_INPUTS, name='gemv_w4a16')
    p = workloads.w4_problem(seed, M, K, N)
    # distinct weight sets: same distribution, different bits (rolled copies), so no launch finds its data cached
    # (`distinct` < layers: the launches cycle through that many sets only)
    sets = []
    for l in range(layers if distinct is None else distinct):
        sets.append((torch.roll(p['qweight'], l, 0).to(dev), torch.roll(p['scales'], l, 0).to(dev), torch.roll(p['qzeros'], l, 0).to(dev)))
    sets = [sets[l % len(sets)] for l in range(layers)]
    x = p['x'].to(dev)
    ys = [torch.empty(M, N, dtype=torch.float16, device=dev) for _ in range(layers)]

    def one_pass():
        for (qw, sc, qz), y in zip(sets, ys):
            op(x, qw, sc, qz, out=y)
    sec = time_graph(torch, capi, one_pass, steps, warmup)
    per_launch = sec / layers
    by = workloads.w4_bytes(M, K, N)
    return {'workload': f"int4 g128 {'GEMV' if M <= 8 else 'GEMM'} M={M} K={K} N={N}", 'bytes_per_launch': by, 'launches_per_step': layers,
            'sec_per_step': sec, 'us_per_launch': per_launch * 1e6, 'gbps': by / per_launch / 1e9}


def bench_gemv_packed(torch, autort, capi, workloads, K, N, steps, warmup, seed, layers=LAYERS):
    """The same GEMV over weights repacked once by `autort.ops.w4_prepack` (tiles of 16 columns over all of K, one block
    per tile, no K-splits), timed exactly as `bench_gemv`: `layers` distinct weight sets per replayed graph.  The
    algorithmic bytes are those of the benchmark format (the packed form is 0.75 % larger)."""
    dev = autort.device()
    p = workloads.w4_problem(seed, 1, K, N)
    packs = []
    for l in range(layers):
        qw, sc, qz = (torch.roll(p[k], l, 0).to(dev) for k in ('qweight', 'scales', 'qzeros'))
        packs.append(autort.ops.w4_prepack(qw, sc, qz))
        del qw, sc, qz
    x = p['x'].to(dev).view(-1)
    ys = [torch.empty(N, dtype=torch.float16, device=dev) for _ in range(layers)]

    def one_pass():
        for pk, y in zip(packs, ys):
            autort.ops.gemv_w4p(x, pk, y, shape=(K, N))
    sec = time_graph(torch, capi, one_pass, steps, warmup) / layers
    by = workloads.w4_bytes(1, K, N)
    return {'workload': f'int4 g128 GEMV M=1 K={K} N={N}, weights repacked once (16 columns x K per block)',
            'us_per_launch': round(sec * 1e6, 3), 'gbps': round(by / sec / 1e9, 1), 'roofline_frac': round(by / sec / 1e9 / HBM_PEAK_GBPS, 4),
            'packed_bytes': int(packs[0].numel())}


def bench_gemm_f16(torch, autort, capi, workloads, steps, warmup, seed, n):
    from antares_amd.autort import patterns
    dev = autort.device()
    op = autort.export(ir=patterns.GEMM_F16_IR, inputs=patterns.GEMM_F16_INPUTS, name='gemm_f16')
    a, b = (t.to(dev) for t in workloads.gemm_inputs(seed, n))
    c = torch.empty(n, n, dtype=torch.float16, device=dev)
    sec = time_graph(torch, capi, lambda: op(a, b, out=c), steps, warmup, warm_ms=40.0)
    tflops = 2.0 * n * n * n / sec / 1e12
    return {'workload': f'fp16 GEMM M=N=K={n} (fp32 accumulate)', 'us_per_launch': sec * 1e6, 'tflops': tflops,
            'roofline_bound': 'mfma', 'roofline_frac': tflops / MFMA_F16_PEAK_TFLOPS}


def bench_gemm_f32(torch, autort, capi, steps, warmup, seed, n):
    """The float32 matrix product as AntaresIR.md:115 writes it (the README's `gemm_f32`), on the fp32 matrix instructions."""
    from antares_amd.autort import patterns
    dev = autort.device()
    op = autort.export(ir=patterns.GEMM_F32_IR, inputs=patterns.GEMM_F32_INPUTS, name='gemm_f32')
    g = torch.Generator('cpu').manual_seed(seed)
    a, b = (torch.randn(n, n, generator=g).to(dev) for _ in range(2))
    c = torch.empty(n, n, dtype=torch.float32, device=dev)
    sec = time_graph(torch, capi, lambda: op(a, b, out=c), steps, warmup, warm_ms=40.0)
    tflops = 2.0 * n * n * n / sec / 1e12
    return {'workload': f'fp32 GEMM M=N=K={n}', 'us_per_launch': sec * 1e6, 'tflops': tflops,
            'roofline_bound': 'mfma', 'roofline_frac': tflops / MFMA_F32_PEAK_TFLOPS}


def bench_sigmoid(torch, autort, capi, workloads, steps, warmup, seed, n=4_096_000, copies=16):
    dev = autort.device()
    op = autort.export(ir='sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))', inputs=['data=float32[N:4096000]'], config='tune:5')
    base = workloads.sigmoid_input(seed, n)
    xs = [torch.roll(base, i).to(dev) for i in range(copies)]
    outs = [torch.empty_like(x) for x in xs]

    def one_pass():
        for x, o in zip(xs, outs):
            op(x, out=o)
    sec = time_graph(torch, capi, one_pass, steps, warmup) / copies
    return {'workload': f'sigmoid f32 N={n}', 'bytes_per_launch': 8 * n, 'us_per_launch': sec * 1e6, 'gbps': 8 * n / sec / 1e9,
            'roofline_frac': 8 * n / sec / 1e9 / HBM_PEAK_GBPS}


def bench_partition(torch, autort, capi, workloads, steps, warmup, seed, n=16_777_216, copies=4):
    dev = autort.device()
    base = workloads.partition_input(seed, n)
    xs = [torch.roll(base, i).to(dev) for i in range(copies)]
    outs = [torch.empty_like(x) for x in xs]

    def one_pass():
        for x, o in zip(xs, outs):
            autort.ops.partition_even_first_i32(x, o)
    sec = time_graph(torch, capi, one_pass, max(5, steps // 5), warmup) / copies
    return {'workload': f'stable even-first partition int32 N={n}', 'bytes_per_launch': 8 * n, 'us_per_call': sec * 1e6,
            'gbps': 8 * n / sec / 1e9, 'roofline_frac': 8 * n / sec / 1e9 / HBM_PEAK_GBPS, 'melem_per_s': n / sec / 1e6}


def bench_decode(torch, autort, capi, seed, prompt_len=128, decode_steps=256, cpu_steps=0, att_parts=8):
    """BASELINE configuration 5: 32-layer Llama-2-7B-shaped int4 decode through autort.ops,
    batch 1, random-init weights, a 128-token random prompt fed token by token, then
    256 greedy steps; every step is one replay of the same recorded HIP graph.  The
    timed region is the 256 greedy steps."""
    from antares_amd.llama import LlamaConfig, LlamaInt4Decoder, random_weights
    cfg = LlamaConfig(max_seq=prompt_len + decode_steps)
    t0 = time.time()
    weights = random_weights(cfg, seed)
    gen_s = time.time() - t0
    dec = LlamaInt4Decoder(cfg, weights, att_parts=att_parts)
    g = torch.Generator().manual_seed(seed + 7)
    prompt = torch.randint(0, cfg.vocab, (prompt_len,), generator=g, dtype=torch.int64).to(torch.int32)
    prompt_dev = prompt.to(dec.dev)
    dec.capture(greedy=True, prompt=prompt_dev)
    stream = side_stream(torch)
    # the first greedy tokens of the replayed graph, to be compared with the eager 13-launch form further down
    check_steps = 8
    dec.key_cache.zero_()
    dec.val_cache.zero_()
    dec.reset(int(prompt[0]), 0)
    graph_tokens = []
    with torch.cuda.stream(stream):
        for _ in range(prompt_len - 1):
            dec.graph.replay()
        for _ in range(check_steps):
            dec.graph.replay()
            stream.synchronize()
            graph_tokens.append(int(dec.token.item()))
    dec.key_cache.zero_()
    dec.val_cache.zero_()
    dec.reset(int(prompt[0]), 0)
    tokens = []
    with torch.cuda.stream(stream):
        for _ in range(prompt_len - 1):          # positions 0 .. prompt_len-2 consume the prompt
            dec.graph.replay()
        stream.synchronize()
        start, stop = capi.Event(), capi.Event()
        start.record(stream.cuda_stream)
        for _ in range(decode_steps):
            dec.graph.replay()
        stop.record(stream.cuda_stream)
        ms = start.elapsed_ms(stop)
        stream.synchronize()
    sec_per_token = ms * 1e-3 / decode_steps
    mean_s = prompt_len - 1 + (decode_steps + 1) / 2.0           # mean attended length over the timed steps
    kv_bytes = cfg.n_layers * 2 * mean_s * cfg.dim * 2
    bytes_per_token = cfg.weight_bytes_per_token() + kv_bytes
    final_pos, last_token = int(dec.pos.item()), int(dec.token.item())
    # The same prompt taken in one pass (projections as batched int4 GEMMs on the matrix cores, causal attention over
    # the prompt): reported next to the decode rate, not part of it.
    dec.key_cache.zero_()
    dec.val_cache.zero_()
    dec.prefill(prompt_dev)                              # the first call builds and loads the operators of this length
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.prefill(prompt_dev)
    torch.cuda.synchronize()
    prefill_ms = (time.perf_counter() - t0) * 1e3
    # the same prompt and the first greedy steps through the decoder that mirrors the sample line by line (thirteen
    # launches per layer, one Python call per operator, no graph, split-K kernels over the benchmark layout)
    plain = LlamaInt4Decoder(cfg, weights, fused=False)
    plain.reset(int(prompt[0]), 0)
    eager_tokens = []
    for i in range(prompt_len - 1 + check_steps):
        plain.step()
        plain.advance(prompt_dev)
        if i >= prompt_len - 1:
            eager_tokens.append(int(plain.token.item()))
    del plain
    out = {'workload': f'Llama-2-7B-shaped int4 decode, {cfg.n_layers} layers, batch 1, prompt {prompt_len} + {decode_steps} greedy steps',
           'projections': 'q|k|v, gate|up, down, lm_head over weights repacked once (16 columns x K per block); o over the benchmark layout'
           if dec.packed else 'benchmark layout, split-K',
           'greedy_tokens_first_8': {'replayed_graph': graph_tokens, 'eager_13_launch_form': eager_tokens, 'equal': graph_tokens == eager_tokens},
           'tokens_per_s': round(1.0 / sec_per_token, 2), 'ms_per_token': round(sec_per_token * 1e3, 4),
           'weight_bytes_per_token': cfg.weight_bytes_per_token(), 'mean_kv_bytes_per_token': int(kv_bytes),
           'hbm_gbps': round(bytes_per_token / sec_per_token / 1e9, 1),
           'roofline_frac': round(bytes_per_token / sec_per_token / 1e9 / HBM_PEAK_GBPS, 4),
           'final_pos': final_pos, 'last_token': last_token,
           'prompt': 'fed token by token through the same graph', 'whole_prompt_prefill_ms': round(prefill_ms, 2),
           'weight_init_s': round(gen_s, 1)}
    if cpu_steps > 0:
        out['cpu_baseline'] = cpu_baseline_decode(cfg, weights, int(prompt[0]), cpu_steps)
    return out


def cpu_baseline_decode(cfg, weights, first_token, steps):
    """The oracle's decode step with its GEMVs on the rank-striding thread pool; `steps`
    positions from an empty cache (the weight stream, which dominates, does not depend on position)."""
    import numpy as np
    from antares_amd.autort import patterns
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule, threads
    from oracle.llama_ref import LlamaRef
    mod = CpuModule(parse_program(patterns.W4A16_IR, patterns.W4A16_INPUTS), nranks=256)

    def linear(x, lin):
        return mod(x=np.ascontiguousarray(x), qweight=lin['qweight'].numpy().view('int8'), scales=lin['scales'].numpy(),
                   qzeros=lin['qzeros'].numpy().view('int8'))['y']
    ref = LlamaRef(cfg, weights, linear=linear)
    tok = first_token
    t0 = time.perf_counter()
    for pos in range(steps):
        tok = int(np.argmax(ref.forward(tok, pos).astype(np.float32)))
    sec = (time.perf_counter() - t0) / steps
    return {'value': round(1.0 / sec, 4), 'unit': 'tokens/s', 'cores': threads(), 'kind': 'port',
            'sample': f'{steps} decode steps of the same 32-layer model from an empty cache, {sec:.2f} s per token'}


def cpu_baseline_gemv(workloads, K, N, M, seed, budget_s=15.0):
    """The CPU oracle (loop nests of the reference's CPU backend, same compiler
    flags, rank-striding thread pool) on the headline program."""
    from antares_amd.autort import patterns
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    p = workloads.w4_problem(seed, M, K, N)
    mod = CpuModule(parse_program(patterns.W4A16_IR, patterns.W4A16_INPUTS), nranks=256)
    t = mod.time(budget_s=budget_s, x=p['x'].numpy(), qweight=p['qweight'].numpy().view('int8'),
                 scales=p['scales'].numpy(), qzeros=p['qzeros'].numpy().view('int8'))
    by = workloads.w4_bytes(M, K, N)
    return {'value': by / t['seconds'] / 1e9, 'unit': 'GB/s', 'cores': t['threads'], 'kind': 'port',
            'sample': f'{t["runs"]} timed run(s) of the same GEMV (M={M} K={K} N={N}) after 1 warm-up + 1 probe, '
                      f'{t["seconds"] * 1e3:.1f} ms per run'}


def cpu_time_program(ir, inputs, tensors, budget_s):
    """Seconds per run of an einstein_v2 program on the CPU oracle (rank-striding thread pool, reference's flags)."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    return CpuModule(parse_program(ir, inputs), nranks=256).time(budget_s=budget_s, **tensors)


def cpu_baseline_extras(workloads, seed):
    """CPU oracle beside the other configurations, each on a bounded sample: workload name -> cpu_baseline object."""
    import numpy as np
    from antares_amd.autort import patterns
    from oracle import hot_ops
    out = {}
    # int4 GEMM, M = 64: the same program as the headline with 64 rows of x
    K, N, M, n_sample = 4096, 11008, 64, 2752          # a quarter of the columns: the loop nest costs the same per column
    p = workloads.w4_problem(seed, M, K, n_sample)
    t = cpu_time_program(patterns.W4A16_IR, patterns.W4A16_INPUTS,
                         dict(x=p['x'].numpy(), qweight=p['qweight'].numpy().view('int8'), scales=p['scales'].numpy(),
                              qzeros=p['qzeros'].numpy().view('int8')), budget_s=2.0)
    by = workloads.w4_bytes(M, K, n_sample)
    out[f'int4 g128 GEMM M={M} K={K} N={N}'] = {
        'value': round(by / t['seconds'] / 1e9, 4), 'unit': 'GB/s', 'cores': t['threads'], 'kind': 'port',
        'sample': f'{t["runs"]} timed run(s) of the same GEMM on {n_sample} of the {N} columns, {t["seconds"] * 1e3:.0f} ms per run'}
    # fp16 GEMM: a 1024^3 corner of the 4096^3 problem (the loop nest does 2 flop per step whatever the size)
    n = 1024
    a, b = workloads.gemm_inputs(seed, n)
    t = cpu_time_program(patterns.GEMM_F16_IR, patterns.GEMM_F16_INPUTS, dict(a=a.numpy(), b=b.numpy()), budget_s=4.0)
    out['fp16 GEMM M=N=K=4096 (fp32 accumulate)'] = {
        'value': round(2.0 * n ** 3 / t['seconds'] / 1e12, 5), 'unit': 'TFLOP/s', 'cores': t['threads'], 'kind': 'port',
        'sample': f'{t["runs"]} timed run(s) of the same program at M=N=K={n}, {t["seconds"] * 1e3:.0f} ms per run'}
    # sigmoid at full size
    n = 4_096_000
    x = workloads.sigmoid_input(seed, n)
    t = cpu_time_program('sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))', ['data=float32[N:4096000]'], dict(data=x.numpy()),
                         budget_s=2.0)
    out[f'sigmoid f32 N={n}'] = {'value': round(8 * n / t['seconds'] / 1e9, 3), 'unit': 'GB/s', 'cores': t['threads'], 'kind': 'port',
                                 'sample': f'{t["runs"]} timed run(s) at full size, {t["seconds"] * 1e3:.2f} ms per run'}
    # partition at full size: the plain-C restatement of the sample's three steps, one thread
    n = 16_777_216
    v = workloads.partition_input(seed, n).numpy()
    hot_ops.sort_even_first_i32(v)
    t0 = time.perf_counter()
    runs = 3
    for _ in range(runs):
        hot_ops.sort_even_first_i32(v)
    sec = (time.perf_counter() - t0) / runs
    out[f'stable even-first partition int32 N={n}'] = {
        'value': round(8 * n / sec / 1e9, 3), 'unit': 'GB/s', 'cores': 1, 'kind': 'port',
        'sample': f'{runs} timed run(s) at full size after 1 warm-up, {sec * 1e3:.1f} ms per run'}
    return out


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py: this build measures one GPU only (no collectives, no sharding); run with --gpus 1', file=sys.stderr)
        sys.exit(2)
    import torch
    import autort
    from antares_amd import workloads
    from antares_amd.runtime import capi
    capi.init(0)
    if args.calibrate_copy:
        print(json.dumps(calibrate_copy(torch, capi, *args.calibrate_copy)), flush=True)
        return
    if args.read_floor:
        print(json.dumps(bench_read_floor(torch, capi, args.steps, args.warmup)), flush=True)
        return
    if args.stream_floors:
        print(json.dumps(bench_stream_floors(torch, capi, args.steps, args.warmup)), flush=True)
        return
    if args.phase_chain:
        print(json.dumps(bench_phase_chain(torch, capi)), flush=True)
        return
    if args.attention:
        print(json.dumps(bench_attention(torch, autort, capi, args.steps, args.warmup)), flush=True)
        return
    if args.gemv_knobs:
        print(json.dumps(bench_gemv_knobs(torch, autort, capi, workloads, args.steps, args.warmup)), flush=True)
        return
    if args.lowering:
        bench_lowering(torch, autort, capi, args.steps, args.warmup)
        return
    K, N, M = 4096, 11008, 1
    head = bench_gemv(torch, autort, capi, workloads, K, N, M, args.steps, args.warmup, args.seed)
    result = {
        'metric': 'int4_gemv_hbm_gbps', 'value': round(head['gbps'], 2), 'unit': 'GB/s', 'n_gpus': 1,
        'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(head['sec_per_step'] * 1e3, 5),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'u4*f16->f32', 'data': 'synthetic',
        'config': {'workload': head['workload'], 'launches_per_step': head['launches_per_step'], 'group': 128,
                   'weights': 'uint8 [K/2,N] two nibbles along K; fp16 scale + 4-bit zero per group',
                   'distinct_weight_sets': head['launches_per_step'], 'timed_through': 'HIP graph replay'},
        'roofline': {'bound': 'hbm', 'achieved': round(head['gbps'], 2), 'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
                     'frac': round(head['gbps'] / HBM_PEAK_GBPS, 4), 'traffic': traffic_from_summary(),
                     'kernel': 'gemv_w4a16_kernel', 'bytes_per_launch': head['bytes_per_launch'],
                     'us_per_launch': round(head['us_per_launch'], 3)},
    }
    if not args.no_extra:
        # the floor of a single launch over the same weight bytes (no arithmetic), measured the same way
        result['roofline']['read_only_launch'] = bench_read_floor(torch, capi, args.steps, args.warmup)
        # the same launch timed as the reference's harness times a kernel (graph_evaluator/run_graph.cpp:214-236: the
        # same tensors in every run): the 22.5 MB of weights then come from the caches, not from HBM, so this is no
        # bandwidth figure - it is reported to show what the rotation of 32 weight sets above takes away
        same = bench_gemv(torch, autort, capi, workloads, K, N, M, args.steps, args.warmup, args.seed, layers=32, distinct=1)
        result['roofline']['same_tensors_every_launch'] = {
            'us_per_launch': round(same['us_per_launch'], 3), 'algorithmic_gbps': round(same['gbps'], 1),
            'note': 'weights served by the caches; not an HBM rate'}
        # the headline shape over weights repacked once (layout named in the row): reported beside the headline, which
        # stays on the benchmark's [K/2, N] layout
        result['roofline']['repacked_weights'] = bench_gemv_packed(torch, autort, capi, workloads, K, N, args.steps, args.warmup, args.seed)
        extra = []
        for (k, n) in [(4096, 4096), (11008, 4096), (4096, 32000)]:
            extra.append(bench_gemv_packed(torch, autort, capi, workloads, k, n, max(10, args.steps // 2), args.warmup, args.seed,
                                           layers=32 if n < 32000 else 8))
        for (k, n) in [(4096, 4096), (11008, 4096), (4096, 32000)]:
            r = bench_gemv(torch, autort, capi, workloads, k, n, 1, max(10, args.steps // 2), args.warmup, args.seed,
                           layers=32 if n < 32000 else 8)
            extra.append({'workload': r['workload'], 'us_per_launch': round(r['us_per_launch'], 3), 'gbps': round(r['gbps'], 1),
                          'roofline_frac': round(r['gbps'] / HBM_PEAK_GBPS, 4)})
        for (k, n) in [(4096, 4096), (4096, 11008), (11008, 4096), (4096, 32000)]:
            r = bench_gemv(torch, autort, capi, workloads, k, n, 64, max(10, args.steps // 2), args.warmup, args.seed, layers=8)
            tflops = 2.0 * 64 * k * n / (r['us_per_launch'] * 1e-6) / 1e12
            extra.append({'workload': r['workload'], 'us_per_launch': round(r['us_per_launch'], 3), 'gbps': round(r['gbps'], 1),
                          'roofline_frac': round(r['gbps'] / HBM_PEAK_GBPS, 4), 'tflops': round(tflops, 1),
                          'mfma_frac': round(tflops / MFMA_F16_PEAK_TFLOPS, 4)})
        for n in (4096, 8192):
            r = bench_gemm_f16(torch, autort, capi, workloads, max(5, args.steps // 4), args.warmup, args.seed, n)
            extra.append({k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()})
        r = bench_gemm_f32(torch, autort, capi, max(5, args.steps // 4), args.warmup, args.seed, 4096)
        extra.append({k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()})
        for fn in (bench_sigmoid, bench_partition):
            r = fn(torch, autort, capi, workloads, args.steps, args.warmup, args.seed)
            extra.append({k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()})
        if not args.no_cpu:
            cpu = cpu_baseline_extras(workloads, args.seed)
            for e in extra:
                if e['workload'] in cpu:
                    e['cpu_baseline'] = cpu[e['workload']]
        result['extra'] = extra
    if not args.no_decode:
        result['decode'] = bench_decode(torch, autort, capi, args.seed, cpu_steps=0 if args.no_cpu else args.decode_cpu_steps,
                                        att_parts=args.att_parts)
    if not args.no_cpu:
        result['cpu_baseline'] = cpu_baseline_gemv(workloads, K, N, M, args.seed)
        result['cpu_baseline']['value'] = round(result['cpu_baseline']['value'], 4)
    print(json.dumps(result), flush=True)


if __name__ == '__main__':
    main()
