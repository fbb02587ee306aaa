"""Recognition of operator patterns that have a hand-written gfx950 kernel.

A program is recognised by the canonical text of its fused statements (tensor
and axis names replaced by order of appearance), so the user's spelling of
names does not matter.  The part each of the caller's tensors plays is taken
from that same order: ``match`` returns the handler together with a map from
the registered program's tensor names (the handler's vocabulary: ``x``,
``qweight`` ...) to the caller's names.  A handler returns True when it ran the
operator, or False to leave it to the generic lowering (shapes it does not
cover).
"""
from __future__ import annotations

from typing import Callable, Dict, Optional, Tuple

from ctypes import c_void_p

import torch

from ..ir import Graph, fuse_elementwise, parse_program
from ..runtime import capi

_TABLE: Dict[str, Tuple[Callable, list]] = {}      # canonical key -> (handler, the registered program's tensor order)


def register(ir: str, inputs, handler: Callable):
    g = fuse_elementwise(parse_program(ir, inputs))
    key = g.canonical_key()
    _TABLE[key] = (handler, g.canonical_tensor_order())
    return key


def match(fused: Graph) -> Optional[Tuple[Callable, Dict[str, str]]]:
    """(handler, roles) for a recognised program, else None.  ``roles`` maps the registered program's tensor names
    to the names the caller's program uses for the tensors in the same places."""
    hit = _TABLE.get(fused.canonical_key())
    if hit is None or not _axes_span_their_dimensions(fused):
        return None
    handler, registered = hit
    return handler, dict(zip(registered, fused.canonical_tensor_order()))


def _axes_span_their_dimensions(fused: Graph) -> bool:
    """The canonical key drops extents, and the handlers take every size from the operands' shapes: a program that
    restricts an axis (`... where K in 100`, `... where M in 100`) spells the same statements but computes something
    else - a shorter sum, a smaller output.  Such a program is left to the generic lowering: a hand kernel is taken
    only when every axis that indexes a tensor dimension directly runs over exactly that dimension."""
    from ..ir.nodes import walk
    for st in fused.statements:
        extent = dict(st.data_axes + st.reduce_axes)
        uses = [(st.output, st.out_index)]
        uses += [(n.name, n.args) for n in walk(st.root) if n.kind == 'load']
        for name, index in uses:
            info = fused.tensors.get(name)
            if info is None:
                continue
            shape = list(info.shape)
            if len(index) != len(shape):
                continue                          # scalars (`[]` against `[1]`) carry no axis
            for ix, dim in zip(index, shape):
                if ix.kind == 'axis' and ix.name in extent and extent[ix.name] != dim:
                    return False
    return True


# ---------------------------------------------------------------------------
# int4 GEMV in the reference's weight format (samples/05_llama2_7b_int4.py:135-139)
# ---------------------------------------------------------------------------
GPTQ_GEMV_IR = """
  input1[S, N] = (qweight[S / 8, N] >> (S % 8 * 4)).call(strs.bitwise_and, 15) * input0[S].like(1)
  w[S, N] = scales[S / 128, N] * (input1[S, N] - 8)
  my_result[N] +=! input0[S] * w[S, N].to(input0.dtype())
"""


def _gptq_inputs(xdt: str, sdt: str):
    return [f'input0={xdt}[S:4096]', 'qweight=int32[L:512, N:12288]', f'scales={sdt}[K:32, N:12288]']


def _gptq_handler(op, bound, env, stream) -> bool:
    r = op.fast_roles
    x, q, s, out = bound[r['input0']], bound[r['qweight']], bound[r['scales']], bound[r['my_result']]
    x_f16, s_f16 = int(x.dtype == torch.float16), int(s.dtype == torch.float16)
    K, N = x.shape[0], q.shape[1]
    qp = q.data_ptr()
    if K % 128 or N % 4 or q.shape[0] * 8 != K or s.shape[0] * 128 != K or qp % 16:
        return False
    capi.check(capi.lib().art_gemv_gptq(c_void_p(x.data_ptr()), c_void_p(qp), c_void_p(s.data_ptr()),
                                       c_void_p(out.data_ptr()), K, N, x_f16, s_f16, c_void_p(stream)))
    return True


for _x in ('float32', 'float16'):
    for _s in ('float32', 'float16'):
        register(GPTQ_GEMV_IR, _gptq_inputs(_x, _s), _gptq_handler)


# ---------------------------------------------------------------------------
# int4 g128 GEMV / skinny GEMM with per-group zero points:
#   y[m,n] = sum_k x[m,k] * fp16( s[k/128,n] * (q[k,n] - z[k/128,n]) )     fp32 accumulate, fp16 out
# qweight uint8 [K/2,N] (low nibble = even k), qzeros uint8 [K/128,N/2] (low nibble = even n).
# ---------------------------------------------------------------------------
W4A16_IR = """
  acc[M, N] +=! x[M, K].to(`float32`) * (scales[K / 128, N] * (((qweight[K / 2, N] >> (K % 2 * 4)).call(strs.bitwise_and, 15) - (qzeros[K / 128, N / 2] >> (N % 2 * 4)).call(strs.bitwise_and, 15)) * scales[K / 128, N].like(1))).to(`float32`)
  y[M, N] = acc[M, N].to(`float16`)
"""
W4A16_INPUTS = ['x=float16[M:1, K:4096]', 'qweight=int8[KH:2048, N:11008]', 'scales=float16[G:32, N:11008]',
                'qzeros=int8[G:32, NH:5504]']


def tune_hand_kernel(op, key: str, candidates, run, trials: int, clones):
    """``config="tune:N"`` for a hand-written kernel: times up to N values of its launch parameter for the shape of
    this call (the reference's tuner walks the knob space of the schedule that runs, tuner/OpEvo/main.py:467-616; a
    hand kernel has one knob with a handful of values, so the walk is exhaustive up to N).  ``run(value, tensors)``
    enqueues one launch; ``clones`` yields sets of operand tensors - the timing rotates over several copies, since
    one buffer launched over and over would be served by the memory-side cache and favour the wrong choice - whose
    outputs are scratch, never the caller's.  The winner is kept in ``op.tuned[key]`` and in the module file."""
    sets = list(clones)
    stream = torch.cuda.current_stream().cuda_stream
    best = None
    for value in candidates[:max(1, trials)]:
        run(value, sets[0])                                   # warm-up (and the first use of a code path)
        start, stop = capi.Event(), capi.Event()
        start.record(stream)
        runs = max(6, 2 * len(sets))
        for i in range(runs):
            run(value, sets[i % len(sets)])
        stop.record(stream)
        us = start.elapsed_ms(stop) * 1e3 / runs
        if best is None or us < best['us']:
            best = {'value': int(value), 'us': round(us, 3)}
    op.tuned[key] = best
    op.persist()
    return best


def _w4a16_handler(op, bound, env, stream) -> bool:
    r = op.fast_roles
    x, q, s, z, y = bound[r['x']], bound[r['qweight']], bound[r['scales']], bound[r['qzeros']], bound[r['y']]
    M, K = x.shape
    N = q.shape[1]
    if K % 128 or N % 16 or q.shape[0] * 2 != K or s.shape[0] * 128 != K or z.shape[1] * 2 != N \
            or q.data_ptr() % 16 or x.data_ptr() % 16 or z.data_ptr() % 8 or y.data_ptr() % 8:
        return False
    # the vector-unit kernel streams the weights once per four rows (7.5 / 11.1 / 13.0 / 15.3 us for 1..4 rows of
    # 4096 x 11008, 22 us for five), the matrix-core kernel once per 64 rows (16 us for 4..32 rows): four rows and
    # more go there
    lib = capi.lib()
    gemv = M <= 3

    def run(value, t, st=None):
        args = (c_void_p(t[0].data_ptr()), c_void_p(t[1].data_ptr()), c_void_p(t[2].data_ptr()), c_void_p(t[3].data_ptr()),
                c_void_p(t[4].data_ptr()), M, K, N)
        if gemv:         # value = 16 * rows per lane + wavefronts per block (0: the library's choice of both)
            capi.check(lib.art_gemv_w4a16_knobs(*args, int(value) >> 4, int(value) & 15, c_void_p(stream if st is None else st)))
        else:
            capi.check(lib.art_gemm_w4a16_tuned(*args, int(value), c_void_p(stream if st is None else st)))

    # the launch parameters of the kernel that runs: (rows per lane, wavefronts per block) of the GEMV - two factors
    # searched as a product space, as the reference's tuner walks the factor spaces of a schedule's knobs
    # (tuner/OpEvo/main.py:154-293) -, (K-splits, rows per block) of the GEMM
    key = f"{'gemv_w4a16.rows_x16_plus_waves' if gemv else 'gemm_w4a16.k_splits'}|{M},{K},{N}"
    saved = op.tuned.get(key)
    trials = op.config.get('tune')
    if saved is None and isinstance(trials, int) and trials > 0 and not torch.cuda.is_current_stream_capturing():
        per_set = q.numel() + 2 * s.numel() + z.numel()
        copies = max(1, min(8, (256 << 20) // max(per_set, 1)))
        clones = [(x, q.clone(), s.clone(), z.clone(), torch.empty_like(y)) for _ in range(copies)]
        if gemv:
            cands = [16 * rows + waves for rows in (8, 4) for waves in ((4, 8) if M == 1 else (4,))]
        else:
            counts = [v for v in (1, 2, 3, 4, 5, 6, 8, 10, 12, 16, 20, 24, 32) if v <= K // 128]
            # 512 + v: v K-splits over blocks of 64 rows; 256 + v: over blocks of 32 rows (twice the blocks)
            cands = [0] + [512 + v for v in counts] + ([256 + v for v in counts] if M > 32 else [])
        saved = tune_hand_kernel(op, key, cands, lambda v, t: run(v, t, torch.cuda.current_stream().cuda_stream), trials, clones)
        del clones
    run(saved['value'] if saved is not None else 0, (x, q, s, z, y))
    return True


register(W4A16_IR, W4A16_INPUTS, _w4a16_handler)


# ---------------------------------------------------------------------------
# fp16 GEMM with fp32 accumulation: C[M,N] = A[M,K] @ B[K,N] (AntaresIR.md:115 with the casts that
# make the accumulator fp32)
# ---------------------------------------------------------------------------
GEMM_F16_IR = """
  acc[M, N] +=! a[M, K].to(`float32`) * b[K, N].to(`float32`)
  c[M, N] = acc[M, N].to(`float16`)
"""
GEMM_F16_INPUTS = ['a=float16[M:4096, K:4096]', 'b=float16[K:4096, N:4096]']


def _gemm_f16_handler(op, bound, env, stream) -> bool:
    r = op.fast_roles
    a, b, c = bound[r['a']], bound[r['b']], bound[r['c']]
    M, K = a.shape
    N = b.shape[1]
    if N % 8 or K % 64 or a.data_ptr() % 16 or b.data_ptr() % 16 or c.data_ptr() % 16:
        return False

    def run(value, t, st=None):
        capi.check(capi.lib().art_gemm_f16_tuned(c_void_p(t[0].data_ptr()), c_void_p(t[1].data_ptr()), c_void_p(t[2].data_ptr()), M, N, K,
                                                 int(value), c_void_p(stream if st is None else st)))
    # the launch parameter: threads per block (2 x 2 wavefronts of 128 x 128 outputs, or 2 x 4 of 128 x 64)
    key = f'gemm_f16.threads|{M},{K},{N}'
    saved = op.tuned.get(key)
    trials = op.config.get('tune')
    if saved is None and isinstance(trials, int) and trials > 0 and not torch.cuda.is_current_stream_capturing():
        saved = tune_hand_kernel(op, key, [256, 512], lambda v, t: run(v, t, torch.cuda.current_stream().cuda_stream), trials,
                                 [(a, b, torch.empty_like(c))])
    run(saved['value'] if saved is not None else 0, (a, b, c))
    return True


register(GEMM_F16_IR, GEMM_F16_INPUTS, _gemm_f16_handler)


# ---------------------------------------------------------------------------
# fp32 GEMM: C[M,N] = A[M,K] @ B[K,N] (AntaresIR.md:115 as written; the README's `gemm_f32`)
# ---------------------------------------------------------------------------
GEMM_F32_IR = 'c[M, N] +=! a[M, K] * b[K, N]'
GEMM_F32_INPUTS = ['a=float32[M:4096, K:4096]', 'b=float32[K:4096, N:4096]']


def _gemm_f32_handler(op, bound, env, stream) -> bool:
    r = op.fast_roles
    a, b, c = bound[r['a']], bound[r['b']], bound[r['c']]
    M, K = a.shape
    N = b.shape[1]
    # small products are left to the generic lowering: a launch of the tiled kernel needs a few hundred tiles to pay
    if N % 4 or K % 32 or N < 4 or M * N < 128 * 128 * 32 or a.data_ptr() % 16 or b.data_ptr() % 16:
        return False

    def run(_, t, st=None):
        capi.check(capi.lib().art_gemm_f32(c_void_p(t[0].data_ptr()), c_void_p(t[1].data_ptr()), c_void_p(t[2].data_ptr()), M, N, K,
                                          c_void_p(stream if st is None else st)))
    # the kernel has no launch parameter to search; a tuning run records its time for the shape in the module file
    key = f'gemm_f32|{M},{K},{N}'
    trials = op.config.get('tune')
    if key not in op.tuned and isinstance(trials, int) and trials > 0 and not torch.cuda.is_current_stream_capturing():
        tune_hand_kernel(op, key, [0], lambda v, t: run(v, t, torch.cuda.current_stream().cuda_stream), 1, [(a, b, torch.empty_like(c))])
    run(0, (a, b, c))
    return True


register(GEMM_F32_IR, GEMM_F32_INPUTS, _gemm_f32_handler)


# ---------------------------------------------------------------------------
# batched fp32 GEMM: C[B,M,N] = A[B,M,K] @ B[B,K,N] (AntaresIR.md:121)
# ---------------------------------------------------------------------------
BATCH_GEMM_F32_IR = 'c[B, M, N] +=! a[B, M, K] * b[B, K, N]'
BATCH_GEMM_F32_INPUTS = ['a=float32[B:3, M:1024, K:512]', 'b=float32[B:3, K:512, N:512]']


def _batch_gemm_f32_handler(op, bound, env, stream) -> bool:
    r = op.fast_roles
    a, b, c = bound[r['a']], bound[r['b']], bound[r['c']]
    batch, M, K = a.shape
    N = b.shape[2]
    # as for the single product: the tiled kernel needs a few hundred tiles to pay
    if N % 4 or K % 32 or N < 4 or batch > 65535 or batch * M * N < 128 * 128 * 32 or a.data_ptr() % 16 or b.data_ptr() % 16 \
            or (M * K) % 4 or (K * N) % 4:
        return False
    capi.check(capi.lib().art_gemm_f32_batched(c_void_p(a.data_ptr()), c_void_p(b.data_ptr()), c_void_p(c.data_ptr()), batch, M, N, K,
                                              c_void_p(stream)))
    return True


register(BATCH_GEMM_F32_IR, BATCH_GEMM_F32_INPUTS, _batch_gemm_f32_handler)


# ---------------------------------------------------------------------------
# fp32 GEMM with an operand stored the other way round: A as [K, M], B as [N, K] (a linear layer's weight)
# ---------------------------------------------------------------------------
def _gemm_f32_layout_handler(trans_a: bool, trans_b: bool):
    def handler(op, bound, env, stream) -> bool:
        r = op.fast_roles
        a, b, c = bound[r['a']], bound[r['b']], bound[r['c']]
        (K, M) = a.shape if trans_a else a.shape[::-1]
        N = b.shape[0] if trans_b else b.shape[1]
        if K % 32 or (not trans_b and N % 4) or (trans_a and M % 4) or M * N < 128 * 128 * 32 or a.data_ptr() % 16 or b.data_ptr() % 16:
            return False
        capi.check(capi.lib().art_gemm_f32_ex(c_void_p(a.data_ptr()), c_void_p(b.data_ptr()), c_void_p(c.data_ptr()), 1, M, N, K,
                                             int(trans_a), int(trans_b), c_void_p(stream)))
        return True
    return handler


register('c[M, N] +=! a[K, M] * b[K, N]', ['a=float32[K:512, M:512]', 'b=float32[K:512, N:512]'], _gemm_f32_layout_handler(True, False))
register('c[M, N] +=! a[M, K] * b[N, K]', ['a=float32[M:512, K:512]', 'b=float32[N:512, K:512]'], _gemm_f32_layout_handler(False, True))
register('c[M, N] +=! a[K, M] * b[N, K]', ['a=float32[K:512, M:512]', 'b=float32[N:512, K:512]'], _gemm_f32_layout_handler(True, True))
