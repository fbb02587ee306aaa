"""Recognition of operator patterns that have a hand-written gfx950 kernel.

A program is recognised by the canonical text of its fused statements (tensor
and axis names replaced by order of appearance), so the user's spelling of
names does not matter.  A handler returns True when it ran the operator, or
False to leave it to the generic lowering (shapes it does not cover).
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

from ctypes import c_void_p

from ..ir import Graph, fuse_elementwise, parse_program
from ..runtime import capi

_TABLE: Dict[str, Callable] = {}


def register(ir: str, inputs, handler: Callable):
    key = fuse_elementwise(parse_program(ir, inputs)).canonical_key()
    _TABLE[key] = handler
    return key


def match(fused: Graph) -> Optional[Callable]:
    return _TABLE.get(fused.canonical_key())


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


def _gptq_roles(op):
    """Which declared tensor is x, qweight, scales and the output (the ABI order is by name; roles go by dtype and
    rank).  Worked out once per operator."""
    roles = getattr(op, '_gptq_roles', None)
    if roles is None:
        g = op.fused
        names = {n: g.tensors[n] for n in g.abi_inputs}
        q_name = next(n for n, t in names.items() if t.dtype == 'int32')
        x_name = next(n for n, t in names.items() if len(t.shape) == 1)
        s_name = next(n for n in names if n not in (q_name, x_name))
        roles = (x_name, q_name, s_name, g.abi_outputs[0], int(names[x_name].dtype == 'float16'),
                 int(names[s_name].dtype == 'float16'))
        op._gptq_roles = roles
    return roles


def _gptq_handler(op, bound, env, stream) -> bool:
    x_name, q_name, s_name, out_name, x_f16, s_f16 = _gptq_roles(op)
    out = bound[out_name]
    x, q, s = bound[x_name], bound[q_name], bound[s_name]
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


def _w4a16_handler(op, bound, env, stream) -> bool:
    x, q, s, z, y = bound['x'], bound['qweight'], bound['scales'], bound['qzeros'], bound['y']
    M, K = x.shape
    N = q.shape[1]
    if K % 128 or N % 16 or q.shape[0] * 2 != K or s.shape[0] * 128 != K or z.shape[1] * 2 != N \
            or q.data_ptr() % 16 or x.data_ptr() % 16 or z.data_ptr() % 8 or y.data_ptr() % 8:
        return False
    # the vector-unit kernel streams the weights once per four rows (7.5 / 11.1 / 13.0 / 15.3 us for 1..4 rows of
    # 4096 x 11008, 22 us for five), the matrix-core kernel once per 64 rows (16 us for 4..32 rows): four rows and
    # more go there
    entry = capi.lib().art_gemv_w4a16 if M <= 3 else capi.lib().art_gemm_w4a16
    capi.check(entry(c_void_p(x.data_ptr()), c_void_p(q.data_ptr()), c_void_p(s.data_ptr()),
                                        c_void_p(z.data_ptr()), c_void_p(y.data_ptr()), M, K, N, c_void_p(stream)))
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
    a, b, c = bound['a'], bound['b'], bound['c']
    M, K = a.shape
    N = b.shape[1]
    if N % 8 or K % 64 or a.data_ptr() % 16 or b.data_ptr() % 16 or c.data_ptr() % 16:
        return False
    capi.check(capi.lib().art_gemm_f16(c_void_p(a.data_ptr()), c_void_p(b.data_ptr()), c_void_p(c.data_ptr()), M, N, K,
                                      c_void_p(stream)))
    return True


register(GEMM_F16_IR, GEMM_F16_INPUTS, _gemm_f16_handler)
