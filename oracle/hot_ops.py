"""TEST INFRASTRUCTURE ONLY — numpy-facing wrappers of libref_hotops.so (the
plain-C restatements in hot_ops.c).  Only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import this."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, 'libref_hotops.so')
        if not os.path.exists(path):
            subprocess.check_call(['make', '-s', '-C', _HERE, 'libref_hotops.so'])
        _lib = ctypes.CDLL(path)
    return _lib


def _p(a: np.ndarray):
    assert a.flags['C_CONTIGUOUS']
    return ctypes.c_void_p(a.ctypes.data)


def sigmoid_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().ref_sigmoid_f32(_p(x), _p(out), ctypes.c_longlong(x.size))
    return out


def sort_even_first_i32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.int32)
    out = np.empty_like(x)
    rc = lib().ref_sort_even_first_i32(_p(x), _p(out), ctypes.c_longlong(x.size))
    assert rc == 0
    return out


def gemm_w4a16(x, qweight, scales, qzeros) -> np.ndarray:
    """x fp16 [M,K], qweight uint8 [K/2,N], scales fp16 [K/128,N], qzeros uint8 [K/128,N/2] -> fp16 [M,N]."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    qweight = np.ascontiguousarray(qweight).view(np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.float16)
    qzeros = np.ascontiguousarray(qzeros).view(np.uint8)
    M, K = x.shape
    N = qweight.shape[1]
    assert qweight.shape[0] * 2 == K and scales.shape == (K // 128, N) and qzeros.shape == (K // 128, N // 2)
    y = np.empty((M, N), dtype=np.float16)
    lib().ref_gemm_w4a16(_p(x), _p(qweight), _p(scales), _p(qzeros), _p(y), M, K, N)
    return y


def gemv_gptq_f32(x, qweight, scales) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    qweight = np.ascontiguousarray(qweight, dtype=np.int32)
    scales = np.ascontiguousarray(scales)
    assert scales.dtype in (np.float32, np.float16)
    K, N = x.shape[0], qweight.shape[1]
    y = np.empty(N, dtype=np.float32)
    lib().ref_gemv_gptq_f32(_p(x), _p(qweight), _p(scales), int(scales.dtype == np.float16), _p(y), K, N)
    return y


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def rmsnorm(x, vsum, w, inv_n=None, eps=1e-5, out_dtype=np.float32) -> np.ndarray:
    """Inputs of any float dtype are widened exactly to fp32, the result is rounded to out_dtype."""
    x, w = _f32(x).reshape(-1), _f32(w).reshape(-1)
    out = np.empty_like(x)
    vs = None if vsum is None else _f32(vsum).reshape(-1)
    lib().ref_rmsnorm_f32(_p(x), _p(vs) if vs is not None else None, _p(w), _p(out), x.size,
                          ctypes.c_float(1.0 / x.size if inv_n is None else inv_n), ctypes.c_float(eps))
    return out.astype(out_dtype)


def rotary(x, inv_freq, pos: int) -> np.ndarray:
    """x: [heads, 2, half] (any float dtype); result has x's dtype and shape [heads, 2*half]."""
    dt = np.asarray(x).dtype
    xf, f = _f32(x), _f32(inv_freq).reshape(-1)
    heads, _, half = xf.shape
    out = np.empty((heads, 2 * half), np.float32)
    lib().ref_rotary_f32(_p(xf), _p(f), _p(out), heads, 2 * half, int(pos))
    return out.astype(dt)


def rotate(coef, data, pos: int) -> np.ndarray:
    dt = np.asarray(data).dtype
    c, d = _f32(coef).reshape(-1), _f32(data).reshape(-1)
    out = np.empty_like(d)
    lib().ref_rotate_f32(_p(c), _p(d), _p(out), d.size, int(pos))
    return out.astype(dt)


def attention(q, k, v, att_f: float) -> np.ndarray:
    """q [H,D], k/v [S,H,D] (any float dtype) -> [H,D] in q's dtype."""
    dt = np.asarray(q).dtype
    qf, kf, vf = _f32(q), _f32(k), _f32(v)
    S, H, D = kf.shape
    out = np.empty((H, D), np.float32)
    lib().ref_attention_f32(_p(qf), _p(kf), _p(vf), ctypes.c_float(att_f), _p(out), S, H, D)
    return out.astype(dt)
