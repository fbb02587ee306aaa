"""Operators that ship with the package: the fused partition and the Llama
decode operators.  Each is a thin Python wrapper that checks shapes on the
host and calls one typed entry point of libantares_amd.so."""
from __future__ import annotations

from ctypes import c_void_p

import torch

from ..runtime import capi
from .builtin import builtin
from .op import current_stream_handle


def _require_cuda(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError('autort built-in operators need GPU tensors; there is no CPU fallback')
        if not t.is_contiguous():
            raise ValueError('autort built-in operators need dense (contiguous) tensors')
    capi.init(tensors[0].device.index or 0)


class PartitionEvenFirst:
    """``autort.ops.partition_even_first_i32(x[, out])``: all even values of an
    int32 vector in input order, then all odd values in input order — the result
    of the classify / cumsum / bucket pipeline of samples/01_sort_even_first.py:9-27
    in one fused operator."""
    name = 'partition_even_first_i32'
    BLOCK_CAPS = (1024, 512, 2048, 256, 4096)          # values of the launch parameter a tuning run tries, default first

    def __init__(self):
        self.tuned = {}                                 # str(n) -> {'value': cap on blocks, 'us': ...}
        self._loaded = False

    def _saved(self):
        """Winners of earlier tuning runs, kept in the operator store as `partition_even_first_i32.tuned.json`."""
        if not self._loaded:
            self._loaded = True
            import json
            import os
            from . import store
            try:
                with open(os.path.join(store.ops_dir(), self.name + '.tuned.json')) as f:
                    self.tuned.update(json.load(f))
            except (OSError, ValueError):
                pass
        return self.tuned

    def persist(self):
        import json
        import os
        from . import store
        try:
            os.makedirs(store.ops_dir(), exist_ok=True)
            path = os.path.join(store.ops_dir(), self.name + '.tuned.json')
            with open(f'{path}.{os.getpid()}.tmp', 'w') as f:
                json.dump(self.tuned, f, sort_keys=True)
            os.replace(f'{path}.{os.getpid()}.tmp', path)
        except OSError:
            pass

    def _launch(self, x, out, cap):
        capi.check(capi.lib().art_partition_even_first_i32_tuned(c_void_p(x.data_ptr()), c_void_p(out.data_ptr()), x.numel(),
                                                                int(cap), c_void_p(current_stream_handle())))

    def tune(self, x: torch.Tensor, trials: int = 5):
        """Times up to `trials` caps on the number of blocks for vectors of x's length (on rotating copies of x, into
        scratch outputs) and keeps the fastest for later calls and later sessions; returns the record."""
        from .patterns import tune_hand_kernel
        _require_cuda(x)
        n = x.numel()
        copies = max(1, min(4, (256 << 20) // max(8 * n, 1)))
        clones = [(x if c == 0 else x.clone(), torch.empty_like(x)) for c in range(copies)]
        self.config = {}
        return tune_hand_kernel(self, str(n), list(self.BLOCK_CAPS), lambda v, t: self._launch(t[0], t[1], v), trials, clones)

    def __call__(self, x: torch.Tensor, out: torch.Tensor = None, extra=None):
        if x.dtype != torch.int32 or x.dim() != 1:
            raise TypeError('partition_even_first_i32 expects a 1-D int32 tensor')
        if out is None:
            out = torch.empty_like(x)
        if out.dtype != torch.int32 or out.numel() != x.numel():
            raise TypeError('partition_even_first_i32: out must be int32 with as many elements as the input')
        _require_cuda(x, out)
        saved = self._saved().get(str(x.numel()))
        self._launch(x, out, saved['value'] if saved else 0)
        return out


@builtin('partition_even_first_i32')
def _partition():
    return PartitionEvenFirst()


# ---------------------------------------------------------------------------
# Llama decode operators (call sites: samples/05_llama2_7b_int4.py:128-131,157-158,165)
# ---------------------------------------------------------------------------
_DT = {torch.float32: 0, torch.float16: 1}
RMS_EPS = 1e-5


def _dt(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _DT:
        raise TypeError(f'{what} must be float32 or float16, got {t.dtype}')
    return _DT[t.dtype]


def _pos_args(extra, what: str):
    """``extra=[pos]``: a Python int, or a 1-element int32 GPU tensor (read on the
    device, so a recorded HIP graph can be replayed for every position)."""
    if not extra:
        raise TypeError(f'{what} needs extra=[pos]')
    pos = extra[0]
    if isinstance(pos, torch.Tensor):
        if pos.dtype != torch.int32 or pos.numel() != 1 or not pos.is_cuda:
            raise TypeError(f'{what}: a tensor position must be a 1-element int32 GPU tensor')
        return c_void_p(pos.data_ptr()), 0
    return c_void_p(0), int(pos)


class RmsNorm:
    """``rmsnorm_f32(x[N], vsum[1], w[N], extra=[1/N]) -> out[N]``:
    ``out = x * rsqrt(vsum * extra[0] + eps) * w`` with eps = 1e-5 (``extra[1]``
    overrides it).  ``vsum`` is the caller's fp32 sum of squares; passing ``None``
    lets the kernel compute it.  ``x`` may also be [rows, N] with one vsum per row."""

    def __init__(self, out_dtype: torch.dtype):
        self.out_dtype = out_dtype
        self.name = 'rmsnorm_f32' if out_dtype == torch.float32 else 'rmsnorm_f16'

    def __call__(self, x, vsum, w, out=None, extra=None):
        n = w.numel()
        rows = x.numel() // n
        if rows * n != x.numel() or n == 0:
            raise ValueError(f'{self.name}: x has {x.numel()} elements, weight {n}')
        inv_n = float(extra[0]) if extra else 1.0 / n
        eps = float(extra[1]) if extra and len(extra) > 1 else RMS_EPS
        if out is None:
            out = torch.empty(x.shape, dtype=self.out_dtype, device=x.device)
        if out.numel() != x.numel():
            raise ValueError(f'{self.name}: out has the wrong size')
        tensors = [x, w, out]
        vptr = c_void_p(0)
        if vsum is not None:
            vsum = vsum.view(-1)
            if vsum.dtype != torch.float32 or vsum.numel() != rows:
                raise TypeError(f'{self.name}: vsum must be float32 with one value per row')
            tensors.append(vsum)
            vptr = c_void_p(vsum.data_ptr())
        _require_cuda(*tensors)
        capi.check(capi.lib().art_rmsnorm(c_void_p(x.data_ptr()), vptr, c_void_p(w.data_ptr()), c_void_p(out.data_ptr()),
                                         rows, n, inv_n, eps, _dt(x, 'x'), _dt(w, 'weight'), _dt(out, 'out'),
                                         c_void_p(current_stream_handle())))
        return out


class Rotary:
    """``rotary_f32(x[H,2,D/2], inv_freq[D], out[H,D], extra=[pos])`` (rotate-half
    form) and ``rotate_f32(coef[1,dim/2], data[dim], out[dim], extra=[pos])``
    (interleaved pairs, samples/03_llama_tiny.py:68-70)."""

    def __init__(self, name: str, interleaved: bool):
        self.name, self.interleaved = name, interleaved

    def __call__(self, a, b, out=None, extra=None):
        x, freq = (b, a) if self.interleaved else (a, b)
        if out is None:
            out = torch.empty_like(x)
        if self.interleaved:
            heads, head_dim = 1, x.numel()
            if freq.numel() * 2 != x.numel():
                raise ValueError(f'{self.name}: coefficient tensor must have one entry per pair')
        else:
            if x.dim() != 3 or x.shape[1] != 2:
                raise ValueError(f'{self.name}: x must be viewed as [heads, 2, head_dim/2]')
            heads, head_dim = x.shape[0], 2 * x.shape[2]
            if freq.numel() < head_dim // 2:
                raise ValueError(f'{self.name}: inv_freq is too short')
        _require_cuda(x, freq, out)
        pos_dev, pos = _pos_args(extra, self.name)
        stride, out_rows = 0, 0
        if out.numel() != x.numel():
            # a whole [positions, heads*head_dim] cache: the row is chosen by the device-side position
            if not pos_dev.value or out.numel() % x.numel() != 0:
                raise ValueError(f'{self.name}: out must match x in size (or be a cache with extra=[position tensor])')
            stride, out_rows = x.numel(), out.numel() // x.numel()
        if out.dtype != x.dtype:
            raise ValueError(f'{self.name}: out must have the dtype of x')
        capi.check(capi.lib().art_rotary(c_void_p(x.data_ptr()), c_void_p(freq.data_ptr()), c_void_p(out.data_ptr()), heads,
                                        head_dim, int(self.interleaved), pos_dev, pos, stride, out_rows, _dt(x, 'x'), _dt(freq, 'inv_freq'),
                                        _dt(out, 'out'), c_void_p(current_stream_handle())))
        return out


class DecodeAttention:
    """``attention_f32(q[H,D], k[S,H,D], v[S,H,D], att_f[1]) -> out[H,D]``: scores
    ``att_f * q.k``, softmax over S, weighted sum of v (the torch spelling is at
    samples/03_llama_tiny.py:94-99).  ``extra=[pos]`` with a 1-element int32 GPU
    tensor makes the kernel use S = pos + 1 read on the device (k, v are then the
    whole cache)."""

    def __init__(self, name: str):
        self.name = name

    def __call__(self, q, k, v, att_f, out=None, extra=None):
        if q.dim() != 2 or k.dim() != 3 or k.shape != v.shape or k.shape[1:] != q.shape:
            raise ValueError(f'{self.name}: expected q[H,D], k[S,H,D], v[S,H,D]; got {list(q.shape)}, {list(k.shape)}, {list(v.shape)}')
        if att_f.dtype != torch.float32 or att_f.numel() != 1:
            raise TypeError(f'{self.name}: att_f must be a 1-element float32 tensor')
        if k.dtype != v.dtype:
            raise TypeError(f'{self.name}: k and v must have the same dtype')
        if out is None:
            out = torch.empty_like(q)
        _require_cuda(q, k, v, att_f, out)
        pos_dev = c_void_p(0)
        if extra and isinstance(extra[0], torch.Tensor):
            pos_dev, _ = _pos_args(extra, self.name)
        capi.check(capi.lib().art_decode_attention(c_void_p(q.data_ptr()), c_void_p(k.data_ptr()), c_void_p(v.data_ptr()),
                                                  c_void_p(att_f.data_ptr()), c_void_p(out.data_ptr()), k.shape[0], q.shape[0],
                                                  q.shape[1], pos_dev, _dt(q, 'q'), _dt(k, 'k'), _dt(out, 'out'),
                                                  c_void_p(current_stream_handle())))
        return out


class CausalAttention:
    """``attention_causal_f16(q[T,H,D], k[S,H,D], v[S,H,D], att_f[1]) -> out[T,H,D]`` with S >= T: position t attends to
    rows 0..t of k and v (views of the key / value cache), i.e. ``attention_f16`` for the T positions of a prompt in
    one launch on the matrix cores."""
    name = 'attention_causal_f16'

    def __call__(self, q, k, v, att_f, out=None, extra=None):
        if q.dim() != 3 or k.dim() != 3 or k.shape != v.shape or k.shape[1:] != q.shape[1:] or k.shape[0] < q.shape[0]:
            raise ValueError(f'{self.name}: expected q[T,H,D], k[S,H,D], v[S,H,D] with S >= T; got {list(q.shape)}, {list(k.shape)}, {list(v.shape)}')
        for t in (q, k, v):
            if t.dtype != torch.float16:
                raise TypeError(f'{self.name}: q, k and v must be float16')
        if att_f.dtype != torch.float32 or att_f.numel() != 1:
            raise TypeError(f'{self.name}: att_f must be a 1-element float32 tensor')
        if out is None:
            out = torch.empty_like(q)
        if out.dtype != torch.float16 or out.shape != q.shape:
            raise TypeError(f'{self.name}: out must be float16 of the shape of q')
        _require_cuda(q, k, v, att_f, out)
        T, H, D = q.shape
        capi.check(capi.lib().art_prefill_attention(c_void_p(q.data_ptr()), c_void_p(k.data_ptr()), c_void_p(v.data_ptr()),
                                                   c_void_p(att_f.data_ptr()), c_void_p(out.data_ptr()), T, H, D, H * D,
                                                   c_void_p(current_stream_handle())))
        return out


builtin('attention_causal_f16')(lambda: CausalAttention())
builtin('rmsnorm_f32')(lambda: RmsNorm(torch.float32))
builtin('rmsnorm_f16')(lambda: RmsNorm(torch.float16))
builtin('rotary_f32')(lambda: Rotary('rotary_f32', False))
builtin('rotary_f16')(lambda: Rotary('rotary_f16', False))
builtin('rotate_f32')(lambda: Rotary('rotate_f32', True))
builtin('rotate_f16')(lambda: Rotary('rotate_f16', True))
builtin('attention_f32')(lambda: DecodeAttention('attention_f32'))
builtin('attention_f16')(lambda: DecodeAttention('attention_f16'))


SUMSQ_WORDS = 256      # 64-bit words of a sum-of-squares buffer (one per 128 columns of the projection that fills it)


def _sumsq_buffers(who, *buffers):
    given = [b for b in buffers if b is not None]
    for b in given:
        if b.dtype != torch.int64 or b.numel() != SUMSQ_WORDS or not b.is_contiguous():
            raise TypeError(f'{who}: a sum-of-squares buffer is a contiguous int64 tensor of {SUMSQ_WORDS} words')
    return given


def _ptr_or_null(t):
    return c_void_p(t.data_ptr() if t is not None else 0)


class GemvW4Fused:
    """``gemv_w4a16_fused(x[K], qweight, scales, qzeros, out[N], norm_weight=None, residual=None, eps=1e-5)``:
    the packed int4 GEMV with an RMSNorm of its input and/or a residual add of its output folded in
    (the operators around every projection of the decode step, samples/05_llama2_7b_int4.py:150-173)."""
    name = 'gemv_w4a16_fused'

    def __call__(self, x, qweight, scales, qzeros, out=None, norm_weight=None, residual=None, eps=RMS_EPS, swiglu=False,
                 extra=None, sumsq_in=None, sumsq_out=None, sumsq_clear=None):
        """``swiglu=True``: ``x`` holds gate | up (2*K values) and the product is taken with silu(gate) * up.
        ``sumsq_*``: int64[256] buffers that hand sum(y^2) from the projection that writes a residual stream
        (``sumsq_out``, which also zeroes ``sumsq_clear`` for the next writer) to the one that normalises it
        (``sumsq_in`` with ``norm_weight``), see ``art_gemv_w4a16_fused_sumsq``."""
        K, N = qweight.shape[0] * 2, qweight.shape[1]
        if x.numel() != (2 * K if swiglu else K):
            raise ValueError('gemv_w4a16_fused: x has the wrong length')
        if x.dtype != torch.float16 or scales.dtype != torch.float16:
            raise TypeError('gemv_w4a16_fused: x and scales must be float16')
        if qweight.shape[0] * 2 != K or scales.shape != (K // 128, N) or qzeros.shape != (K // 128, N // 2):
            raise ValueError('gemv_w4a16_fused: operand shapes do not match K, N')
        if out is None:
            out = torch.empty(N, dtype=torch.float16, device=x.device)
        tensors = [x, qweight, scales, qzeros, out]
        for t, what in ((norm_weight, 'norm_weight'), (residual, 'residual')):
            if t is not None:
                if t.dtype != torch.float16 or t.numel() != (K if what == 'norm_weight' else N):
                    raise TypeError(f'gemv_w4a16_fused: {what} must be float16 of matching length')
                tensors.append(t)
        tensors += _sumsq_buffers('gemv_w4a16_fused', sumsq_in, sumsq_out, sumsq_clear)
        _require_cuda(*tensors)
        capi.check(capi.lib().art_gemv_w4a16_fused_sumsq(
            c_void_p(x.data_ptr()), c_void_p(qweight.data_ptr()), c_void_p(scales.data_ptr()), c_void_p(qzeros.data_ptr()),
            c_void_p(out.data_ptr()), K, N, c_void_p(norm_weight.data_ptr() if norm_weight is not None else 0), float(eps),
            c_void_p(residual.data_ptr() if residual is not None else 0), int(bool(swiglu)), _ptr_or_null(sumsq_in),
            _ptr_or_null(sumsq_out), _ptr_or_null(sumsq_clear), c_void_p(current_stream_handle())))
        return out


class W4Prepack:
    """``w4_prepack(qweight[K/2, N], scales[K/128, N], qzeros[K/128, N/2]) -> packed``: the one-time repacking of an
    int4 matrix for ``gemv_w4p`` - tiles of 16 columns over all of K stored contiguously, in the order the kernel's
    wavefronts read them (the load-time weight preparation of samples/05_llama2_7b_int4.py:34-66).  ``packed`` is a
    uint8 tensor that remembers K and N (``packed.w4_shape``)."""
    name = 'w4_prepack'

    def __call__(self, qweight, scales, qzeros, out=None, extra=None):
        K, N = qweight.shape[0] * 2, qweight.shape[1]
        if qweight.dtype != torch.uint8 or qzeros.dtype != torch.uint8 or scales.dtype != torch.float16:
            raise TypeError('w4_prepack: qweight and qzeros must be uint8, scales float16')
        if scales.shape != (K // 128, N) or qzeros.shape != (K // 128, N // 2):
            raise ValueError('w4_prepack: operand shapes do not match K, N')
        nbytes = capi.lib().art_w4_prepack_bytes(K, N)
        if nbytes == 0:
            raise ValueError(f'w4_prepack: unsupported shape K={K} N={N} (K % 128 == 0, K <= 16384, N % 16 == 0)')
        if out is None:
            out = torch.empty(nbytes, dtype=torch.uint8, device=qweight.device)
        elif out.dtype != torch.uint8 or out.numel() != nbytes or not out.is_contiguous():
            raise TypeError(f'w4_prepack: out must be a contiguous uint8 tensor of {nbytes} bytes')
        for t in (qweight, scales, qzeros):
            if not t.is_contiguous():
                raise ValueError('w4_prepack: operands must be contiguous')
        _require_cuda(qweight, scales, qzeros, out)
        capi.check(capi.lib().art_w4_prepack(c_void_p(qweight.data_ptr()), c_void_p(scales.data_ptr()), c_void_p(qzeros.data_ptr()),
                                            c_void_p(out.data_ptr()), K, N, c_void_p(current_stream_handle())))
        out.w4_shape = (K, N)
        return out


class GemvW4Packed:
    """``gemv_w4p(x[K], packed, out=None, norm_weight=None, residual=None, eps=1e-5, swiglu_out=False, shape=None)``:
    the int4 GEMV over weights repacked by ``w4_prepack`` - one block per 16 columns over all of K, no K-splits.
    ``norm_weight``: RMSNorm of x folded in; ``residual``: added to the rounded product (``out`` may be the residual);
    ``swiglu_out``: the matrix holds gate and up columns interleaved in blocks of 8 (``interleave_gate_up``) and
    ``out[N/2]`` receives fp16(silu(gate) * up).  ``shape`` = (K, N) when ``packed`` does not carry ``w4_shape``."""
    name = 'gemv_w4p'

    def __call__(self, x, packed, out=None, norm_weight=None, residual=None, eps=RMS_EPS, swiglu_out=False, shape=None, extra=None):
        K, N = shape if shape is not None else getattr(packed, 'w4_shape', (None, None))
        if K is None:
            raise ValueError('gemv_w4p: pass shape=(K, N) or a tensor returned by w4_prepack')
        if x.dtype != torch.float16 or x.numel() != K:
            raise TypeError(f'gemv_w4p: x must be float16 of {K} values')
        if packed.dtype != torch.uint8 or packed.numel() != capi.lib().art_w4_prepack_bytes(K, N):
            raise ValueError('gemv_w4p: packed does not have the size of a repacked K x N matrix')
        n_out = N // 2 if swiglu_out else N
        if out is None:
            out = torch.empty(n_out, dtype=torch.float16, device=x.device)
        elif out.dtype != torch.float16 or out.numel() != n_out:
            raise TypeError(f'gemv_w4p: out must be float16 of {n_out} values')
        tensors = [x, packed, out]
        for t, what, n in ((norm_weight, 'norm_weight', K), (residual, 'residual', N)):
            if t is not None:
                if t.dtype != torch.float16 or t.numel() != n:
                    raise TypeError(f'gemv_w4p: {what} must be float16 of {n} values')
                tensors.append(t)
        _require_cuda(*tensors)
        capi.check(capi.lib().art_gemv_w4p(c_void_p(x.data_ptr()), c_void_p(packed.data_ptr()), c_void_p(out.data_ptr()), K, N,
                                          _ptr_or_null(norm_weight), float(eps), _ptr_or_null(residual), int(bool(swiglu_out)),
                                          c_void_p(current_stream_handle())))
        return out


def interleave_gate_up(gate: dict, up: dict) -> dict:
    """Columns of two int4 matrices of the same shape (dicts of qweight / scales / qzeros) interleaved in blocks of 8:
    g0..g7 u0..u7 g8..g15 u8..u15 ... - the column order ``gemv_w4p(swiglu_out=True)`` expects, so that a block of 16
    columns holds 8 gate columns and the matching 8 up columns."""
    def mix(a, b, cols_per_elem):
        blk = 8 // cols_per_elem          # elements of the last axis that make 8 columns
        rows, n = a.shape
        return torch.stack([a.view(rows, n // blk, blk), b.view(rows, n // blk, blk)], dim=2).reshape(rows, 2 * n).contiguous()
    return {'qweight': mix(gate['qweight'], up['qweight'], 1), 'scales': mix(gate['scales'], up['scales'], 1),
            'qzeros': mix(gate['qzeros'], up['qzeros'], 2)}


builtin('w4_prepack')(lambda: W4Prepack())
builtin('gemv_w4p')(lambda: GemvW4Packed())


class AttentionRope:
    """``attention_rope_f16(qkv[3*H*D], inv_freq[D], key_cache[S,H*D], val_cache[S,H*D], att_f[1], out[H,D], extra=[pos_tensor])``:
    rotary embedding of q and k, both cache writes and the attention over rows 0..pos, one launch per layer."""
    name = 'attention_rope_f16'

    def __call__(self, qkv, inv_freq, key_cache, val_cache, att_f, out, extra=None):
        heads, head_dim = out.shape
        if qkv.numel() != 3 * heads * head_dim or key_cache.shape[-1] != heads * head_dim or val_cache.shape != key_cache.shape:
            raise ValueError('attention_rope_f16: shapes do not fit together')
        for t in (qkv, inv_freq, key_cache, val_cache, out):
            if t.dtype != torch.float16:
                raise TypeError('attention_rope_f16: tensors must be float16')
        if att_f.dtype != torch.float32 or att_f.numel() != 1:
            raise TypeError('attention_rope_f16: att_f must be a 1-element float32 tensor')
        _require_cuda(qkv, inv_freq, key_cache, val_cache, att_f, out)
        pos_dev, _ = _pos_args(extra, self.name)
        if not pos_dev.value:
            raise TypeError('attention_rope_f16: extra=[pos] must be a 1-element int32 GPU tensor')
        capi.check(capi.lib().art_decode_attention_rope(c_void_p(qkv.data_ptr()), c_void_p(inv_freq.data_ptr()),
                                                       c_void_p(key_cache.data_ptr()), c_void_p(val_cache.data_ptr()),
                                                       c_void_p(att_f.data_ptr()), c_void_p(out.data_ptr()), heads, head_dim, pos_dev,
                                                       key_cache.numel() // (heads * head_dim), c_void_p(current_stream_handle())))
        return out


class AttentionRopeSplit:
    """``attention_rope_split_f16(qkv[3*H*D], inv_freq[D], key_cache, val_cache, att_f[1], partial[H, P, 132], extra=[pos_tensor])``:
    ``attention_rope_f16`` spread over P blocks per head.  ``partial`` (float32) receives, per head and part, 128
    unnormalised sums, the running maximum and the running sum; ``gemv_w4a16_attn`` merges them while it loads x."""
    name = 'attention_rope_split_f16'

    def __call__(self, qkv, inv_freq, key_cache, val_cache, att_f, partial, extra=None):
        if partial.dim() != 3 or partial.shape[2] != 132 or partial.dtype != torch.float32:
            raise TypeError('attention_rope_split_f16: partial must be float32 [heads, parts, 132]')
        heads, parts = partial.shape[0], partial.shape[1]
        head_dim = key_cache.shape[-1] // heads
        if qkv.numel() != 3 * heads * head_dim or val_cache.shape != key_cache.shape or not 2 <= parts <= 8:
            raise ValueError('attention_rope_split_f16: shapes do not fit together (2..8 parts)')
        for t in (qkv, inv_freq, key_cache, val_cache):
            if t.dtype != torch.float16:
                raise TypeError('attention_rope_split_f16: qkv, inv_freq and the caches must be float16')
        if att_f.dtype != torch.float32 or att_f.numel() != 1:
            raise TypeError('attention_rope_split_f16: att_f must be a 1-element float32 tensor')
        _require_cuda(qkv, inv_freq, key_cache, val_cache, att_f, partial)
        pos_dev, _ = _pos_args(extra, self.name)
        if not pos_dev.value:
            raise TypeError('attention_rope_split_f16: extra=[pos] must be a 1-element int32 GPU tensor')
        capi.check(capi.lib().art_decode_attention_rope_split(
            c_void_p(qkv.data_ptr()), c_void_p(inv_freq.data_ptr()), c_void_p(key_cache.data_ptr()), c_void_p(val_cache.data_ptr()),
            c_void_p(att_f.data_ptr()), c_void_p(partial.data_ptr()), heads, head_dim, pos_dev,
            key_cache.numel() // (heads * head_dim), parts,
            c_void_p(current_stream_handle())))
        return partial


class GemmW4Residual:
    """``gemm_w4a16_residual(x[M,K], qweight, scales, qzeros, out[M,N], residual=None)``: the packed int4 product for a
    batch of rows on the matrix cores with the residual add folded in (``out`` may be the residual itself)."""
    name = 'gemm_w4a16_residual'

    def __call__(self, x, qweight, scales, qzeros, out, residual=None):
        M, K = x.shape
        N = qweight.shape[1]
        if qweight.shape[0] * 2 != K or scales.shape != (K // 128, N) or qzeros.shape != (K // 128, N // 2) or out.shape != (M, N):
            raise ValueError('gemm_w4a16_residual: operand shapes do not match M, K, N')
        if x.dtype != torch.float16 or scales.dtype != torch.float16 or out.dtype != torch.float16 or \
                (residual is not None and (residual.dtype != torch.float16 or residual.shape != out.shape)):
            raise TypeError('gemm_w4a16_residual: x, scales, out and residual must be float16 (residual of the shape of out)')
        _require_cuda(*([x, qweight, scales, qzeros, out] + ([residual] if residual is not None else [])))
        capi.check(capi.lib().art_gemm_w4a16_residual(
            c_void_p(x.data_ptr()), c_void_p(qweight.data_ptr()), c_void_p(scales.data_ptr()), c_void_p(qzeros.data_ptr()),
            c_void_p(out.data_ptr()), c_void_p(residual.data_ptr() if residual is not None else 0), M, K, N, 0,
            c_void_p(current_stream_handle())))
        return out


builtin('gemm_w4a16_residual')(lambda: GemmW4Residual())


class GemvW4Attn:
    """``gemv_w4a16_attn(partial[H, P, 132], qweight, scales, qzeros, out[N], residual=None)``: the int4 projection of a
    split attention's output (merged on the fly) with the residual add folded in."""
    name = 'gemv_w4a16_attn'

    def __call__(self, partial, qweight, scales, qzeros, out, residual=None, sumsq_out=None, sumsq_clear=None):
        K, N = qweight.shape[0] * 2, qweight.shape[1]
        if partial.dim() != 3 or partial.shape[2] != 132 or partial.dtype != torch.float32 or partial.shape[0] * 128 != K:
            raise TypeError('gemv_w4a16_attn: partial must be float32 [K/128, parts, 132]')
        if scales.shape != (K // 128, N) or qzeros.shape != (K // 128, N // 2) or out.numel() != N:
            raise ValueError('gemv_w4a16_attn: operand shapes do not match K, N')
        if scales.dtype != torch.float16 or out.dtype != torch.float16 or (residual is not None and residual.dtype != torch.float16):
            raise TypeError('gemv_w4a16_attn: scales, out and residual must be float16')
        _require_cuda(*([partial, qweight, scales, qzeros, out] + ([residual] if residual is not None else []) +
                        _sumsq_buffers('gemv_w4a16_attn', sumsq_out, sumsq_clear)))
        capi.check(capi.lib().art_gemv_w4a16_attn_sumsq(
            c_void_p(partial.data_ptr()), partial.shape[1], c_void_p(qweight.data_ptr()), c_void_p(scales.data_ptr()),
            c_void_p(qzeros.data_ptr()), c_void_p(out.data_ptr()), K, N,
            c_void_p(residual.data_ptr() if residual is not None else 0), _ptr_or_null(sumsq_out), _ptr_or_null(sumsq_clear),
            c_void_p(current_stream_handle())))
        return out


class RopeQkvStore:
    """``rope_qkv_store_f16(qkv[3*H*D], inv_freq[D], q_out[H,D], key_cache[S,H*D], val_cache[S,H*D], extra=[pos_tensor])``:
    rotary embedding of q and k (k straight into its cache row) and the copy of v into its cache row, one launch."""

    def __init__(self, name):
        self.name = name

    def __call__(self, qkv, inv_freq, q_out, key_cache, val_cache, extra=None):
        heads, head_dim = q_out.shape
        if qkv.numel() != 3 * heads * head_dim or key_cache.shape[-1] != heads * head_dim or val_cache.shape != key_cache.shape:
            raise ValueError(f'{self.name}: shapes do not fit together')
        if not (qkv.dtype == q_out.dtype == key_cache.dtype == val_cache.dtype):
            raise TypeError(f'{self.name}: qkv, q_out and the caches must share one dtype')
        _require_cuda(qkv, inv_freq, q_out, key_cache, val_cache)
        pos_dev, _ = _pos_args(extra, self.name)
        if not pos_dev.value:
            raise TypeError(f'{self.name}: extra=[pos] must be a 1-element int32 GPU tensor')
        capi.check(capi.lib().art_rope_qkv_store(c_void_p(qkv.data_ptr()), c_void_p(inv_freq.data_ptr()), c_void_p(q_out.data_ptr()),
                                                c_void_p(key_cache.data_ptr()), c_void_p(val_cache.data_ptr()), heads, head_dim,
                                                pos_dev, key_cache.numel() // (heads * head_dim), _dt(qkv, 'qkv'), _dt(inv_freq, 'inv_freq'), c_void_p(current_stream_handle())))
        return q_out


class RopeQkvStoreRows:
    """``rope_qkv_store_rows_f16(qkv[T, 3*H*D], inv_freq[D], q_out[T,H,D], key_cache[S,H*D], val_cache[S,H*D], extra=[first_pos])``:
    ``rope_qkv_store_f16`` for the T tokens of a prompt, token t at position first_pos + t (a host integer, default 0)."""
    name = 'rope_qkv_store_rows_f16'

    def __call__(self, qkv, inv_freq, q_out, key_cache, val_cache, extra=None):
        T, heads, head_dim = q_out.shape
        if qkv.shape != (T, 3 * heads * head_dim) or key_cache.shape[-1] != heads * head_dim or val_cache.shape != key_cache.shape:
            raise ValueError(f'{self.name}: shapes do not fit together')
        for t in (qkv, inv_freq, q_out, key_cache, val_cache):
            if t.dtype != torch.float16:
                raise TypeError(f'{self.name}: tensors must be float16')
        first = int(extra[0]) if extra else 0
        _require_cuda(qkv, inv_freq, q_out, key_cache, val_cache)
        capi.check(capi.lib().art_rope_qkv_store_rows(c_void_p(qkv.data_ptr()), c_void_p(inv_freq.data_ptr()), c_void_p(q_out.data_ptr()),
                                                     c_void_p(key_cache.data_ptr()), c_void_p(val_cache.data_ptr()), T, heads, head_dim,
                                                     first, key_cache.numel() // (heads * head_dim), c_void_p(current_stream_handle())))
        return q_out


builtin('rope_qkv_store_rows_f16')(lambda: RopeQkvStoreRows())


class GreedyNext:
    """``greedy_next_f16(logits[V], prompt[L] or None, token[1], pos[1], embed[V, D], x[D])``: the bookkeeping
    between two decode steps in one launch - pos += 1; token = prompt[pos] while the prompt lasts, else
    argmax(logits); x = embed[token].  token, pos and prompt are int32 GPU tensors."""
    name = 'greedy_next_f16'

    def __call__(self, logits, prompt, token, pos, embed, x):
        vocab, dim = embed.shape
        if logits.numel() != vocab or x.numel() != dim or token.numel() != 1 or pos.numel() != 1:
            raise ValueError('greedy_next_f16: shapes do not fit together')
        if not (logits.dtype == embed.dtype == x.dtype == torch.float16):
            raise TypeError('greedy_next_f16: logits, embed and x must be float16')
        ints = [token, pos] + ([prompt] if prompt is not None and prompt.numel() else [])
        if any(t.dtype != torch.int32 for t in ints):
            raise TypeError('greedy_next_f16: token, pos and prompt must be int32')
        _require_cuda(logits, embed, x, *ints)
        has_prompt = len(ints) == 3
        capi.check(capi.lib().art_greedy_next(c_void_p(logits.data_ptr()), vocab, c_void_p(prompt.data_ptr() if has_prompt else 0),
                                             prompt.numel() if has_prompt else 0, c_void_p(token.data_ptr()), c_void_p(pos.data_ptr()),
                                             c_void_p(embed.data_ptr()), dim, c_void_p(x.data_ptr()), c_void_p(current_stream_handle())))
        return token


builtin('greedy_next_f16')(lambda: GreedyNext())
builtin('gemv_w4a16_fused')(lambda: GemvW4Fused())
builtin('attention_rope_f16')(lambda: AttentionRope())
builtin('attention_rope_split_f16')(lambda: AttentionRopeSplit())
builtin('gemv_w4a16_attn')(lambda: GemvW4Attn())
builtin('rope_qkv_store_f16')(lambda: RopeQkvStore('rope_qkv_store_f16'))
builtin('rope_qkv_store_f32')(lambda: RopeQkvStore('rope_qkv_store_f32'))
