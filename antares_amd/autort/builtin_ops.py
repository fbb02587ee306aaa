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

    def __call__(self, x: torch.Tensor, out: torch.Tensor = None, extra=None):
        if x.dtype != torch.int32 or x.dim() != 1:
            raise TypeError('partition_even_first_i32 expects a 1-D int32 tensor')
        if out is None:
            out = torch.empty_like(x)
        if out.dtype != torch.int32 or out.numel() != x.numel():
            raise TypeError('partition_even_first_i32: out must be int32 with as many elements as the input')
        _require_cuda(x, out)
        capi.check(capi.lib().art_partition_even_first_i32(c_void_p(x.data_ptr()), c_void_p(out.data_ptr()),
                                                          x.numel(), c_void_p(current_stream_handle())))
        return out


@builtin('partition_even_first_i32')
def _partition():
    return PartitionEvenFirst()
