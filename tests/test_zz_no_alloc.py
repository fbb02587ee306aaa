"""art_gemv_w4a16_noalloc (split-K accumulators in an array that is part of the code object, no allocation on any
call) against art_gemv_w4a16 (accumulators in the library's allocated workspace), both through the C ABI."""
from ctypes import c_void_p

import numpy as np
import pytest
import torch

from antares_amd import workloads

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures('oracle_built')]


def _call(entry, p, y, M, K, N):
    from antares_amd.runtime import capi
    stream = torch.cuda.current_stream().cuda_stream
    capi.check(entry(c_void_p(p['x'].data_ptr()), c_void_p(p['qweight'].data_ptr()), c_void_p(p['scales'].data_ptr()),
                     c_void_p(p['qzeros'].data_ptr()), c_void_p(y.data_ptr()), M, K, N, c_void_p(stream)))


def test_noalloc_entry_point_matches_the_allocating_one():
    from antares_amd.runtime import capi
    from oracle import hot_ops
    capi.init(0)
    lib = capi.lib()
    dev = torch.device('cuda', 0)
    # two calls in a row, the second one smaller (it must find the accumulators the first one used at zero),
    # then a shape without K-split and one with four rows at the largest N the array takes
    for M, K, N in [(1, 11008, 4096), (1, 4096, 1040), (2, 4096, 11008), (1, 512, 256), (4, 1024, 32000), (3, 11008, 512)]:
        print(f'[case] no-alloc GEMV M={M} K={K} N={N}', flush=True)
        host = workloads.w4_problem(M + K + N, M, K, N)
        p = {k: host[k].to(dev) for k in ('x', 'qweight', 'scales', 'qzeros')}
        want = torch.full((M, N), float('nan'), dtype=torch.float16, device=dev)
        got = torch.full((M, N), float('nan'), dtype=torch.float16, device=dev)
        _call(lib.art_gemv_w4a16, p, want, M, K, N)
        _call(lib.art_gemv_w4a16_noalloc, p, got, M, K, N)
        torch.cuda.synchronize()
        assert torch.equal(got, want)                    # same kernel, same fixed-point meeting of the K-splits: same bits
        ref = hot_ops.gemm_w4a16(host['x'].numpy(), host['qweight'].numpy(), host['scales'].numpy(), host['qzeros'].numpy())
        assert np.allclose(got.float().cpu().numpy(), ref.astype(np.float32), rtol=1e-2, atol=1e-2)
        # again: the launch left its accumulators clean
        again = torch.empty_like(got)
        _call(lib.art_gemv_w4a16_noalloc, p, again, M, K, N)
        torch.cuda.synchronize()
        assert torch.equal(again, want)
    # a stream the library has never seen: the allocating entry point would set up a workspace for it, this one needs nothing
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        _call(lib.art_gemv_w4a16_noalloc, p, again, M, K, N)
    side.synchronize()
    assert torch.equal(again, want)


def test_noalloc_entry_point_refuses_what_does_not_fit():
    from antares_amd.runtime import capi
    capi.init(0)
    lib = capi.lib()
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device='cuda')
    a = c_void_p(buf.data_ptr())
    y = c_void_p(buf.data_ptr() + (1 << 19))
    assert lib.art_gemv_w4a16_noalloc(a, a, a, a, y, 1, 4096, 131072 + 16, None) != 0
    assert b'exceeds' in lib.art_last_error()
    assert lib.art_gemv_w4a16_noalloc(a, a, a, a, y, 4, 4096, 32784, None) != 0
    assert b'exceeds' in lib.art_last_error()
    assert lib.art_gemv_w4a16_noalloc(a, a, a, a, y, 5, 4096, 4096, None) != 0
    assert b'1..4' in lib.art_last_error()
