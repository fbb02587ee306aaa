"""The int4 GEMV over repacked weights (`autort.ops.w4_prepack` + `autort.ops.gemv_w4p`, C ABI `art_w4_prepack` /
`art_gemv_w4p`) against the CPU oracle: every case starts from the benchmark-format tensors (uint8 [K/2, N], fp16
scales, 4-bit zero points), goes through the repacking on the device and is compared with `hot_ops.gemm_w4a16` on the
same inputs, rtol / atol 1e-2 (the tolerance of the fp16 operators)."""
import numpy as np
import pytest
import torch

from antares_amd import workloads

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures('oracle_built')]

FP16_TOL = dict(rtol=1e-2, atol=1e-2)


@pytest.fixture(scope='module')
def autort():
    import autort as a
    return a


def note(msg):
    print(f'[case] {msg}', flush=True)


def to_dev(p, dev):
    return {k: v.to(dev) for k, v in p.items()}


# ragged sizes: one quantisation group, K below / not a multiple of a wavefront's 1024 values, a single tile,
# the largest K; then the benchmark's four shapes and the two fused projections of the decode step
@pytest.mark.parametrize('K,N', [(128, 16), (256, 64), (384, 144), (1152, 1040), (2048, 16), (16384, 48),
                                 (4096, 4096), (4096, 11008), (11008, 4096), (4096, 32000), (4096, 12288), (4096, 22016),
                                 (2176, 16400), (3968, 16400)])      # an odd number of tiles (1025)
def test_packed_gemv_matches_oracle(autort, K, N):
    from oracle import hot_ops
    note(f'gemv_w4p K={K} N={N}')
    p = workloads.w4_problem(K + N, 1, K, N)
    dev = autort.device()
    d = to_dev(p, dev)
    packed = autort.ops.w4_prepack(d['qweight'], d['scales'], d['qzeros'])
    assert packed.w4_shape == (K, N)
    y = autort.ops.gemv_w4p(d['x'].view(-1), packed)
    torch.cuda.synchronize()
    want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy()).reshape(-1)
    assert np.allclose(y.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)
    # no state between launches: the same bits again, also into a buffer that held something else
    y2 = torch.full_like(y, 7.0)
    autort.ops.gemv_w4p(d['x'].view(-1), packed, y2, shape=(K, N))
    assert torch.equal(y, y2)
    # the split-K kernel over the benchmark layout computes the same sums in another order
    from antares_amd.autort import patterns
    f = autort.export(ir=patterns.W4A16_IR, inputs=patterns.W4A16_INPUTS, name='gemv_w4a16')
    y_split = f(d['x'], d['qweight'], d['scales'], d['qzeros']).view(-1)
    assert torch.allclose(y.float(), y_split.float(), rtol=4e-3, atol=4e-3)


def test_packed_layout_pins_nibble_group_and_column_order(autort):
    """One-hot weights: with scale 1 and zero point 0 everywhere, a single nibble set to 1 at (k, n) and x = 1..K gives
    y[n] = k + 1 and zero elsewhere - for k in every position of a packed word, every group of a record, records
    past the first, and n in every column of a tile."""
    dev = autort.device()
    K, N = 2176, 48           # three records, the last one with one group only
    x = (torch.arange(K, dtype=torch.float32) % 61 + 1).half()       # distinct enough, exact in fp16
    cases = [(k, n) for k in list(range(0, 20)) + [127, 128, 1023, 1024, 1031, 2047, 2048, 2175] for n in (0, 1, 7, 8, 15, 16, 47)]
    scales = torch.ones(K // 128, N, dtype=torch.float16)
    qzeros = torch.zeros(K // 128, N // 2, dtype=torch.uint8)
    for k, n in cases:
        qweight = torch.zeros(K // 2, N, dtype=torch.uint8)
        qweight[k // 2, n] = 1 << (4 * (k % 2))
        packed = autort.ops.w4_prepack(qweight.to(dev), scales.to(dev), qzeros.to(dev))
        y = autort.ops.gemv_w4p(x.to(dev), packed).float().cpu()
        want = torch.zeros(N)
        want[n] = float(x[k])
        assert torch.equal(y, want), (k, n, y.nonzero().tolist(), y[n].item())
    # the zero point of (group, column): q = 0 everywhere, z = 3 at one place, x = 1 -> y[n] = -3 * 128
    note('zero-point order')
    for g, n in [(0, 0), (0, 1), (1, 14), (16, 15), (16, 32)]:
        qz = torch.zeros(K // 128, N // 2, dtype=torch.uint8)
        qz[g, n // 2] = 3 << (4 * (n % 2))
        packed = autort.ops.w4_prepack(torch.zeros(K // 2, N, dtype=torch.uint8, device=dev), scales.to(dev), qz.to(dev))
        y = autort.ops.gemv_w4p(torch.ones(K, dtype=torch.float16, device=dev), packed).float().cpu()
        want = torch.zeros(N)
        want[n] = -384.0
        assert torch.equal(y, want), (g, n)


@pytest.mark.parametrize('K,N', [(512, 256), (1152, 48), (4096, 4096), (4096, 12288), (11008, 4096), (4096, 32000), (3968, 16400)])
def test_packed_gemv_with_rmsnorm_and_residual(autort, K, N):
    """norm_weight / residual folded in, against rmsnorm -> gemv -> add of the oracle, and in place on the residual."""
    from oracle import hot_ops
    note(f'gemv_w4p fused K={K} N={N}')
    dev = autort.device()
    p = workloads.w4_problem(K + N, 1, K, N)
    g = torch.Generator().manual_seed(K)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).half()
    res = torch.randn(N, generator=g).half()
    x = p['x'].view(-1)
    d = to_dev(p, dev)
    packed = autort.ops.w4_prepack(d['qweight'], d['scales'], d['qzeros'])
    got = autort.ops.gemv_w4p(x.to(dev), packed, norm_weight=nw.to(dev), residual=res.to(dev))
    xn = hot_ops.rmsnorm(x.numpy(), None, nw.numpy(), 1.0 / K, 1e-5, np.float16)
    y = hot_ops.gemm_w4a16(xn.reshape(1, K), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy()).reshape(-1)
    want = (y.astype(np.float32) + res.numpy().astype(np.float32)).astype(np.float16)
    assert np.allclose(got.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)
    # each option alone
    only_norm = autort.ops.gemv_w4p(x.to(dev), packed, norm_weight=nw.to(dev))
    assert np.allclose(only_norm.cpu().numpy().astype(np.float32), y.astype(np.float32), **FP16_TOL)
    y_plain = hot_ops.gemm_w4a16(x.numpy().reshape(1, K), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy()).reshape(-1)
    only_res = autort.ops.gemv_w4p(x.to(dev), packed, residual=res.to(dev))
    want_res = (y_plain.astype(np.float32) + res.numpy().astype(np.float32)).astype(np.float16)
    assert np.allclose(only_res.cpu().numpy().astype(np.float32), want_res.astype(np.float32), **FP16_TOL)
    # in place on the residual
    buf = res.to(dev).clone()
    autort.ops.gemv_w4p(x.to(dev), packed, buf, norm_weight=nw.to(dev), residual=buf)
    assert torch.equal(buf, got)
    # against the fused split-K operator over the benchmark layout
    other = autort.ops.gemv_w4a16_fused(x.to(dev), d['qweight'], d['scales'], d['qzeros'], norm_weight=nw.to(dev), residual=res.to(dev))
    assert torch.allclose(got.float(), other.float(), rtol=4e-3, atol=4e-3)


@pytest.mark.parametrize('K,F', [(512, 1024), (1152, 24), (4096, 11008), (2304, 8200)])
def test_packed_gate_up_with_swiglu_output(autort, K, F):
    """gate | up interleaved in blocks of 8 columns, RMSNorm in, SwiGLU out: against the oracle's two projections and
    silu(gate) * up as the decode step of the oracle computes it."""
    from antares_amd.autort.builtin_ops import interleave_gate_up
    from oracle import hot_ops
    note(f'gemv_w4p swiglu K={K} F={F}')
    dev = autort.device()
    gate, up = workloads.w4_problem(K + F, 1, K, F), workloads.w4_problem(K + F + 1, 1, K, F)
    x = gate['x'].view(-1)
    g = torch.Generator().manual_seed(F)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).half()
    mixed = interleave_gate_up({k: gate[k] for k in ('qweight', 'scales', 'qzeros')}, {k: up[k] for k in ('qweight', 'scales', 'qzeros')})
    m = to_dev(mixed, dev)
    packed = autort.ops.w4_prepack(m['qweight'], m['scales'], m['qzeros'])
    got = autort.ops.gemv_w4p(x.to(dev), packed, norm_weight=nw.to(dev), swiglu_out=True)
    assert got.shape == (F,)
    xn = hot_ops.rmsnorm(x.numpy(), None, nw.numpy(), 1.0 / K, 1e-5, np.float16).reshape(1, K)
    gv = hot_ops.gemm_w4a16(xn, gate['qweight'].numpy(), gate['scales'].numpy(), gate['qzeros'].numpy()).reshape(-1).astype(np.float32)
    uv = hot_ops.gemm_w4a16(xn, up['qweight'].numpy(), up['scales'].numpy(), up['qzeros'].numpy()).reshape(-1).astype(np.float32)
    want = (gv / (np.float32(1) + np.exp(-gv)) * uv).astype(np.float16)           # oracle/llama_ref.py, line :171 of the sample
    # the product of two rounded projections: each is within 1e-2 of the oracle's, so is silu(g) * u relative to |u| + |g|
    tol = 1e-2 * (1 + np.abs(gv) + np.abs(uv))
    assert (np.abs(got.cpu().numpy().astype(np.float32) - want.astype(np.float32)) <= tol + 1e-2 * np.abs(want.astype(np.float32))).all()
    # without the norm, and the un-fused form of the same: plain packed product of the interleaved matrix, then SwiGLU by hand
    plain = autort.ops.gemv_w4p(x.to(dev), packed, norm_weight=nw.to(dev)).float().view(F // 8, 2, 8)
    gd, ud = plain[:, 0].reshape(-1), plain[:, 1].reshape(-1)
    by_hand = (gd / (1 + torch.exp(-gd)) * ud).half()
    assert torch.allclose(got.float(), by_hand.float(), rtol=2e-3, atol=2e-3)


def test_packed_gemv_rejects_what_it_cannot_do(autort):
    from ctypes import c_void_p
    from antares_amd.runtime import capi
    dev = autort.device()
    capi.init(dev.index or 0)
    lib = capi.lib()
    assert lib.art_w4_prepack_bytes(4096, 11008) > 2048 * 11008
    assert lib.art_w4_prepack_bytes(4096, 11000) == 0 and lib.art_w4_prepack_bytes(100, 16) == 0 and lib.art_w4_prepack_bytes(16512, 16) == 0
    p = to_dev(workloads.w4_problem(1, 1, 256, 32), dev)
    packed = autort.ops.w4_prepack(p['qweight'], p['scales'], p['qzeros'])
    x, y = p['x'].view(-1), torch.empty(32, dtype=torch.float16, device=dev)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    null = c_void_p(0)
    # y overlapping x, SwiGLU output together with a residual, K beyond the kernel's 16 wavefronts, unaligned packed buffer
    assert lib.art_gemv_w4p(c_void_p(x.data_ptr()), c_void_p(packed.data_ptr()), c_void_p(x.data_ptr()), 256, 32, null, 0.0, null, 0, stream) != 0
    assert b'overlap' in lib.art_last_error()
    assert lib.art_gemv_w4p(c_void_p(x.data_ptr()), c_void_p(packed.data_ptr()), c_void_p(y.data_ptr()), 256, 32, null, 0.0,
                            c_void_p(y.data_ptr()), 1, stream) != 0
    assert lib.art_gemv_w4p(c_void_p(x.data_ptr()), c_void_p(packed.data_ptr()), c_void_p(y.data_ptr()), 16512, 32, null, 0.0, null, 0, stream) != 0
    assert lib.art_gemv_w4p(c_void_p(x.data_ptr()), c_void_p(packed.data_ptr() + 16), c_void_p(y.data_ptr()), 256, 32, null, 0.0, null, 0, stream) != 0
    with pytest.raises(ValueError):
        autort.ops.gemv_w4p(x, packed, shape=(256, 64))                 # packed size does not fit the shape
    with pytest.raises(TypeError):
        autort.ops.gemv_w4p(x.float(), packed)
    torch.cuda.synchronize()
