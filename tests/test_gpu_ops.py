"""GPU parity tests: every operator is called through the autort surface (which
goes through the C-ABI library) and compared with the CPU oracle on the same
seeded inputs.  Integer results must be bit-exact; fp32 within 1e-5, fp16
within rtol 1e-2 / atol 1e-2."""
import sys

import numpy as np
import pytest
import torch

from antares_amd import workloads

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures('oracle_built')]

FP32_TOL = dict(rtol=1e-5, atol=1e-5)
FP16_TOL = dict(rtol=1e-2, atol=1e-2)


@pytest.fixture(scope='module')
def autort():
    import autort as mod
    assert torch.cuda.is_available(), 'these tests need the GPU'
    return mod


def note(msg):
    print(f'[case] {msg}', flush=True)
    sys.stdout.flush()


SIGMOID_IR = 'sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))'


def test_sigmoid_readme_example(autort):
    note('sigmoid N=10')
    f = autort.export(ir=SIGMOID_IR, inputs=['data=float32[N:4096000]'], config='tune:5')
    data = torch.arange(0, 10, dtype=torch.float32, device=autort.device())
    want = [0.5000, 0.7311, 0.8808, 0.9526, 0.9820, 0.9933, 0.9975, 0.9991, 0.9997, 0.9999]
    assert np.allclose(f(data).cpu().numpy(), want, atol=5e-5)
    assert np.allclose(autort.ops.sigmoid_f32(data).cpu().numpy(), want, atol=5e-5)


@pytest.mark.parametrize('n', [0, 1, 3, 4, 5, 1023, 4_096_000, 4_096_003])
def test_sigmoid_matches_oracle(autort, n):
    from oracle import hot_ops
    note(f'sigmoid N={n}')
    f = autort.export(ir=SIGMOID_IR, inputs=['data=float32[N:4096000]'])
    x = workloads.sigmoid_input(7, n)
    got = f(x.to(autort.device())).cpu().numpy()
    assert got.shape == (n,)
    assert np.allclose(got, hot_ops.sigmoid_f32(x.numpy()), **FP32_TOL)


def test_sigmoid_unaligned_view(autort):
    from oracle import hot_ops
    note('sigmoid on a view that is not 16-byte aligned')
    f = autort.export(ir=SIGMOID_IR, inputs=['data=float32[N:4096000]'])
    x = workloads.sigmoid_input(8, 10_001)
    xd = x.to(autort.device())
    out = torch.zeros(10_001, dtype=torch.float32, device=autort.device())
    f(xd[1:], out=out[1:])
    assert np.allclose(out[1:].cpu().numpy(), hot_ops.sigmoid_f32(x.numpy()[1:]), **FP32_TOL)
    assert float(out[0]) == 0.0


def run_sort_sample(autort, x: torch.Tensor) -> torch.Tensor:
    """samples/01_sort_even_first.py:16-27 verbatim in structure."""
    autort.export(ir='space[data[N] % 2, N] = 1', inputs=['data=int32[N]', 'space=int32[2, N]'],
                  config='~N~:[1,256,1]', name='my_classify_i32')
    autort.export(ir='output[ids[N] - 1] = (val[N % val.size(0)]).when(ids[N] > 0)',
                  inputs=['ids=int32[N]', 'val=int32[M]', 'output=int32[M]'], config='~N~:[1,256,1]', name='my_bucket_i32')
    y = torch.zeros([2, x.size(0)], dtype=torch.int32, device=x.device)
    autort.ops.my_classify_i32(x, y)
    ids = torch.cumsum(y.view(-1), 0, dtype=y.dtype) * y.view(-1)
    output = torch.zeros_like(x)
    autort.ops.my_bucket_i32(ids, x, output)
    return output


def test_sort_sample_known_answer(autort):
    note('sort sample, README input')
    x = torch.tensor([101, 102, 208, 99, 1, 127, 62, 8, 336, 336], dtype=torch.int32, device=autort.device())
    assert run_sort_sample(autort, x).cpu().tolist() == [102, 208, 62, 8, 336, 336, 101, 99, 1, 127]
    assert autort.ops.partition_even_first_i32(x).cpu().tolist() == [102, 208, 62, 8, 336, 336, 101, 99, 1, 127]


@pytest.mark.parametrize('n', [1, 2, 63, 64, 65, 4095, 4096, 4097, 8191, 8192, 100_003, 1_048_576])
def test_partition_bit_exact(autort, n):
    from oracle import hot_ops
    note(f'partition N={n}')
    x = workloads.partition_input(100 + n, n)
    want = hot_ops.sort_even_first_i32(x.numpy())
    xd = x.to(autort.device())
    assert np.array_equal(autort.ops.partition_even_first_i32(xd).cpu().numpy(), want)
    assert np.array_equal(run_sort_sample(autort, xd).cpu().numpy(), want)


def test_partition_empty_and_degenerate(autort):
    note('partition edge cases')
    dev = autort.device()
    assert autort.ops.partition_even_first_i32(torch.empty(0, dtype=torch.int32, device=dev)).numel() == 0
    ev = torch.arange(0, 20000, 2, dtype=torch.int32, device=dev)
    assert torch.equal(autort.ops.partition_even_first_i32(ev), ev)
    assert torch.equal(autort.ops.partition_even_first_i32(ev + 1), ev + 1)
    # the output may start anywhere on a 4-byte boundary (its 16-byte stores find their own alignment) and nothing
    # outside it is written
    for shift in (1, 2, 3):
        x = workloads.partition_input(shift, 10_007).to(dev)
        backing = torch.full((10_007 + 8,), -7, dtype=torch.int32, device=dev)
        out = backing[shift:shift + 10_007]
        autort.ops.partition_even_first_i32(x, out)
        xc = x.cpu()
        assert torch.equal(out.cpu(), torch.cat([xc[xc % 2 == 0], xc[xc % 2 == 1]]))
        assert (backing[:shift] == -7).all() and (backing[shift + 10_007:] == -7).all()


def test_partition_full_size_properties(autort):
    note('partition N=16777216 (size-independent properties)')
    x = workloads.partition_input(2, 16_777_216).to(autort.device())
    out = autort.ops.partition_even_first_i32(x)
    want = torch.cat([x[x % 2 == 0], x[x % 2 == 1]])
    assert torch.equal(out, want)
    # idempotent
    assert torch.equal(autort.ops.partition_even_first_i32(out), out)
    # two calls in a row give the same bits (ticket words are restored)
    assert torch.equal(autort.ops.partition_even_first_i32(x), out)


# ------------------------------------------------------------------ int4 GEMV
def w4_op(autort):
    from antares_amd.autort import patterns
    return autort.export(ir=patterns.W4A16_IR, inputs=patterns.W4A16_INPUTS, name='gemv_w4a16')


@pytest.mark.parametrize('M,K,N', [(1, 128, 16), (1, 256, 64), (2, 384, 144), (3, 1024, 1040), (4, 4096, 512), (8, 512, 256),
                                   (1, 4096, 4096), (1, 4096, 11008), (1, 11008, 4096), (1, 4096, 32000)])
def test_w4a16_gemv_matches_oracle(autort, M, K, N):
    from oracle import hot_ops
    note(f'w4a16 M={M} K={K} N={N}')
    p = workloads.w4_problem(K + N + M, M, K, N)
    f = w4_op(autort)
    assert f.fast_path is not None
    dev = autort.device()
    y = f(p['x'].to(dev), p['qweight'].to(dev), p['scales'].to(dev), p['qzeros'].to(dev))
    torch.cuda.synchronize()
    want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    assert np.allclose(y.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)
    # second call must see clean ticket words
    y2 = f(p['x'].to(dev), p['qweight'].to(dev), p['scales'].to(dev), p['qzeros'].to(dev))
    assert torch.equal(y, y2)


@pytest.mark.parametrize('M,K,N', [(9, 128, 16), (17, 256, 144), (32, 384, 1040), (33, 1024, 512), (64, 2048, 272),
                                   (100, 512, 4096), (200, 4096, 512),
                                   (64, 4096, 4096), (64, 4096, 11008), (64, 11008, 4096), (64, 4096, 32000)])
def test_w4a16_gemm_matches_oracle(autort, M, K, N):
    """Batches of four rows and more run on the matrix cores (one pass over the weights per 64 rows)."""
    from oracle import hot_ops
    note(f'w4a16 gemm M={M} K={K} N={N}')
    p = workloads.w4_problem(K + N + M, M, K, N)
    f = w4_op(autort)
    assert f.fast_path is not None
    dev = autort.device()
    args = [p[k].to(dev) for k in ('x', 'qweight', 'scales', 'qzeros')]
    y = f(*args)
    torch.cuda.synchronize()
    want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    assert np.allclose(y.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)
    # K-splits are combined in a fixed order: a second call gives the same bits
    assert torch.equal(y, f(*args))
    # row m of the batch agrees with the same row sent alone through the GEMV kernel
    m = M - 1
    y1 = f(args[0][m:m + 1].contiguous(), *args[1:])
    assert np.allclose(y1.cpu().numpy().astype(np.float32), want[m:m + 1].astype(np.float32), **FP16_TOL)
    # (the GEMM rounds s * (q - z) to fp16 as the oracle does, the GEMV applies s in fp32: both are inside the oracle
    # tolerance, and within half of it of each other)
    assert np.allclose(y1.float().cpu().numpy(), y[m:m + 1].float().cpu().numpy(), rtol=5e-3, atol=5e-3)


@pytest.mark.parametrize('M,K,N', [(4, 512, 256), (5, 1024, 144), (6, 4096, 512), (7, 384, 1040), (8, 4096, 4096)])
def test_w4a16_gemv_entry_point_up_to_eight_rows(autort, M, K, N):
    """`art_gemv_w4a16` takes up to 8 rows (the weights are streamed once per pair of rows); autort.export sends
    4 rows and more to the matrix-core kernel, so the entry point is called directly here."""
    from ctypes import c_void_p
    from antares_amd.runtime import capi
    from oracle import hot_ops
    note(f'art_gemv_w4a16 direct M={M} K={K} N={N}')
    p = workloads.w4_problem(K + N + M, M, K, N)
    dev = autort.device()
    capi.init(dev.index or 0)
    x, q, s_, z = (p[k].to(dev) for k in ('x', 'qweight', 'scales', 'qzeros'))
    y = torch.empty(M, N, dtype=torch.float16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    capi.check(capi.lib().art_gemv_w4a16(c_void_p(x.data_ptr()), c_void_p(q.data_ptr()), c_void_p(s_.data_ptr()),
                                         c_void_p(z.data_ptr()), c_void_p(y.data_ptr()), M, K, N, c_void_p(stream)))
    torch.cuda.synchronize()
    want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    assert np.allclose(y.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)


@pytest.mark.parametrize('poison', [float('nan'), float('inf'), 60000.0])
def test_gemv_with_non_finite_rows_stays_clean(autort, poison):
    """A NaN, an infinity or values that overflow the sum in x must come out as non-finite results (the reference's
    float sums propagate them) and must not leave anything behind in the split-K slots: the same operator called
    on ordinary data right afterwards gives the ordinary answer."""
    from antares_amd.autort import patterns
    from oracle import hot_ops
    note(f'w4a16 / gptq gemv with x poisoned by {poison}')
    dev = autort.device()
    K, N = 4096, 1024
    p = workloads.w4_problem(77, 1, K, N)
    f = w4_op(autort)
    args = [p[k].to(dev) for k in ('x', 'qweight', 'scales', 'qzeros')]
    good = f(*args)
    bad_x = args[0].clone()
    if poison == 60000.0:
        bad_x[:] = poison                        # finite, but every partial sum is far outside fp16
    else:
        bad_x[0, 1000] = poison
    bad = f(bad_x, *args[1:])
    if poison != 60000.0:
        assert not torch.isfinite(bad).any()
    again = f(*args)
    assert torch.equal(again, good)
    want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    assert np.allclose(again.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)
    # the sample's own program (fp32, GPTQ words)
    g = torch.Generator().manual_seed(5)
    q = torch.randint(0, 16, (K, N), generator=g)
    s = torch.rand(K // 128, N, generator=g) * 0.019 + 0.001
    x = torch.randn(K, generator=g)
    h = autort.export(ir=patterns.GPTQ_GEMV_IR, inputs=patterns._gptq_inputs('float32', 'float32'))
    qw = workloads.pack_gptq(q).to(dev)
    good = h(x.to(dev), qw, s.to(dev)).clone()
    bad_x = x.clone()
    if poison == 60000.0:
        bad_x[:] = 1e30                          # the sums are beyond what a split-K slot carries: reported as NaN
    else:
        bad_x[17] = poison
    bad = h(bad_x.to(dev), qw, s.to(dev))
    assert not torch.isfinite(bad).any()
    assert torch.equal(h(x.to(dev), qw, s.to(dev)), good)


def test_w4a16_generic_lowering_agrees(autort):
    """The same program through the generic reduce lowering (no hand kernel)."""
    from oracle import hot_ops
    note('w4a16 through the generic lowering')
    p = workloads.w4_problem(9, 2, 256, 64)
    f = w4_op(autort)
    dev = autort.device()
    bound = {'x': p['x'].to(dev), 'qweight': p['qweight'].to(dev), 'scales': p['scales'].to(dev), 'qzeros': p['qzeros'].to(dev)}
    saved, f.fast_path = f.fast_path, None
    try:
        y = f(bound['x'], bound['qweight'], bound['scales'], bound['qzeros'])
    finally:
        f.fast_path = saved
    want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    assert np.allclose(y.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)


@pytest.mark.parametrize('K,N,sdt', [(4096, 12288, 'float32'), (4096, 4096, 'float16'), (11008, 4096, 'float32'), (256, 36, 'float32')])
def test_gptq_gemv_sample_program(autort, K, N, sdt):
    from antares_amd.autort import patterns
    from oracle import hot_ops
    note(f'gptq gemv K={K} N={N} scales={sdt}')
    g = torch.Generator().manual_seed(K + N)
    q = torch.randint(0, 16, (K, N), generator=g)
    s = (torch.rand(K // 128, N, generator=g) * 0.019 + 0.001).to(torch.float32 if sdt == 'float32' else torch.float16)
    x = torch.randn(K, generator=g)
    qw = workloads.pack_gptq(q)
    f = autort.export(ir=patterns.GPTQ_GEMV_IR, inputs=patterns._gptq_inputs('float32', sdt), config='~N~:[256,8,32],~S~:[64,8]')
    dev = autort.device()
    out = torch.empty(N, dtype=torch.float32, device=dev)
    y = f(x.to(dev), qw.to(dev), s.to(dev), out=out)
    assert y.data_ptr() == out.data_ptr()
    want = hot_ops.gemv_gptq_f32(x.numpy(), qw.numpy(), s.numpy())
    exact = x.numpy().astype(np.float64) @ ((q.numpy().astype(np.float64) - 8) * np.repeat(s.numpy().astype(np.float64), 128, axis=0))
    got = y.cpu().numpy()
    # fp32 sums of K terms: the oracle's own distance from the exact value sets the scale of the tolerance
    tol = max(1e-5, 4 * float(np.abs(want - exact).max()))
    assert np.abs(got - exact).max() <= tol, (np.abs(got - exact).max(), tol)
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------ generic lowering
def test_generic_reduce_variants(autort):
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note('generic reduce: softmax program')
    ir = ('temp0[N] >=! input0[N, C]; temp1[N] +=! (input0[N, C] - temp0[N]).call(`exp`); '
          'output0[N, C] = (input0[N, C] - temp0[N]).call(`exp`) / temp1[N]')
    dev = autort.device()
    for shape in [(32, 1024), (3, 5000), (300, 7)]:
        inp = {'input0': {'dtype': 'float32', 'shape': list(shape)}}
        x = torch.randn(*shape, generator=torch.Generator().manual_seed(1))
        f = autort.export(ir=ir, inputs=['input0=float32[%d, %d]' % shape])
        got = f(x.to(dev)).cpu().numpy()
        want = CpuModule(parse_program(ir, inp))(input0=x.numpy())['output0']
        assert np.allclose(got, want, **FP32_TOL)


def test_generic_matmul_and_scatter(autort):
    note('generic matmul + scatter-add')
    dev = autort.device()
    g = torch.Generator().manual_seed(3)
    a, b = torch.randn(70, 50, generator=g), torch.randn(50, 33, generator=g)
    f = autort.export(ir='output0[N, M] +=! input0[N, K] * input1[K, M]', inputs=['input0=float32[N:70, K:50]', 'input1=float32[K:50, M:33]'])
    assert np.allclose(f(a.to(dev), b.to(dev)).cpu().numpy(), (a.double() @ b.double()).numpy(), rtol=1e-4, atol=1e-4)
    idx = torch.randint(0, 16, (1000,), generator=g, dtype=torch.int64).to(torch.int32)
    upd = torch.randint(0, 100, (1000,), generator=g, dtype=torch.int64).to(torch.int32)
    hist = torch.zeros(16, dtype=torch.int32, device=dev)
    h = autort.export(ir='hist[idx[B]] +=. upd[B]', inputs=['hist=int32[H]', 'idx=int32[B]', 'upd=int32[B]'], name='scatter_add_i32')
    h(hist, idx.to(dev), upd.to(dev))
    want = torch.zeros(16, dtype=torch.int64).index_add_(0, idx.long(), upd.long())
    assert hist.cpu().long().tolist() == want.tolist()


def test_code_object_file_loads_and_runs(autort, tmp_path):
    """art_module_load_file: a code object written to disk (what `hipcc --genco` leaves) is loaded and launched."""
    import ctypes
    from antares_amd.runtime import capi
    note('art_module_load_file')
    capi.init(0)
    image = capi.compile_hip('extern "C" __global__ void twice(float* a, int n) { int i = blockIdx.x * 64 + threadIdx.x; if (i < n) a[i] *= 2.f; }')
    path = tmp_path / 'twice.hsaco'
    path.write_bytes(image)
    h, f = ctypes.c_void_p(), ctypes.c_void_p()
    capi.check(capi.lib().art_module_load_file(str(path).encode(), ctypes.byref(h)))
    capi.check(capi.lib().art_get_function(h, b'twice', ctypes.byref(f)))
    a = torch.arange(100, dtype=torch.float32, device=autort.device())
    capi.launch(f, (2, 1, 1), (64, 1, 1), torch.cuda.current_stream().cuda_stream, [a.data_ptr(), 100])
    torch.cuda.synchronize()
    assert torch.equal(a.cpu(), torch.arange(100, dtype=torch.float32) * 2)


@pytest.mark.parametrize('ir,inputs,shapes', [
    ('output0[] +=! input0[N]', ['input0=float32[N:1048576]'], [(1048576,), (1000003,), (262144,)]),
    ('output0[C] +=! input0[N, C]', ['input0=float32[N:2048, C:512]'], [(2048, 512), (4096, 96)]),
    ('output0[N] >=! input0[N, C]', ['input0=float32[N:8, C:65536]'], [(8, 65536), (3, 40000)]),
    ('output0[N] <=! input0[N, C]', ['input0=float32[8, 32768]'], [(8, 32768)]),
    ('output0[N, M] +=! input0[N, K] * input1[K, M]', ['input0=float32[N:4, K:8192]', 'input1=float32[K:8192, M:16]'], [(4, 8192, 16)]),
    ('output0[] +=! input0[N]', ['input0=int32[N:2097152]'], [(2097152,)]),
])
def test_wide_reductions_are_sliced_and_still_right(autort, ir, inputs, shapes):
    """Reductions with too few outputs to fill the chip run as two statements (slices, then the slices); programs with
    named dimensions get kernels per set of values, and sizes that do not divide fall back to the one-statement form."""
    note(f'wide reduction {ir}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='wide_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    g = torch.Generator().manual_seed(11)
    for shape in shapes:
        if 'input1' in ir:
            n, k, m = shape
            a, b = torch.randn(n, k, generator=g), torch.randn(k, m, generator=g)
            got = op(a.to(dev), b.to(dev)).cpu()
            assert torch.allclose(got, (a.double() @ b.double()).float(), rtol=1e-4, atol=1e-3)
            continue
        if 'int32' in inputs[0]:
            x = torch.randint(-1000, 1000, shape, generator=g, dtype=torch.int32)
            assert int(op(x.to(dev)).cpu()) == int(x.sum())
            continue
        x = torch.randn(shape, generator=g)
        got = op(x.to(dev)).cpu()
        if '>=!' in ir:
            assert torch.equal(got, x.max(dim=1).values)
        elif '<=!' in ir:
            assert torch.equal(got, x.min(dim=1).values)
        elif ir.startswith('output0[C]'):
            assert torch.allclose(got, x.double().sum(0).float(), rtol=1e-4, atol=1e-3)
        else:
            assert abs(float(got) - float(x.double().sum())) < 0.05


@pytest.mark.parametrize('ir,spec,shape,perm', [
    ('output0[C, N] = input0[N, C]', 'input0=float32[N:1000, C:777]', (1000, 777), (1, 0)),
    ('output0[N, H, W, C] = input0[N, C, H, W]', 'input0=float16[N:3, C:70, H:5, W:129]', (3, 70, 5, 129), (0, 2, 3, 1)),
    ('output0[B, C, N] = input0[N, B, C] * 2', 'input0=float32[N:65, B:2, C:64]', (65, 2, 64), (1, 2, 0)),
    ('output0[C, N] = input0[N, C]', 'input0=int32[N:16, C:4096]', (16, 4096), (1, 0)),
])
def test_permutation_copies_go_through_lds_tiles(autort, ir, spec, shape, perm):
    """A copy whose store walks memory along another axis than its load is lowered to 64 x 64 tiles through LDS."""
    note(f'tiled permutation {ir} {shape}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=[spec], name='perm_' + str(abs(hash((ir, spec))) % 10 ** 8))
    assert 'tile' in op.plans[0].variants
    g = torch.Generator().manual_seed(4)
    if 'int32' in spec:
        x = torch.randint(-10 ** 6, 10 ** 6, shape, generator=g, dtype=torch.int32)
    else:
        x = torch.randn(shape, generator=g).to(torch.float16 if 'float16' in spec else torch.float32)
    want = x.permute(*perm).contiguous()
    if '* 2' in ir:
        want = want * 2
    assert torch.equal(op(x.to(dev)).cpu(), want)


@pytest.mark.parametrize('ir,spec,shape,perm', [
    ('output0[C, N] = input0[N, C]', 'input0=float32[N:1024, C:448]', (1024, 448), (1, 0)),
    ('output0[N, H, W, C] = input0[N, C, H, W]', 'input0=float16[N:2, C:128, H:3, W:64]', (2, 128, 3, 64), (0, 2, 3, 1)),
    ('output0[B, C, N] = input0[N, B, C] * 2', 'input0=float32[N:192, B:3, C:64]', (192, 3, 64), (1, 2, 0)),
    ('output0[C, N] = input0[N, C].cast(`float32`)', 'input0=int32[N:64, C:4096]', (64, 4096), (1, 0)),
])
def test_permutation_copies_of_whole_tiles_move_16_byte_vectors(autort, ir, spec, shape, perm):
    """With whole 64 x 64 tiles and aligned tensors the transposing variant reads and writes 16-byte vectors; a view
    that is not 16-byte aligned takes the scalar tiles, with the same result."""
    note(f'vector-tiled permutation {ir} {shape}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=[spec], name='permv_' + str(abs(hash((ir, spec))) % 10 ** 8))
    plan = op.plans[0]
    assert 'tilevec' in plan.variants
    g = torch.Generator().manual_seed(5)
    if 'int32' in spec:
        x = torch.randint(-10 ** 6, 10 ** 6, shape, generator=g, dtype=torch.int32)
    else:
        x = torch.randn(shape, generator=g).to(torch.float16 if 'float16' in spec else torch.float32)
    want = x.permute(*perm).contiguous()
    if '* 2' in ir:
        want = want * 2
    if 'cast' in ir:
        want = want.float()
    xd = x.to(dev)
    env = {k: v for k, v in zip([d.split(':')[0] for d in spec[spec.index('[') + 1:-1].split(', ')], shape)}
    out = torch.empty(want.shape, dtype=want.dtype, device=dev)
    assert plan.choose(env, {'input0': xd.data_ptr(), 'output0': out.data_ptr()})[0] == plan.variants['tilevec']
    assert torch.equal(op(xd).cpu(), want)
    # the same values 4 bytes further on: not aligned for vectors
    flat = torch.empty(x.numel() + 4, dtype=x.dtype, device=dev)
    skip = 4 // x.element_size()
    shifted = flat[skip:skip + x.numel()].view(shape)
    shifted.copy_(xd)
    assert plan.choose(env, {'input0': shifted.data_ptr(), 'output0': out.data_ptr()})[0] == plan.variants['tile']
    assert torch.equal(op(shifted).cpu(), want)


def test_split_k_launches_on_two_streams_do_not_disturb_each_other(autort):
    """Every stream has a workspace of its own: GEMVs with K-splits enqueued on two streams at the same time give
    the bits they give alone, and an aliasing y is refused."""
    from ctypes import c_void_p
    from antares_amd.runtime import capi
    note('split-K GEMVs on two streams')
    dev = autort.device()
    f = w4_op(autort)
    pa, pb = workloads.w4_problem(31, 1, 11008, 4096), workloads.w4_problem(32, 1, 11008, 4096)
    a = [pa[k].to(dev) for k in ('x', 'qweight', 'scales', 'qzeros')]
    b = [pb[k].to(dev) for k in ('x', 'qweight', 'scales', 'qzeros')]
    alone_a, alone_b = f(*a).clone(), f(*b).clone()
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a = [torch.empty_like(alone_a) for _ in range(20)]
    outs_b = [torch.empty_like(alone_b) for _ in range(20)]
    for i in range(20):
        with torch.cuda.stream(s1):
            f(*a, out=outs_a[i])
        with torch.cuda.stream(s2):
            f(*b, out=outs_b[i])
    torch.cuda.synchronize()
    for i in range(20):
        assert torch.equal(outs_a[i], alone_a) and torch.equal(outs_b[i], alone_b), i
    # y overlapping x is refused by the entry points (only the residual may alias y)
    x = a[0]
    rc = capi.lib().art_gemv_w4a16(c_void_p(x.data_ptr()), c_void_p(a[1].data_ptr()), c_void_p(a[2].data_ptr()),
                                   c_void_p(a[3].data_ptr()), c_void_p(x.data_ptr() + 64), 1, 11008, 4096, None)
    assert rc != 0 and b'overlap' in capi.lib().art_last_error()
    rc = capi.lib().art_gemv_w4a16_fused(c_void_p(x.data_ptr()), c_void_p(a[1].data_ptr()), c_void_p(a[2].data_ptr()),
                                         c_void_p(a[3].data_ptr()), c_void_p(x.data_ptr()), 11008, 4096, None, 1e-5, None, 0, None)
    assert rc != 0 and b'overlap' in capi.lib().art_last_error()


def test_fp16_reductions_where_tree_order_leaves_the_sequential_oracle(autort):
    """A reduction written in fp16 accumulates in fp16 on both sides (the reference's rule), but the GPU adds in tree
    order and the oracle in index order.  For 64 to 1024 terms of N(0,1) data the GPU stays within the fp16 tolerance
    of the float64 sum; the sequential oracle itself drifts from it (0.03 at 64 terms, 0.4 at 1024, where 1e-2 of the
    result's size is 0.3), so the two are compared with the oracle's own drift added to the tolerance.  Far beyond
    that they part for good: 16384 positive terms stall a sequential fp16 sum (at 2048 an addend below 1 is rounded
    away), while the tree keeps adding numbers of similar size - there the GPU result must be the one closer to the
    float64 sum, and within the fp16 tolerance of it."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    dev = autort.device()
    ir = 'output0[N] +=! input0[N, C]'
    for C in (64, 256, 1024):
        note(f'fp16 row sums, C={C}')
        x = torch.randn(48, C, generator=torch.Generator().manual_seed(C)).half()
        f = autort.export(ir=ir, inputs=[f'input0=float16[48, {C}]'], name=f'rowsum_f16_{C}')
        got = f(x.to(dev)).float().cpu().numpy()
        want = CpuModule(parse_program(ir, {'input0': {'dtype': 'float16', 'shape': [48, C]}}), fast_math=False)(input0=x.numpy())['output0']
        exact = x.double().sum(1).numpy()
        # sums of C terms of unit variance: sqrt(C) in size; fp16 keeps 2^-11 of that per addition
        tol = 1e-2 * max(1.0, C ** 0.5)
        assert np.abs(got - exact).max() <= tol, (C, np.abs(got - exact).max())
        drift = np.abs(want.astype(np.float64) - exact).max()
        assert np.abs(got - want.astype(np.float32)).max() <= tol + drift, (C, np.abs(got - want.astype(np.float32)).max(), drift)
    C = 16384
    note(f'fp16 row sums of positive data, C={C}')
    x = torch.rand(8, C, generator=torch.Generator().manual_seed(7)).half()
    f = autort.export(ir=ir, inputs=[f'input0=float16[8, {C}]'], name=f'rowsum_f16_{C}')
    got = f(x.to(dev)).float().cpu().numpy()
    want = CpuModule(parse_program(ir, {'input0': {'dtype': 'float16', 'shape': [8, C]}}), fast_math=False)(input0=x.numpy())['output0'].astype(np.float32)
    exact = x.double().sum(1).numpy()                      # about 8192
    assert np.all(want < 0.5 * exact)                      # the sequential fp16 sum has stalled (near 2048)
    assert np.allclose(got, exact, rtol=1e-2)              # the tree-ordered one has not
    assert np.all(np.abs(got - exact) < np.abs(want - exact))


@pytest.mark.parametrize('M,K,N', [(5, 512, 272), (64, 4096, 4096), (128, 1024, 1040), (200, 4096, 512)])
def test_w4a16_gemm_with_the_residual_folded_in(autort, M, K, N):
    """gemm_w4a16_residual: y = fp16(fp16(x @ W) + residual), in place on the residual, with and without K-splits."""
    from oracle import hot_ops
    note(f'w4a16 gemm + residual M={M} K={K} N={N}')
    dev = autort.device()
    p = workloads.w4_problem(K + N + M, M, K, N)
    res = torch.randn(M, N, generator=torch.Generator().manual_seed(M)).half()
    prod = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    want = (prod.astype(np.float32) + res.numpy().astype(np.float32)).astype(np.float16).astype(np.float32)
    d = [p[k].to(dev) for k in ('x', 'qweight', 'scales', 'qzeros')]
    acc = res.to(dev).clone()
    autort.ops.gemm_w4a16_residual(*d, acc, residual=acc)
    assert np.allclose(acc.float().cpu().numpy(), want, **FP16_TOL)
    out = torch.empty_like(acc)
    autort.ops.gemm_w4a16_residual(*d, out, residual=res.to(dev))
    assert torch.equal(out, acc)
    plain = torch.empty_like(acc)
    autort.ops.gemm_w4a16_residual(*d, plain)
    assert np.allclose(plain.float().cpu().numpy(), prod.astype(np.float32), **FP16_TOL)


ROW_VECTOR_CASES = [
    # program, inputs, shapes of the inputs, does the row-vector variant apply to these extents
    ('output0[N, C] = input0[N, C] + input1[C]', ['input0=float32[N:300, C:1024]', 'input1=float32[C:1024]'], [(300, 1024), (1024,)], True),
    ('output0[N, C] = input0[input1[N], C]', ['input0=float32[V:500, C:256]', 'input1=int32[N:1000]'], [(500, 256), (1000,)], True),
    ('emb[T, D] = table[tok[T], D]', ['table=float16[V:320, D:4096]', 'tok=int32[T:37]'], [(320, 4096), (37,)], True),
    ('output0[B, N, C] = (input0[B, N, C].to(`float32`) * input1[B, C] + input2[N]).to(`float16`)',
     ['input0=float16[B:3, N:50, C:72]', 'input1=float32[B:3, C:72]', 'input2=float32[N:50]'], [(3, 50, 72), (3, 72), (50,)], True),
    ('output0[N, C] = input0[N, C] * C + input1[N]', ['input0=int32[N:33, C:64]', 'input1=int32[N:33]'], [(33, 64), (33,)], True),
    # a last extent that is no multiple of the vector: the scalar kernel runs
    ('output0[N, C] = input0[N, C] + input1[C]', ['input0=float32[N:30, C:1023]', 'input1=float32[C:1023]'], [(30, 1023), (1023,)], False),
]


@pytest.mark.parametrize('ir,inputs,shapes,applies', ROW_VECTOR_CASES)
def test_row_vector_maps_match_the_oracle(autort, ir, inputs, shapes, applies):
    """Maps whose loads are runs along the last axis or constant along it (bias rows, gathered rows) move 16-byte
    vectors per lane; results are the oracle's, and the scalar kernel takes over where the extents do not fit."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'row-vector map {ir} {shapes}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='rowvec_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    plan = op.plans[0]
    assert 'rowvec' in plan.variants and 'vec' not in plan.variants
    g = torch.Generator().manual_seed(len(ir))
    tensors, names = [], []
    for spec, shape in zip(inputs, shapes):
        name, rest = spec.split('=')
        names.append(name)
        if rest.startswith('int32'):
            hi = 320 if 'tok' in name else (500 if name == 'input1' and 'input0[input1' in ir else 1000)
            tensors.append(torch.randint(0, hi, shape, generator=g, dtype=torch.int32))
        else:
            tensors.append(torch.randn(shape, generator=g).to(torch.float16 if rest.startswith('float16') else torch.float32))
    env = {}
    for spec, shape in zip(inputs, shapes):
        dims = spec.split('[', 1)[1].rstrip(']').split(',')
        for d, v in zip(dims, shape):
            env[d.split(':')[0].strip()] = v
    ptrs = {n: 0 for n in plan.args}
    assert (plan.choose(env, ptrs)[0] == plan.variants['rowvec']) == applies
    got = op(*[t.to(dev) for t in tensors]).cpu().numpy()
    out_name = ir.split('[', 1)[0].strip()
    want = CpuModule(parse_program(ir, inputs), fast_math=False)(**{n: t.numpy() for n, t in zip(names, tensors)})[out_name]
    if got.dtype.kind == 'i':
        assert np.array_equal(got, want)
    else:
        assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=1e-2 if got.dtype == np.float16 else 1e-5,
                           atol=1e-2 if got.dtype == np.float16 else 1e-5)
    # an operand that is not 16-byte aligned falls back to the scalar kernel, same result
    if applies and tensors[0].dtype != torch.int32:
        base = torch.empty(tensors[0].numel() + 1, dtype=tensors[0].dtype, device=dev)
        view = base[1:].view(tensors[0].shape)
        view.copy_(tensors[0])
        got2 = op(view, *[t.to(dev) for t in tensors[1:]]).cpu().numpy()
        assert np.array_equal(got2, got)


def dims_of(inputs, shapes):
    """{named dimension: value} of tensors of these shapes for input specs like `input0=float32[N:8, C:16]`."""
    env = {}
    for spec, shape in zip(inputs, shapes):
        for d, v in zip(spec.split('[', 1)[1].rstrip(']').split(','), shape):
            if ':' in d:
                env[d.split(':')[0].strip()] = v
    return env


PATCH_CASES = [
    ('output0[N, M] +=! input0[N, K] * input1[K, M]', ['input0=float32[N:64, K:96]', 'input1=float32[K:96, M:128]'], [(64, 96), (96, 128)]),
    ('output0[B, N, M] +=! input0[B, N, K] * input1[B, K, M]', ['input0=float32[B:3, N:32, K:40]', 'input1=float32[B:3, K:40, M:64]'],
     [(3, 32, 40), (3, 40, 64)]),
    ('output0[N, M] +=! input0[N, K] * input1[M, K]', ['input0=float16[N:32, K:64]', 'input1=float16[M:48, K:64]'], [(32, 64), (48, 64)]),
    ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[F, C, KH, KW] where HO in 10, WO in 12',
     ['input0=float32[N:2, C:5, H:12, W:14]', 'input1=float32[F:8, C:5, KH:3, KW:3]'], [(2, 5, 12, 14), (8, 5, 3, 3)]),
    ('output0[N, M] >=! input0[N, K] + input1[K, M]', ['input0=int32[N:16, K:33]', 'input1=int32[K:33, M:20]'], [(16, 33), (33, 20)]),
    # a depthwise filter whose size comes as named dimensions: the kernels of this call have 3 x 3 written into them
    ('output0[N, C, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[C, KH, KW] where HO in 12, WO in 16',
     ['input0=float32[N:3, C:7, H:14, W:18]', 'input1=float32[C:7, KH:3, KW:3]'], [(3, 7, 14, 18), (7, 3, 3)]),
]


@pytest.mark.parametrize('ir,inputs,shapes', PATCH_CASES)
def test_register_tiled_contractions_match_the_oracle(autort, ir, inputs, shapes, monkeypatch):
    """The reduce variant in which a thread owns 4 x 4 neighbouring outputs (what large contractions get) gives the
    oracle's results, and the bits of the one-output-per-thread variant, whose order of accumulation it keeps."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'register-tiled reduce {ir} {shapes}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='patch_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    plan = op.plans_for(dims_of(inputs, shapes))[0]
    assert 'patch' in plan.variants
    g = torch.Generator().manual_seed(len(ir))
    names = [spec.split('=')[0] for spec in inputs]
    tensors = [torch.randint(-1000, 1000, shp, generator=g, dtype=torch.int32) if 'int32' in spec else
               (torch.randn(shp, generator=g) * 0.5).to(torch.float16 if 'float16' in spec else torch.float32)
               for spec, shp in zip(inputs, shapes)]
    total = op(*[t.to(dev) for t in tensors]).numel()
    results = {}
    for tag in ('patch', 'thread'):
        work = total // 16 if tag == 'patch' else total
        monkeypatch.setattr(plan, 'choose', lambda env, ptrs, tag=tag, work=work: (plan.variants[tag], (work + 255) // 256, 256))
        results[tag] = op(*[t.to(dev) for t in tensors]).cpu()
    assert torch.equal(results['patch'], results['thread'])
    out_name = ir.split('[', 1)[0].strip()
    want = CpuModule(parse_program(ir, inputs), fast_math=False)(**{n: t.numpy() for n, t in zip(names, tensors)})[out_name]
    got = results['patch'].numpy()
    if got.dtype.kind == 'i':
        assert np.array_equal(got, want)
    else:
        tol = 1e-2 if got.dtype == np.float16 else 1e-4
        assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=tol, atol=tol)


def test_large_contractions_take_the_register_tiled_variant(autort):
    """Without the matrix-instruction variant a 2048 x 2048 x 256 fp32 matrix product is large enough for the
    register-tiled one (a 1024 x 1024 one is not); the result is the float64 product's."""
    note('register-tiled reduce picked for a 2048x2048x256 fp32 matmul')
    dev = autort.device()
    op = autort.export(ir='output0[N, M] +=! input0[N, K] * input1[K, M]', inputs=['input0=float32[N:2048, K:256]', 'input1=float32[K:256, M:2048]'],
                       name='patch_matmul_2048')
    op.fast_path = None               # the generic lowering is what is tested here
    plan = op.plans[0]
    zero = {n: 0 for n in plan.args}
    assert plan.choose({'N': 2048, 'K': 256, 'M': 2048}, zero)[0] == plan.variants['matrixv']
    for tag in [t for t in plan.variants if t.startswith('matrix')]:
        del plan.variants[tag]
    assert plan.choose({'N': 2048, 'K': 256, 'M': 2048}, zero)[0] == plan.variants['patch']
    assert plan.choose({'N': 2046, 'K': 256, 'M': 2048}, zero)[0] != plan.variants['patch']
    assert plan.choose({'N': 1024, 'K': 256, 'M': 1024}, zero)[0] != plan.variants['patch']
    g = torch.Generator().manual_seed(2)
    a, b = torch.randn(2048, 256, generator=g), torch.randn(256, 2048, generator=g)
    got = op(a.to(dev), b.to(dev)).cpu()
    want = (a.double() @ b.double()).float()
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-3)


MATRIX_CASES = [
    # a convolution; the same with stride 2; a batched product with ragged tiles and k = 5 x 16; fp16 operands cast to
    # float32 with B stored [N, K]; elementwise work on one factor (AntaresIR.md:247 over all of K); a product whose
    # output axes are stored columns first
    ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[F, C, KH, KW] where HO in 32, WO in 32',
     ['input0=float32[N:8, C:16, H:34, W:34]', 'input1=float32[F:64, C:16, KH:3, KW:3]'], [(8, 16, 34, 34), (64, 16, 3, 3)]),
    ('output0[N, F, HO, WO] +=! input0[N, C, HO * 2 + KH, WO * 2 + KW] * input1[F, C, KH, KW] where HO in 32, WO in 32',
     ['input0=float32[N:8, C:16, H:66, W:66]', 'input1=float32[F:70, C:16, KH:3, KW:3]'], [(8, 16, 66, 66), (70, 16, 3, 3)]),
    ('output0[B, N, M] +=! input0[B, N, K] * input1[B, K, M]', ['input0=float32[B:3, N:700, K:80]', 'input1=float32[B:3, K:80, M:520]'],
     [(3, 700, 80), (3, 80, 520)]),
    ('output0[N, M] +=! input0[N, K].to(`float32`) * input1[M, K].to(`float32`)', ['input0=float16[N:1024, K:64]', 'input1=float16[M:1000, K:64]'],
     [(1024, 64), (1000, 64)]),
    ('temp0[K, N] = input0[N, K] + 100; output0[N, M] +=! temp0[K, N] * input1[K, M]',
     ['input0=float32[N:1024, K:512]', 'input1=float32[K:512, M:1024]'], [(1024, 512), (512, 1024)]),
    ('output0[M, N] +=! input0[N, K] * input1[K, M]', ['input0=float32[N:1030, K:64]', 'input1=float32[K:64, M:1024]'], [(1030, 64), (64, 1024)]),
    # k that is no multiple of the tile: a first-layer convolution (3 channels, 7 x 7, stride 2: k = 147), a product with k = 250
    ('output0[N, F, HO, WO] +=! input0[N, C, HO * 2 + KH, WO * 2 + KW] * input1[F, C, KH, KW] where HO in 29, WO in 29',
     ['input0=float32[N:10, C:3, H:64, W:64]', 'input1=float32[F:64, C:3, KH:7, KW:7]'], [(10, 3, 64, 64), (64, 3, 7, 7)]),
    ('output0[N, M] +=! input0[N, K] * input1[M, K]', ['input0=float32[N:1024, K:250]', 'input1=float32[M:1024, K:250]'], [(1024, 250), (1024, 250)]),
    # fp16 operands that are only cast up stay fp16 in the tiles (v_mfma_f32_32x32x16_f16): B stored [K, M], k = 2.5 tiles;
    # a batched product of fp16 operands
    ('output0[N, M] +=! input0[N, K].to(`float32`) * input1[K, M].to(`float32`)', ['input0=float16[N:1100, K:80]', 'input1=float16[K:80, M:1024]'],
     [(1100, 80), (80, 1024)]),
    ('output0[B, N, M] +=! input0[B, N, K].to(`float32`) * input1[B, M, K].to(`float32`)',
     ['input0=float16[B:4, N:520, K:96]', 'input1=float16[B:4, M:500, K:96]'], [(4, 520, 96), (4, 500, 96)]),
    # guarded factors: a convolution that pads by one with zeros (AntaresIR.md:166), in float32 and with fp16 tiles; a
    # product whose first operand is shifted along k and cut where it runs out, lanes along k
    ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH - 1, WO + KW - 1].when([HO + KH - 1 >= 0, HO + KH - 1 < 32, WO + KW - 1 >= 0, '
     'WO + KW - 1 < 32], 0.0) * input1[F, C, KH, KW] where HO in 32, WO in 32',
     ['input0=float32[N:6, C:16, H:32, W:32]', 'input1=float32[F:64, C:16, KH:3, KW:3]'], [(6, 16, 32, 32), (64, 16, 3, 3)]),
    ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH - 1, WO + KW - 1].to(`float32`).when([HO + KH - 1 >= 0, HO + KH - 1 < 30, '
     'WO + KW - 1 >= 0, WO + KW - 1 < 30], 0.0) * input1[F, C, KH, KW].to(`float32`) where HO in 30, WO in 30',
     ['input0=float16[N:5, C:20, H:30, W:30]', 'input1=float16[F:72, C:20, KH:3, KW:3]'], [(5, 20, 30, 30), (72, 20, 3, 3)]),
    ('output0[N, M] +=! input0[N, K + 5].when([K + 5 < 80], 0.0) * input1[K, M] where K in 80',
     ['input0=float32[N:1024, J:80]', 'input1=float32[K:80, M:1024]'], [(1024, 80), (80, 1024)]),
    # channels last (image `[N, H, W, C]`, filter `[KH, KW, C, F]`): the image in 16-byte vectors of channels, the filter staged as it
    # lies; the same with fp16 operands and 24 channels (k = 216: 6.75 tiles)
    ('output0[N, HO, WO, F] +=! input0[N, HO + KH, WO + KW, C] * input1[KH, KW, C, F] where HO in 20, WO in 20',
     ['input0=float32[N:5, H:22, W:22, C:16]', 'input1=float32[KH:3, KW:3, C:16, F:72]'], [(5, 22, 22, 16), (3, 3, 16, 72)]),
    ('output0[N, HO, WO, F] +=! input0[N, HO + KH, WO + KW, C].to(`float32`) * input1[KH, KW, C, F].to(`float32`) where HO in 20, WO in 20',
     ['input0=float16[N:5, H:22, W:22, C:24]', 'input1=float16[KH:3, KW:3, C:24, F:72]'], [(5, 22, 22, 24), (3, 3, 24, 72)]),
    # the guarded factor second: the filter's output channels are the rows, the padded image's positions the columns
    ('output0[F, N, HO, WO] +=! input1[F, C, KH, KW] * input0[N, C, HO + KH - 2, WO + KW - 2].when([HO + KH - 2 >= 0, HO + KH - 2 < 20, '
     'WO + KW - 2 >= 0, WO + KW - 2 < 24], 0.0) where HO in 20, WO in 24',
     ['input0=float32[N:4, C:12, H:20, W:24]', 'input1=float32[F:96, C:12, KH:5, KW:5]'], [(4, 12, 20, 24), (96, 12, 5, 5)]),
]


@pytest.mark.parametrize('ir,inputs,shapes,how', [c + (None,) for c in MATRIX_CASES] +
                         [c + ('guards in the kernel',) for c in MATRIX_CASES if '.when(' in c[0]])
def test_contractions_on_the_matrix_instructions_match_the_oracle(autort, monkeypatch, ir, inputs, shapes, how):
    """Sums of products of two loads whose indices split into a row (or column) part and a k part run on
    v_mfma_f32_32x32x2_f32 when k is a multiple of 16 and there are enough tiles; results are the oracle's to the
    rounding of a float32 sum in another order, and the register-tiled variant gives the same to that rounding.
    A zero-padded factor is normally copied into a padded tensor first (one more statement in front); the cases marked
    'guards in the kernel' switch that off, so that the contraction itself evaluates the conditions - what a program
    gets whose conditions the rewrite does not take."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'matrix-instruction contraction {ir[:60]} {shapes} {how or ""}')
    dev = autort.device()
    if how:
        monkeypatch.setattr('antares_amd.autort.op.pad_guarded_factors', lambda graph, env=None: graph)
    op = autort.export(ir=ir, inputs=inputs, name='mfma_' + str(abs(hash((ir, tuple(inputs), how))) % 10 ** 8))
    op.fast_path = None
    env = dims_of(inputs, shapes)
    plan = op.plans_for(env)[-1]                  # a filter of a few named elements gets kernels of its own
    if '.when(' in ir:
        padded = any(n.endswith('__pad') for n in plan.args)
        assert padded == (how is None) and len(op.plans_for(env)) == (2 if padded else 1)
    assert plan.choose(env, {n: 0 for n in plan.args})[0] in [v for t, v in plan.variants.items() if t.startswith('matrix')]
    assert plan.row_group is None                 # nothing else takes the statement
    g = torch.Generator().manual_seed(len(ir))
    tensors = [torch.randn(shape, generator=g).to(torch.float16 if 'float16' in spec else torch.float32) for spec, shape in zip(inputs, shapes)]
    names = [spec.split('=')[0] for spec in inputs]
    want = CpuModule(parse_program(ir, inputs), fast_math=False)(**{n: t.numpy() for n, t in zip(names, tensors)})['output0']
    K = 1
    for ax, e in plan.reduce_axes:
        K *= e if isinstance(e, int) else env[e]
    scale = 100.0 if '+ 100' in ir else 1.0
    tol = 2e-5 * scale * K ** 0.5 * 4
    M, N, B = (int(np.prod([e if isinstance(e, int) else env[e] for e in plan.matrix[k]])) for k in ('m', 'n', 'batch'))
    rule = plan.choose
    sizes = [('matrix', 128), ('matrix64', 64)]                # blocks of 128 x 128 and of 64 x 64 outputs
    if 'matrixv' in plan.variants and (plan._matrix_choice(env, {n: 0 for n in plan.args})[0] or '').endswith('v'):
        sizes += [('matrixv', 128), ('matrix64v', 64)]          # ... and their forms that fetch rows of k in 16-byte vectors
        ptrs = {n: 0 for n in plan.args}
        assert plan.choose(env, ptrs)[0] in (plan.variants['matrixv'], plan.variants['matrix64v'])
        ptrs[plan.matrix['vec_tensors'][0]] = 8                 # a tensor that is not 16-byte aligned: scalar fetches
        assert plan.choose(env, ptrs)[0] in (plan.variants['matrix'], plan.variants['matrix64'])
    for tag, side in sizes:
        blocks = ((M + side - 1) // side) * ((N + side - 1) // side) * B
        plan.choose = lambda env_, ptrs, tag=tag, blocks=blocks: (plan.variants[tag], blocks, 256)
        got = op(*[t.to(dev) for t in tensors]).cpu().numpy()
        assert got.shape == want.shape
        assert np.allclose(got, want, rtol=1e-4, atol=tol), (tag, np.abs(got - want).max())
    # the same statement through the register-tiled variant
    plan.choose = rule
    for tag in [t for t in plan.variants if t.startswith('matrix')]:
        del plan.variants[tag]
    apart = op(*[t.to(dev) for t in tensors]).cpu().numpy()
    assert np.allclose(got, apart, rtol=1e-4, atol=tol)


@pytest.mark.parametrize('ir,inputs,shapes', [
    ('output0[N, M] +=! input0[N, K] * input1[K, M]', ['input0=float16[N:1024, K:512]', 'input1=float16[K:512, M:1000]'], [(1024, 512), (512, 1000)]),
    ('output0[B, N, M] +=! input0[B, N, K] * input1[B, M, K]', ['input0=float16[B:3, N:300, K:200]', 'input1=float16[B:3, M:260, K:200]'],
     [(3, 300, 200), (3, 260, 200)]),
])
def test_fp16_contractions_sum_in_float32_on_the_matrix_instructions(autort, ir, inputs, shapes):
    """A float16 sum of products of two float16 loads (AntaresIR.md:115 with float16 tensors) runs on
    v_mfma_f32_32x32x16_f16: exact products, a float32 sum, one rounding at the end.  The reference rounds every product
    and every partial sum to float16 (the oracle does the same); the GPU result must be within one float16 rounding
    of the float64 result, never further from it than the oracle's, and within the oracle's own drift of the oracle."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'fp16 contraction on the matrix instructions {ir} {shapes}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='mfma_f16_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    op.fast_path = None
    env = dims_of(inputs, shapes)
    plan = op.plans_for(env)[-1]
    g = torch.Generator().manual_seed(len(ir))
    a, b = [(torch.randn(shape, generator=g) * 0.5).half() for shape in shapes]
    want = CpuModule(parse_program(ir, inputs), fast_math=False)(input0=a.numpy(), input1=b.numpy())['output0'].astype(np.float64)
    exact = torch.einsum('...nk,...km->...nm', a.double(), b.double() if ir.endswith('[K, M]') else b.double().transpose(-1, -2)).numpy()
    drift = np.abs(want - exact).max()
    M, N, B = (int(np.prod([e if isinstance(e, int) else env[e] for e in plan.matrix[k]])) for k in ('m', 'n', 'batch'))
    assert plan.choose(env, {n: 0 for n in plan.args})[0] in (plan.variants['matrixv'], plan.variants['matrix64v'])
    for tag, side in (('matrix', 128), ('matrix64', 64), ('matrixv', 128), ('matrix64v', 64)):
        blocks = ((M + side - 1) // side) * ((N + side - 1) // side) * B
        plan.choose = lambda env_, ptrs, tag=tag, blocks=blocks: (plan.variants[tag], blocks, 256)
        out = op(a.to(dev), b.to(dev))
        assert out.dtype == torch.float16 and tuple(out.shape) == exact.shape
        got = out.cpu().numpy().astype(np.float64)
        # one float16 rounding of the result, plus what a float32 sum of K terms of this size may be off by
        assert np.all(np.abs(got - exact) <= 2.0 ** -10 * np.abs(exact) + 2e-4), (tag, np.abs(got - exact).max())
        assert np.abs(got - exact).max() <= drift and np.abs(got - want).max() <= 2 * drift + 1e-3, (tag, drift)


@pytest.mark.parametrize('ir,inputs,shapes,vectors', [
    ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[F, C, KH, KW] where HO in 7, WO in 7',
     ['input0=float32[N:4, C:512, H:9, W:9]', 'input1=float32[F:256, C:512, KH:3, KW:3]'], [(4, 512, 9, 9), (256, 512, 3, 3)], True),
    ('output0[N, M] +=! input0[N, K] * input1[M, K]', ['input0=float32[N:320, K:4096]', 'input1=float32[M:512, K:4096]'], [(320, 4096), (512, 4096)], True),
    ('output0[B, N, M] +=! input0[B, N, K] * input1[B, K, M]', ['input0=float32[B:2, N:256, K:2048]', 'input1=float32[B:2, K:2048, M:200]'],
     [(2, 256, 2048), (2, 2048, 200)], True),
    ('output0[N, M] +=! input0[N, K].to(`float32`) * input1[M, K].to(`float32`)', ['input0=float16[1024, 2048]', 'input1=float16[512, 2048]'],
     [(1024, 2048), (512, 2048)], True),
])
def test_contractions_with_few_output_tiles_are_cut_into_slices_of_k(autort, ir, inputs, shapes, vectors):
    """A contraction whose 64 x 64 output tiles number fewer than two per compute unit, over at least 1024 values of k,
    runs as a batch of slices of k on the matrix instructions plus a sum over the slices; an operand that lies as rows
    of k keeps its 16-byte fetches inside a slice.  Results against the oracle, to the rounding of a float32 sum in
    another order."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'sliced contraction {ir[:60]} {shapes}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='sliced_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    op.fast_path = None
    env = dims_of(inputs, shapes)
    plans = op.plans_for(env)
    assert len(plans) == 2 and plans[0].matrix is not None and plans[1].matrix is None
    sym, blocks, _ = plans[0].choose(env, {n: 0 for n in plans[0].args})
    assert blocks >= 512 or plans[0].matrix['batch'][0] == 8          # the slices fill the chip, or there are 8 of them
    assert sym in [v for t, v in plans[0].variants.items() if t.startswith('matrix') and t.endswith('v') == vectors]
    g = torch.Generator().manual_seed(len(ir))
    tensors = [torch.randn(shape, generator=g).to(torch.float16 if 'float16' in spec else torch.float32) for spec, shape in zip(inputs, shapes)]
    names = [spec.split('=')[0] for spec in inputs]
    want = CpuModule(parse_program(ir, inputs), fast_math=False)(**{n: t.numpy() for n, t in zip(names, tensors)})['output0']
    K = int(np.prod([e if isinstance(e, int) else env[e] for _, e in parse_program(ir, inputs).statements[0].reduce_axes]))
    got = op(*[t.to(dev) for t in tensors]).cpu().numpy()
    assert got.shape == want.shape and np.allclose(got, want, rtol=1e-4, atol=2e-5 * K ** 0.5 * 4), np.abs(got - want).max()


@pytest.mark.parametrize('ir,inputs,shapes', [
    # both operands stored along rows; the second one only, batched (the V of an attention), ragged tiles, k = 2.5 tiles
    ('output0[N, M] +=! input0[K, N].to(`float32`) * input1[K, M].to(`float32`)', ['input0=float16[K:96, N:1000]', 'input1=float16[K:96, M:520]'],
     [(96, 1000), (96, 520)]),
    ('output0[B, S, D] +=! input0[B, S, T].to(`float32`) * input1[B, T, D].to(`float32`)', ['input0=float16[B:3, S:300, T:80]', 'input1=float16[B:3, T:80, D:128]'],
     [(3, 300, 80), (3, 80, 128)]),
    # float32: both operands along rows; the second one only, batched, k = 2.5 tiles of the big blocks
    ('output0[N, M] +=! input0[K, N] * input1[K, M]', ['input0=float32[K:72, N:1000]', 'input1=float32[K:72, M:516]'], [(72, 1000), (72, 516)]),
    ('output0[B, S, D] +=! input0[B, S, T] * input1[B, T, D]', ['input0=float32[B:3, S:300, T:40]', 'input1=float32[B:3, T:40, D:128]'],
     [(3, 300, 40), (3, 40, 128)]),
])
def test_operands_stored_along_rows_are_staged_as_they_lie(autort, ir, inputs, shapes):
    """An operand whose neighbouring rows (columns) are neighbours in memory - `input1[K, M]` - is fetched in 16-byte
    vectors of rows and staged in LDS as [k][row]; fp16 tiles are transposed on their way to the matrix instruction by
    ds_read_b64_tr_b16, float32 ones are read element by element.  The result is that of the kernels that stage it row
    by row, bit for bit, and the oracle's."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'fp16 operands staged as they lie {ir} {shapes}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='mfma_tr_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    op.fast_path = None
    env = dims_of(inputs, shapes)
    plan = op.plans_for(env)[-1]
    zero = {n: 0 for n in plan.args}
    assert plan.choose(env, zero)[0] in (plan.variants['matrixv'], plan.variants['matrix64v'])
    odd = {k: (v + 2 if k in ('M', 'D') else v) for k, v in env.items()}          # a row length that is no whole number of vectors
    assert plan.choose(odd, zero)[0] in (plan.variants['matrix'], plan.variants['matrix64'])
    g = torch.Generator().manual_seed(len(ir))
    a, b = [(torch.randn(shape, generator=g) * 0.5).to(torch.float16 if 'float16' in inputs[0] else torch.float32) for shape in shapes]
    want = CpuModule(parse_program(ir, inputs), fast_math=False)(input0=a.numpy(), input1=b.numpy())['output0']
    M, N, B = (int(np.prod([e if isinstance(e, int) else env[e] for e in plan.matrix[k]])) for k in ('m', 'n', 'batch'))
    got = {}
    for tag, side in (('matrix', 128), ('matrix64', 64), ('matrixv', 128), ('matrix64v', 64)):
        blocks = ((M + side - 1) // side) * ((N + side - 1) // side) * B
        plan.choose = lambda env_, ptrs, tag=tag, blocks=blocks: (plan.variants[tag], blocks, 256)
        got[tag] = op(a.to(dev), b.to(dev)).cpu().numpy()
        assert np.allclose(got[tag], want, rtol=1e-4, atol=1e-3), (tag, np.abs(got[tag] - want).max())
    # the same products in the same order of k inside a tile: the bits agree between the two ways of staging
    assert np.array_equal(got['matrix'], got['matrixv']) and np.array_equal(got['matrix64'], got['matrix64v'])


@pytest.mark.parametrize('ir,inputs,shapes', [
    ('output0[N, M] +=! input0[N, K].cast(`int32`) * input1[M, K].cast(`int32`)', ['input0=int8[N:1000, K:528]', 'input1=int8[M:1024, K:528]'],
     [(1000, 528), (1024, 528)]),
    ('output0[N, M] +=! input0[N, K].cast(`int32`) * input1[K, M].cast(`int32`)', ['input0=int8[N:300, K:200]', 'input1=int8[K:200, M:260]'],
     [(300, 200), (200, 260)]),
    ('output0[B, N, M] +=! input0[B, N, K].cast(`int32`) * input1[B, M, K].cast(`int32`)', ['input0=int8[B:2, N:256, K:4096]', 'input1=int8[B:2, M:192, K:4096]'],
     [(2, 256, 4096), (2, 192, 4096)]),
    # the second operand stored along its columns, whole vectors of them: staged as it lies, transposed by ds_read_b64_tr_b8
    ('output0[N, M] +=! input0[N, K].cast(`int32`) * input1[K, M].cast(`int32`)', ['input0=int8[N:200, K:160]', 'input1=int8[K:160, M:272]'],
     [(200, 160), (160, 272)]),
])
def test_int8_contractions_are_bit_exact_on_the_matrix_instructions(autort, ir, inputs, shapes):
    """An int32 sum of products of two int8 loads cast to int32 runs on v_mfma_i32_32x32x32_i8: exact products, exact
    sums, and integer sums do not depend on their order - every kernel gives the integers of a 64-bit product (and the
    oracle's), bit for bit; the third case is also cut into slices of k."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'int8 contraction on the matrix instructions {ir} {shapes}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='mfma_i8_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    op.fast_path = None
    env = dims_of(inputs, shapes)
    plan = op.plans_for(env)[0]
    assert plan.matrix is not None and len(op.plans_for(env)) == (2 if 'B:2' in inputs[0] else 1)
    g = torch.Generator().manual_seed(len(ir))
    a, b = [torch.randint(-128, 128, shape, generator=g, dtype=torch.int8) for shape in shapes]
    exact = torch.einsum('...nk,...km->...nm', a.long(), b.long() if ir.split('input1')[1].startswith('[K, M]') else b.long().transpose(-1, -2)).to(torch.int32).numpy()
    if a.numel() <= 1 << 20:
        want = CpuModule(parse_program(ir, inputs), fast_math=False)(input0=a.numpy(), input1=b.numpy())['output0']
        assert np.array_equal(want, exact)
    M, N, B = (int(np.prod([e if isinstance(e, int) else env[e] for e in plan.matrix[k]])) for k in ('m', 'n', 'batch'))
    for tag, side in (('matrix', 128), ('matrix64', 64), ('matrixv', 128), ('matrix64v', 64)):
        if tag not in plan.variants or (tag.endswith('v') and not (plan._matrix_choice(env, {n: 0 for n in plan.args})[0] or '').endswith('v')):
            continue                # the vector kernels are launched for whole vectors only
        blocks = ((M + side - 1) // side) * ((N + side - 1) // side) * B
        plan.choose = lambda env_, ptrs, tag=tag, blocks=blocks: (plan.variants[tag], blocks, 256)
        got = op(a.to(dev), b.to(dev))
        assert got.dtype == torch.int32 and np.array_equal(got.cpu().numpy(), exact), tag


@pytest.mark.parametrize('in_kernel', [False, True])
def test_int8_padded_convolution_is_bit_exact(autort, monkeypatch, in_kernel):
    """A zero-padded 3 x 3 convolution of int8 images and filters into int32 on v_mfma_i32_32x32x32_i8, with the image
    copied into a padded tensor first and with the conditions evaluated in the contraction: torch's integers both ways."""
    note(f'int8 padded convolution, guards {"in the kernel" if in_kernel else "in a padded copy"}')
    dev = autort.device()
    if in_kernel:
        monkeypatch.setattr('antares_amd.autort.op.pad_guarded_factors', lambda graph, env=None: graph)
    ir = ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH - 1, WO + KW - 1].cast(`int32`).when([HO + KH - 1 >= 0, HO + KH - 1 < 20, '
          'WO + KW - 1 >= 0, WO + KW - 1 < 20], 0) * input1[F, C, KH, KW].cast(`int32`) where HO in 20, WO in 20')
    op = autort.export(ir=ir, inputs=['input0=int8[N:3, C:24, H:20, W:20]', 'input1=int8[F:72, C:24, KH:3, KW:3]'], name=f'conv_i8_{int(in_kernel)}')
    env = {'N': 3, 'C': 24, 'H': 20, 'W': 20, 'F': 72, 'KH': 3, 'KW': 3}
    plans = op.plans_for(env)
    assert len(plans) == (1 if in_kernel else 2) and plans[-1].matrix is not None and plans[-1].matrix['half_tiles']
    g = torch.Generator().manual_seed(9)
    x, w = torch.randint(-128, 128, (3, 24, 20, 20), generator=g, dtype=torch.int8), torch.randint(-128, 128, (72, 24, 3, 3), generator=g, dtype=torch.int8)
    want = torch.nn.functional.conv2d(x.double(), w.double(), padding=1).to(torch.int32)        # sums below 2^53: exact
    got = op(x.to(dev), w.to(dev)).cpu()
    assert got.dtype == torch.int32 and torch.equal(got, want)


TAIL_CASES = [
    # AntaresIR.md:248-250 (ConvBiasRelu tail fusion); a product with a scaled result, a per-column and a per-element
    # term under a tanh; a float16 result of a float32 sum; a column-wise maximum with a conditional store behind it
    ('conv_out[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[KH, KW, C, F] where HO in 30, WO in 30; '
     'conv_bias[N, F, HO, WO] = conv_out[N, F, HO, WO] + input2[0, 0, 0, F]; '
     'output0[N, F, HO, WO] = conv_bias[N, F, HO, WO].when(conv_bias[N, F, HO, WO] > 0.0, 0.0)',
     ['input0=float32[N:4, C:16, H:32, W:32]', 'input1=float32[KH:3, KW:3, C:16, F:64]', 'input2=float32[1, 1, 1, F:64]'],
     [(4, 16, 32, 32), (3, 3, 16, 64), (1, 1, 1, 64)], True),
    ('acc[N, M] +=! input0[N, K] * input1[M, K]; output0[N, M] = (acc[N, M] * 0.5 + input2[M] + input3[N, M]).call(`tanh`)',
     ['input0=float32[N:300, K:256]', 'input1=float32[M:200, K:256]', 'input2=float32[M:200]', 'input3=float32[N:300, M:200]'],
     [(300, 256), (200, 256), (200,), (300, 200)], True),
    ('acc[B, N, M] +=! input0[B, N, K].to(`float32`) * input1[B, K, M].to(`float32`); output0[B, N, M] = (acc[B, N, M] + input2[B, M]).to(`float16`)',
     ['input0=float16[B:3, N:128, K:64]', 'input1=float16[B:3, K:64, M:160]', 'input2=float32[B:3, M:160]'], [(3, 128, 64), (3, 64, 160), (3, 160)], True),
    ('top[C] >=! input0[N, C]; output0[C] = top[C].when(top[C] > input1[C])', ['input0=float32[N:40, C:20000]', 'input1=float32[C:20000]', 'output0=float32[C:20000]'],
     [(40, 20000), (20000,), (20000,)], False),
]


@pytest.mark.parametrize('ir,inputs,shapes,matrix', TAIL_CASES)
def test_a_map_behind_a_reduction_is_applied_at_its_stores(autort, ir, inputs, shapes, matrix):
    """Tail fusion (AntaresIR.md:248-250): the kernels of the reduction store f(result, other tensors) straight into the
    map's output; the reduction's own output is never written and the map's kernels are not launched.  Every variant of
    the fused kernels against the oracle, which runs the statements one by one."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'tail fusion {ir[:60]} {shapes}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='tail_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    op.fast_path = None
    env = dims_of(inputs, shapes)
    plans = op.plans_for(env)
    assert len(plans) == 2 and plans[0].covers == 2 and plans[0].output == 'output0' and plans[0].args[-1] == 'output0'
    assert not any(a in plans[0].args for a in ('acc', 'conv_out', 'top'))
    assert ('matrix' in plans[0].variants) == matrix
    g = torch.Generator().manual_seed(len(ir))
    tensors = [(torch.randn(shape, generator=g) * 0.5).to(torch.float16 if 'float16' in spec else torch.float32) for spec, shape in zip(inputs, shapes)]
    names = [spec.split('=')[0] for spec in inputs]
    want = CpuModule(parse_program(ir, inputs), fast_math=False)(**{n: t.numpy().copy() for n, t in zip(names, tensors)})['output0'].astype(np.float32)
    plan, total = plans[0], int(np.prod(want.shape))
    launches = [('thread', (total + 255) // 256), ('wave', (total + 3) // 4), ('block', total)]
    if 'patch' in plan.variants and plan._patches(env, total):
        launches.append(('patch', (plan._patches(env, total) + 255) // 256))
    if matrix:
        M, N, B = (int(np.prod([e if isinstance(e, int) else env[e] for e in plan.matrix[k]])) for k in ('m', 'n', 'batch'))
        launches += [(tag, ((M + side - 1) // side) * ((N + side - 1) // side) * B) for tag, side in (('matrix', 128), ('matrix64', 64)) if tag in plan.variants]
        if (plan._matrix_choice(env, {n: 0 for n in plan.args})[0] or '').endswith('v'):       # whole vectors everywhere they are fetched
            launches += [(tag, ((M + side - 1) // side) * ((N + side - 1) // side) * B) for tag, side in (('matrixv', 128), ('matrix64v', 64))]
    tol = 1e-2 if want.dtype == np.float16 or 'float16' in ir else 2e-4
    for tag, grid in launches:
        plan.choose = lambda env_, ptrs, tag=tag, grid=grid: (plan.variants[tag], min(grid, 65536), 256)
        got = op(*[t.clone().to(dev) for t in tensors]).float().cpu().numpy()
        assert got.shape == want.shape and np.allclose(got, want, rtol=tol, atol=tol), (tag, np.abs(got - want).max())


def test_one_operator_called_at_several_sizes_gets_the_rewrites_of_each(autort):
    """A padded convolution with bias and ReLU exported once with named dimensions and called with three batch sizes and
    two filter sizes: every call finds (or builds) the kernels of its own dimension values - filter size written in,
    operand padded by a statement in front, tail applied at the stores - and gives torch's result."""
    note('padded conv + bias + relu at several sizes through one operator')
    dev = autort.device()
    ir = ('conv[N, F, HO, WO] +=! input0[N, C, HO + KH - KH.val() / 2, WO + KW - KW.val() / 2].when([HO + KH - KH.val() / 2 >= 0, '
          'HO + KH - KH.val() / 2 < 24, WO + KW - KW.val() / 2 >= 0, WO + KW - KW.val() / 2 < 24], 0.0) * input1[F, C, KH, KW] where HO in 24, WO in 24; '
          'output0[N, F, HO, WO] = (conv[N, F, HO, WO] + input2[F]).call(`max`, [0.0])')
    op = autort.export(ir=ir, inputs=['input0=float32[N:4, C:16, H:24, W:24]', 'input1=float32[F:64, C:16, KH:3, KW:3]', 'input2=float32[F:64]'],
                       name='conv_bias_relu_sizes')
    g = torch.Generator().manual_seed(5)
    seen = set()
    for n, k in ((4, 3), (2, 3), (7, 5), (4, 3)):
        x, w, b = torch.randn(n, 16, 24, 24, generator=g), torch.randn(64, 16, k, k, generator=g) * 0.1, torch.randn(64, generator=g)
        got = op(x.to(dev), w.to(dev), b.to(dev)).cpu()
        want = torch.relu(torch.nn.functional.conv2d(x.double(), w.double(), b.double(), padding=k // 2)).float()
        assert got.shape == want.shape and torch.allclose(got, want, rtol=1e-4, atol=1e-3), (n, k, (got - want).abs().max())
        seen.add((n, k))
        assert len(op._variants) == len(seen)
    env = {'N': 7, 'C': 16, 'H': 24, 'W': 24, 'F': 64, 'KH': 5, 'KW': 5}
    plans = op.plans_for(env)
    # the copy padded by two on each side, then the contraction with the tail at its stores (the map's own plan is not launched)
    assert [p.output for p in plans] == ['input0__pad', 'output0', 'output0'] and plans[1].covers == 2 and plans[1].matrix is not None
    assert dict(plans[1].reduce_axes)['KH'] == 5


ROW_GROUP_CASES = [
    # program, inputs, shapes, does the row kernel run at these extents
    ('temp0[N] >=! input0[N, C]; temp1[N] +=! (input0[N, C] - temp0[N]).call(`exp`); '
     'output0[N, C] = (input0[N, C] - temp0[N]).call(`exp`) / temp1[N]', ['input0=float32[N:37, C:1000]'], [(37, 1000)], True),
    ('temp0[N] +=! input0[N, C]; temp1[N] +=! input0[N, C] * input0[N, C]; '
     'output0[N, C] = (input0[N, C] * C.val() - temp0[N]) * (temp1[N] * C.val() - temp0[N] * temp0[N] + 1e-5).call(`rsqrt`)',
     ['input0=float32[N:32, C:1024]'], [(32, 1024)], True),
    # rows of a 3-D tensor, a per-column weight and a per-row shift besides the row itself, fp16 storage
    ('ss[B, N] +=! x[B, N, C].to(`float32`) * x[B, N, C].to(`float32`); '
     'y[B, N, C] = (x[B, N, C].to(`float32`) * (ss[B, N] / C.val() + 1e-5).call(`rsqrt`) * w[C].to(`float32`) + shift[B, N]).to(`float16`)',
     ['x=float16[B:3, N:17, C:520]', 'w=float16[C:520]', 'shift=float32[B:3, N:17]'], [(3, 17, 520), (520,), (3, 17)], True),
    # integer rows: maximum and count of the maxima, exact
    ('top[N] >=! v[N, C]; hits[N] +=! (v[N, C] == top[N]).to(`int32`); out[N, C] = (top[N] - v[N, C]) * hits[N]',
     ['v=int32[N:50, C:300]'], [(50, 300)], True),
    # many short rows (a wavefront per row), fp16 vectors of 8; a long row that is walked; a row of 16 vectors per lane
    ('ss[N] +=! x[N, C].to(`float32`) * x[N, C].to(`float32`); '
     'y[N, C] = (x[N, C].to(`float32`) * (ss[N] / C.val() + 1e-5).call(`rsqrt`) * w[C].to(`float32`)).to(`float16`)',
     ['x=float16[N:9001, C:264]', 'w=float16[C:264]'], [(9001, 264), (264,)], True),
    ('temp0[N] +=! input0[N, C]; temp1[N] +=! input0[N, C] * input0[N, C]; '
     'output0[N, C] = (input0[N, C] * C.val() - temp0[N]) * (temp1[N] * C.val() - temp0[N] * temp0[N] + 1e-5).call(`rsqrt`)',
     ['input0=float32[N:5, C:20001]'], [(5, 20001)], True),
    ('temp0[N] +=! input0[N, C]; temp1[N] +=! input0[N, C] * input0[N, C]; '
     'output0[N, C] = (input0[N, C] * C.val() - temp0[N]) * (temp1[N] * C.val() - temp0[N] * temp0[N] + 1e-5).call(`rsqrt`)',
     ['input0=float32[N:9, C:12000]'], [(9, 12000)], True),
    # reductions with no map behind them: row sums, an integer row maximum of products with a weight row
    ('output0[N] +=! input0[N, C]', ['input0=float32[N:600, C:1000]'], [(600, 1000)], True),
    ('top[B, N] >=! v[B, N, C] * w[C]', ['v=int32[B:2, N:300, C:300]', 'w=int32[C:300]'], [(2, 300, 300), (300,)], True),
    # short rows: the per-statement kernels run, same result
    ('temp0[N] >=! input0[N, C]; temp1[N] +=! (input0[N, C] - temp0[N]).call(`exp`); '
     'output0[N, C] = (input0[N, C] - temp0[N]).call(`exp`) / temp1[N]', ['input0=float32[N:300, C:64]'], [(300, 64)], False),
]


@pytest.mark.parametrize('ir,inputs,shapes,applies', ROW_GROUP_CASES)
def test_row_reductions_and_their_map_run_as_one_kernel(autort, ir, inputs, shapes, applies):
    """Reductions over the last axis followed by the map that uses them (softmax, layer normalisation,
    AntaresIR.md:226-232) are computed by one kernel, a block per row; results are the oracle's, and they equal
    what the per-statement kernels give to the rounding of the reductions."""
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    note(f'row group {ir[:40]} {shapes}')
    dev = autort.device()
    op = autort.export(ir=ir, inputs=inputs, name='rows_' + str(abs(hash((ir, tuple(inputs)))) % 10 ** 8))
    group = op.plans[0].row_group
    assert group is not None and group.count == len(op.plans) == ir.count(';') + 1
    env = {}
    for spec, shape in zip(inputs, shapes):
        for d, v in zip(spec.split('[', 1)[1].rstrip(']').split(','), shape):
            env[d.split(':')[0].strip()] = v
    assert (group.choose(env, {n: 0 for n in group.args})[1] > 0) == applies
    g = torch.Generator().manual_seed(len(ir))
    tensors, names = [], []
    for spec, shape in zip(inputs, shapes):
        name, rest = spec.split('=')
        names.append(name)
        if rest.startswith('int32'):
            tensors.append(torch.randint(-40, 40, shape, generator=g, dtype=torch.int32))
        else:
            tensors.append(torch.randn(shape, generator=g).to(torch.float16 if rest.startswith('float16') else torch.float32))
    got = op(*[t.to(dev) for t in tensors]).cpu().numpy()
    out_name = ir.rsplit(';', 1)[-1].split('[', 1)[0].strip()
    want = CpuModule(parse_program(ir, inputs), fast_math=False)(**{n: t.numpy() for n, t in zip(names, tensors)})[out_name]
    if got.dtype.kind == 'i':
        assert np.array_equal(got, want)
    else:
        tol = 2e-2 if got.dtype == np.float16 else 2e-5
        assert np.allclose(got.astype(np.float64), want.astype(np.float64), rtol=tol, atol=tol), np.abs(got.astype(np.float64) - want).max()
    # statement by statement (the row kernel switched off): same values up to the order of the sums
    for p in op.plans:
        p.row_group = None
    apart = op(*[t.to(dev) for t in tensors]).cpu().numpy()
    if got.dtype.kind == 'i':
        assert np.array_equal(got, apart)
    else:
        assert np.allclose(got.astype(np.float64), apart.astype(np.float64), rtol=tol, atol=tol)


@pytest.mark.parametrize('ir,ta,tb,M,N,K', [
    ('out[M, N] +=! x[K, M] * w[K, N]', True, False, 1028, 512, 96),
    ('out[M, N] +=! x[M, K] * w[N, K]', False, True, 1000, 1030, 64),       # a linear layer: N need not be a multiple of 4
    ('out[M, N] +=! x[K, M] * w[N, K]', True, True, 2048, 129, 160),
    ('out[M, N] +=! x[M, K] * w[N, K]', False, True, 4096, 4096, 1024),
])
def test_fp32_gemm_with_operands_stored_the_other_way_round(autort, ir, ta, tb, M, N, K):
    """`A^T B`, `A B^T` and `A^T B^T` in float32 go to art_gemm_f32_ex; results are the float64 products' to fp32
    accuracy, and a one-hot operand pins which axis of each operand is k."""
    note(f'gemm_f32 layouts {ir} {M}x{N}x{K}')
    dev = autort.device()
    sa, sb = (f'x=float32[K:{K}, M:{M}]' if ta else f'x=float32[M:{M}, K:{K}]'), (f'w=float32[N:{N}, K:{K}]' if tb else f'w=float32[K:{K}, N:{N}]')
    op = autort.export(ir=ir, inputs=[sa, sb], name=f'gemm_f32_l{int(ta)}{int(tb)}_{M}_{N}_{K}')
    assert op.fast_path is not None
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn((K, M) if ta else (M, K), generator=g)
    b = torch.randn((N, K) if tb else (K, N), generator=g)
    got = op(a.to(dev), b.to(dev)).cpu()
    am, bm = (a.t() if ta else a).double(), (b.t() if tb else b).double()
    want = am @ bm
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-5 * max(1.0, K ** 0.5)), (got.double() - want).abs().max()
    if M <= 2048:
        sel = torch.zeros(M, K)
        sel[torch.arange(M), torch.arange(M) % K] = 1.0              # row m of the result = row m % K of B
        sel_in = sel.t().contiguous() if ta else sel
        assert torch.equal(op(sel_in.to(dev), b.to(dev)).cpu(), (b.t() if tb else b)[torch.arange(M) % K].contiguous())
