"""fp16 GEMM on the matrix cores against the oracle (fp32 accumulate, fp16 out; rtol/atol 1e-2)."""
import numpy as np
import pytest
import torch

from antares_amd import workloads

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures('oracle_built')]
FP16_TOL = dict(rtol=1e-2, atol=1e-2)


@pytest.fixture(scope='module')
def gemm():
    import autort
    from antares_amd.autort import patterns
    return autort, autort.export(ir=patterns.GEMM_F16_IR, inputs=patterns.GEMM_F16_INPUTS, name='gemm_f16')


def oracle_gemm(a, b):
    """fp32-accumulated product of the fp16 operands, rounded to fp16 (float64 sums are exact enough to stand in
    for the fp32 loop nest at these sizes; the oracle's own loop nest is used for the small case below)."""
    return (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32).astype(np.float16)


def test_small_against_loop_nest_oracle(gemm):
    from antares_amd.autort import patterns
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    autort, op = gemm
    print('[case] gemm 256x256x64 vs loop nest', flush=True)
    g = torch.Generator().manual_seed(1)
    a = (torch.randn(256, 64, generator=g) * 0.5).half()
    b = (torch.randn(64, 256, generator=g) * 0.5).half()
    want = CpuModule(parse_program(patterns.GEMM_F16_IR, patterns.GEMM_F16_INPUTS), fast_math=False)(a=a.numpy(), b=b.numpy())['c']
    got = op(a.to(autort.device()), b.to(autort.device())).cpu().numpy()
    assert np.allclose(got.astype(np.float32), want.astype(np.float32), **FP16_TOL)


@pytest.mark.parametrize('M,N,K', [(256, 256, 64), (256, 512, 128), (512, 256, 192), (1024, 2048, 1024), (4096, 4096, 4096),
                                   # edge tiles: any M, N % 8 == 0
                                   (1, 256, 64), (100, 264, 128), (257, 248, 64), (300, 1000, 192), (64, 4096, 4096), (777, 8, 64)])
def test_against_float64_product(gemm, M, N, K):
    autort, op = gemm
    print(f'[case] gemm {M}x{N}x{K}', flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    a = (torch.randn(M, K, generator=g) * 0.02).half()
    b = (torch.randn(K, N, generator=g) * 0.02).half()
    dev = autort.device()
    got = op(a.to(dev), b.to(dev))
    assert op.fast_path is not None and got.dtype == torch.float16 and got.shape == (M, N)
    want = torch.from_numpy(oracle_gemm(a.numpy(), b.numpy()))
    assert torch.allclose(got.cpu().float(), want.float(), **FP16_TOL)
    # identity and one-hot structure: pins operand order / transposition
    if M == N == 256:
        eye = torch.eye(256, dtype=torch.float16)
        bb = (torch.randn(256, 256, generator=g)).half()
        f = autort.export(ir=op.ir, inputs=['a=float16[M:256, K:256]', 'b=float16[K:256, N:256]'], name='gemm_f16_sq')
        assert torch.equal(f(eye.to(dev), bb.to(dev)).cpu(), bb)
        assert torch.equal(f(bb.to(dev), eye.to(dev)).cpu(), bb)


@pytest.mark.parametrize('threads', [256, 512])
@pytest.mark.parametrize('M,N,K', [(256, 256, 64), (300, 1000, 192), (1024, 2048, 1024), (4096, 4096, 1024)])
def test_both_block_shapes_against_float64_product(gemm, threads, M, N, K):
    """`art_gemm_f16_tuned`: the 256 x 256 tile worked by 2 x 2 wavefronts (256 threads) or by 2 x 4 (512 threads) -
    the launch parameter `tune:N` searches; the library's own choice is 256 threads."""
    from ctypes import c_void_p
    from antares_amd.runtime import capi
    autort, _ = gemm
    print(f'[case] art_gemm_f16_tuned threads={threads} {M}x{N}x{K}', flush=True)
    g = torch.Generator().manual_seed(M + N + K + threads)
    a = (torch.randn(M, K, generator=g) * 0.02).half()
    b = (torch.randn(K, N, generator=g) * 0.02).half()
    dev = autort.device()
    capi.init(dev.index or 0)
    ad, bd = a.to(dev), b.to(dev)
    c = torch.empty(M, N, dtype=torch.float16, device=dev)
    capi.check(capi.lib().art_gemm_f16_tuned(c_void_p(ad.data_ptr()), c_void_p(bd.data_ptr()), c_void_p(c.data_ptr()), M, N, K, threads,
                                             c_void_p(torch.cuda.current_stream().cuda_stream)))
    want = torch.from_numpy(oracle_gemm(a.numpy(), b.numpy()))
    assert torch.allclose(c.cpu().float(), want.float(), **FP16_TOL)
    other = torch.empty_like(c)
    capi.check(capi.lib().art_gemm_f16_tuned(c_void_p(ad.data_ptr()), c_void_p(bd.data_ptr()), c_void_p(other.data_ptr()), M, N, K,
                                             768 - threads, c_void_p(torch.cuda.current_stream().cuda_stream)))
    assert torch.equal(c, other)            # same k order per output: the two shapes agree bit for bit
    assert capi.lib().art_gemm_f16_tuned(c_void_p(ad.data_ptr()), c_void_p(bd.data_ptr()), c_void_p(c.data_ptr()), M, N, K, 128,
                                         c_void_p(0)) != 0


def test_shapes_the_kernel_does_not_take_use_the_generic_lowering(gemm):
    """K % 64 != 0 (or N % 8 != 0) is left to the generic reduce lowering."""
    autort, op = gemm
    print('[case] gemm 96x80x40 (generic lowering)', flush=True)
    g = torch.Generator().manual_seed(5)
    a = (torch.randn(96, 40, generator=g) * 0.1).half()
    b = (torch.randn(40, 80, generator=g) * 0.1).half()
    got = op(a.to(autort.device()), b.to(autort.device())).cpu().numpy()
    assert np.allclose(got.astype(np.float32), oracle_gemm(a.numpy(), b.numpy()).astype(np.float32), **FP16_TOL)


def test_8192_cubed_through_a_random_projection(gemm):
    """The larger benchmark size, checked by a property that needs O(n^2) work on the host:
    (A B) v = A (B v) for a random v, in float64 from the fp16 operands and the fp16 result."""
    autort, op = gemm
    n = 8192
    print(f'[case] gemm {n}^3 projection', flush=True)
    a, b = workloads.gemm_inputs(3, n)
    dev = autort.device()
    c = op(a.to(dev), b.to(dev)).cpu()
    g = torch.Generator().manual_seed(9)
    for _ in range(2):
        v = torch.randn(n, generator=g, dtype=torch.float64)
        want = a.double() @ (b.double() @ v)
        got = c.double() @ v
        # every element of C carries a relative rounding error of 2^-11; over a row of n random terms they add up to
        # about sqrt(n) * 2^-11 * |c| * |v| - three times that is the bound
        bound = 3 * (n ** 0.5) * 2.0 ** -11 * c.double().abs().mean() * v.abs().mean() * 1.3
        assert (got - want).abs().max() < bound, ((got - want).abs().max(), bound)
    # and the rows and columns are where they belong: two single-row / single-column spot checks in float64
    i, j = 1234, 4321
    assert abs(float(c[i, j]) - float(a[i].double() @ b[:, j].double())) < 1e-2 * max(1.0, abs(float(c[i, j])))
    assert abs(float(c[n - 1, 0]) - float(a[n - 1].double() @ b[:, 0].double())) < 1e-2 * max(1.0, abs(float(c[n - 1, 0])))
