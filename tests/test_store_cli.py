"""Persisted operators, the command line and the legacy CustomOp surface (CPU parts: no launch)."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SIGMOID = 'sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))'


@pytest.fixture()
def ops_dir(tmp_path, monkeypatch):
    monkeypatch.setenv('AUTORT_OPS_DIR', str(tmp_path / 'ops'))
    monkeypatch.setenv('AUTORT_CACHE_DIR', str(tmp_path / 'cache'))
    return tmp_path / 'ops'


def test_export_writes_a_module_file_and_a_new_session_finds_it(ops_dir):
    import autort
    from antares_amd.autort import store
    op = autort.export(ir=SIGMOID, inputs=['data=float32[N:4096000]'], config='tune:5')
    path = store.module_path('sigmoid_f32')
    assert os.path.isfile(path)
    text = open(path).read()
    assert text.startswith('// MODULE: ') and '// GLOBALS: ' in text        # record first, kernel container after it
    record = store.load('sigmoid_f32')
    assert record['ir'] == SIGMOID and record['inputs'] == ['data=float32[N:4096000]'] and record['config'] == 'tune:5'
    # a later session: nothing registered in the process, the name resolves from the file
    fresh = type(autort.ops)()
    again = fresh.sigmoid_f32
    assert again is not op and again.ir == SIGMOID and again.declared == ['data']
    assert 'sigmoid_f32' in dir(fresh)
    with pytest.raises(AttributeError):
        fresh.no_such_operator_anywhere


def test_module_name_is_checked(ops_dir):
    from antares_amd.autort import store
    for bad in ('', '../x', 'a/b', '.hidden'):
        with pytest.raises(ValueError):
            store.module_path(bad)
    assert store.load('../x') is None


def test_command_line_creates_the_operator(ops_dir):
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, '-m', 'autort', '--ir', SIGMOID, '-i', 'data=float32[N:4096000]', '-c', 'tune:5'],
                       cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert 'Module file for operator `sigmoid_f32` has been exported to' in r.stdout
    assert os.path.isfile(ops_dir / 'sigmoid_f32.mod')
    bad = subprocess.run([sys.executable, '-m', 'autort', '--ir', 'out[N] = nothing[N', '-i', 'data=float32[N]'],
                         cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    assert bad.returncode == 1 and 'autort:' in bad.stderr


def test_custom_op_emit_reports_outputs(ops_dir):
    from antares_amd.autort.custom_op import CustomOp
    a = torch.zeros(8, 16)
    with pytest.raises(RuntimeError):
        CustomOp(ir='out[N, M] = a[N, M] + b[N, M]', input_orders={'a': a, 'b': a})      # device=None means CPU: refused
    op = CustomOp(ir='mid[N, M] = a[N, M] * 2; out[N] +=! mid[N, M] * b[N, M]',
                  input_orders={'a': a, 'b': ('b', torch.float32, [8, 16])}, extra_outputs=['mid'],
                  device=torch.device('cuda')).tune(step=0).emit()
    assert op.output_names == ['mid', 'out'] or op.output_names == ['out', 'mid']
    infos = {n: (dt, shp) for n, dt, shp in op.output_infos}
    assert infos['out'] == (torch.float32, [8]) and infos['mid'] == (torch.float32, [8, 16])
    assert op.kernel_sources.startswith('// GLOBALS: ')
    assert isinstance(op.custom_key, int)
    with pytest.raises(Exception, match='Deprecated Usage'):
        op.to('cuda')


@pytest.mark.gpu
def test_persisted_operator_runs_in_a_fresh_process(ops_dir):
    """README.md:75-86: create on the command line, use from a later session."""
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, '-m', 'autort', '--ir', SIGMOID, '-i', 'data=float32[N:4096000]', '-c', 'tune:5'],
                       cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    code = ('import torch, autort\n'
            'data = torch.arange(0, 10, dtype=torch.float32, device=autort.device())\n'
            'print(["%.4f" % v for v in autort.ops.sigmoid_f32(data).tolist()])\n')
    r = subprocess.run([sys.executable, '-c', code], cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    want = ['0.5000', '0.7311', '0.8808', '0.9526', '0.9820', '0.9933', '0.9975', '0.9991', '0.9997', '0.9999']   # README.md:68
    assert str(want) in r.stdout


@pytest.mark.gpu
def test_custom_op_forward_matches_torch(ops_dir):
    from antares_amd.autort.custom_op import CustomOp
    import autort
    dev = autort.device()
    g = torch.Generator().manual_seed(3)
    a = torch.randn(64, 48, generator=g).to(dev)
    b = torch.randn(64, 48, generator=g).to(dev)
    op = CustomOp(ir='mid[N, M] = a[N, M] * 2; out[N] +=! mid[N, M] * b[N, M]', input_orders={'a': a, 'b': b},
                  extra_outputs=['mid'], device=dev).tune(step=0).emit()
    outs = dict(zip(op.output_names, op(a, b)))
    assert torch.allclose(outs['mid'], a * 2)
    assert torch.allclose(outs['out'], (a * 2 * b).sum(1), rtol=1e-5, atol=1e-5)
    single = CustomOp(ir='out[N, M] = a[N, M] + b[N, M]', input_orders={'a': a, 'b': b}, device=dev).emit()
    assert torch.equal(single(a, b), a + b)


@pytest.mark.gpu
def test_tune_config_times_candidates_and_keeps_the_winner(ops_dir):
    """config="tune:N" (README.md:66): the first call searches launch configurations, the choice is stored in the
    module file and reused by later sessions; results are the same before and after."""
    import autort
    from antares_amd.autort import store
    dev = autort.device()
    x = (torch.rand(1_000_000, generator=torch.Generator().manual_seed(0)) * 16 - 8).to(dev)
    plain = autort.export(ir=SIGMOID, inputs=['data=float32[N:4096000]'], name='sigmoid_plain')
    tuned = autort.export(ir=SIGMOID, inputs=['data=float32[N:4096000]'], config='tune:6', name='sigmoid_tuned')
    want = plain(x)
    got = tuned(x)
    assert torch.equal(got, want)
    from oracle import hot_ops                                   # the checker: the tuned operator against the oracle
    assert np.allclose(got.cpu().numpy(), hot_ops.sigmoid_f32(x.cpu().numpy()), rtol=1e-5, atol=1e-5)
    assert len(tuned.tuned) == 1
    (key, choice), = tuned.tuned.items()
    assert key.startswith('autort_sigmoid_tuned_k0|1000000|') and choice['variant'] in ('vec', 'scalar') and choice['grid'] >= 1
    assert store.load('sigmoid_tuned')['tuned'] == tuned.tuned
    # a later session starts from the stored choice and does not search again
    again = type(autort.ops)().sigmoid_tuned
    assert again.tuned == tuned.tuned
    assert torch.equal(again(x), want) and again.tuned == tuned.tuned
    # a program that accumulates into an in-out tensor is timed on scratch copies, not on the live tensor
    acc = autort.export(ir='hist[data[N] % 16] +=. one[0]', inputs=['data=int32[N]', 'one=int32[1]', 'hist=int32[16]'],
                        config='tune:4', name='hist_tuned')
    data = torch.arange(4096, dtype=torch.int32, device=dev)
    hist = torch.zeros(16, dtype=torch.int32, device=dev)
    acc(data, torch.ones(1, dtype=torch.int32, device=dev), hist)
    assert hist.tolist() == [256] * 16


@pytest.mark.gpu
def test_tune_config_searches_the_hand_kernels_launch_parameters(ops_dir):
    """config="tune:N" on a program that runs on a hand-written kernel searches that kernel's launch parameters (rows
    per lane x wavefronts per block of the int4 GEMV, K-splits x rows per block of the int4 GEMM) for the shape of the call, keeps the winner in the module
    file, and the tuned operator - like every value of the parameter - matches the oracle."""
    import subprocess
    from ctypes import c_void_p
    import autort
    from antares_amd import workloads
    from antares_amd.autort import patterns, store
    from antares_amd.runtime import capi
    from oracle import hot_ops
    subprocess.check_call(['make', '-s', '-C', os.path.join(ROOT, 'oracle'), 'libref_hotops.so'])
    dev = autort.device()
    f = autort.export(ir=patterns.W4A16_IR, inputs=patterns.W4A16_INPUTS, name='w4a16_tuned', config='tune:8')
    lib = capi.lib()
    for M, K, N, key, entry, values in [
            (1, 4096, 4096, 'gemv_w4a16.rows_x16_plus_waves|1,4096,4096', lib.art_gemv_w4a16_knobs, ((0, 0), (8, 4), (4, 4), (8, 8), (4, 8), (0, 8), (4, 0))),
            (1, 11008, 528, 'gemv_w4a16.rows_x16_plus_waves|1,11008,528', lib.art_gemv_w4a16_knobs, ((8, 4), (4, 4), (8, 8), (4, 8))),
            (2, 1024, 1040, 'gemv_w4a16.rows_x16_plus_waves|2,1024,1040', lib.art_gemv_w4a16_knobs, ((8, 4), (4, 4))),
            (64, 4096, 4096, 'gemm_w4a16.k_splits|64,4096,4096', lib.art_gemm_w4a16_tuned, (0, 1, 3, 8, 32, 255, 256 + 2, 256 + 8, 256, 512 + 3))]:
        print(f'[case] tuned int4 product M={M} K={K} N={N}', flush=True)
        p = workloads.w4_problem(M + K + N, M, K, N)
        want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy()).astype(np.float32)
        d = [p[k].to(dev) for k in ('x', 'qweight', 'scales', 'qzeros')]
        if (M, K, N) == (1, 4096, 4096):
            d1, want1 = d, want
        got = f(*d)
        assert np.allclose(got.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)
        choice = f.tuned[key]
        assert choice['us'] > 0 and (choice['value'] in (8 * 16 + 4, 4 * 16 + 4, 8 * 16 + 8, 4 * 16 + 8) if 'gemv' in key
                                    else (choice['value'] & 255) <= K // 128 and choice['value'] >> 8 in (0, 1, 2))
        assert store.load('w4a16_tuned')['tuned'][key] == choice
        assert torch.equal(f(*d), got)                              # the stored choice is used again, no new search
        for v in values:                                            # every value of the parameter gives the oracle's result
            y = torch.full((M, N), float('nan'), dtype=torch.float16, device=dev)
            knobs = v if isinstance(v, tuple) else (v,)
            capi.check(entry(c_void_p(d[0].data_ptr()), c_void_p(d[1].data_ptr()), c_void_p(d[2].data_ptr()), c_void_p(d[3].data_ptr()),
                             c_void_p(y.data_ptr()), M, K, N, *knobs, None))
            torch.cuda.synchronize()
            assert np.allclose(y.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2), v
    # a later session finds the choices
    again = type(autort.ops)().w4a16_tuned
    assert again.tuned == f.tuned and len(again.tuned) == 4
    # a value outside the parameter's range is refused
    assert lib.art_gemv_w4a16_tuned(None, None, None, None, None, 1, 4096, 4096, 5, None) != 0
    assert b'k_per_block' in lib.art_last_error()
    for k_per_block in (256, 512, 1024):                            # the older single knob still names three of the four combinations
        y = torch.full((1, 4096), float('nan'), dtype=torch.float16, device=dev)
        capi.check(lib.art_gemv_w4a16_tuned(c_void_p(d1[0].data_ptr()), c_void_p(d1[1].data_ptr()), c_void_p(d1[2].data_ptr()),
                                            c_void_p(d1[3].data_ptr()), c_void_p(y.data_ptr()), 1, 4096, 4096, k_per_block, None))
        assert np.allclose(y.float().cpu().numpy(), want1, rtol=1e-2, atol=1e-2), k_per_block
    assert lib.art_gemv_w4a16_knobs(None, None, None, None, None, 1, 4096, 4096, 5, 4, None) != 0 and b'rows_per_lane' in lib.art_last_error()
    assert lib.art_gemv_w4a16_knobs(None, None, None, None, None, 2, 4096, 4096, 8, 8, None) != 0 and b'M = 1' in lib.art_last_error()
    assert lib.art_gemm_w4a16_tuned(None, None, None, None, None, 64, 4096, 4096, 0x300, None) != 0
    assert b'rows-per-block' in lib.art_last_error()


@pytest.mark.gpu
def test_partition_tuning_keeps_results_bit_exact(ops_dir):
    """The fused partition's launch parameter (cap on the number of blocks): every value gives the oracle's bits, a
    tuning run keeps the fastest for that length and later sessions read it back."""
    import subprocess
    from ctypes import c_void_p
    import autort
    from antares_amd import workloads
    from antares_amd.autort.builtin_ops import PartitionEvenFirst
    from antares_amd.runtime import capi
    from oracle import hot_ops
    subprocess.check_call(['make', '-s', '-C', os.path.join(ROOT, 'oracle'), 'libref_hotops.so'])
    dev = autort.device()
    n = 3_000_017
    x = workloads.partition_input(5, n)
    want = hot_ops.sort_even_first_i32(x.numpy())
    xd = x.to(dev)
    capi.init(0)
    for cap in (0, 64, 100, 1024, 16384):
        print(f'[case] partition with at most {cap} blocks', flush=True)
        out = torch.zeros_like(xd)
        capi.check(capi.lib().art_partition_even_first_i32_tuned(c_void_p(xd.data_ptr()), c_void_p(out.data_ptr()), n, cap, None))
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want), cap
    assert capi.lib().art_partition_even_first_i32_tuned(c_void_p(xd.data_ptr()), c_void_p(out.data_ptr()), n, 63, None) != 0
    op = PartitionEvenFirst()
    rec = op.tune(xd, trials=4)
    assert rec['value'] in PartitionEvenFirst.BLOCK_CAPS[:4] and rec['us'] > 0
    assert np.array_equal(op(xd).cpu().numpy(), want)
    fresh = PartitionEvenFirst()
    assert np.array_equal(fresh(xd).cpu().numpy(), want) and fresh.tuned[str(n)] == rec


@pytest.mark.gpu
def test_tune_config_searches_the_fp16_gemm_block_shape(ops_dir):
    """config="tune:N" on the fp16 matrix product times both block shapes of `art_gemm_f16_tuned` (256 or 512
    threads per 256 x 256 tile) for the shape of the call and keeps the faster one; the result is the fp64 product
    either way."""
    import autort
    from antares_amd.autort import patterns, store
    dev = autort.device()
    f = autort.export(ir=patterns.GEMM_F16_IR, inputs=patterns.GEMM_F16_INPUTS, name='gemm_f16_tuned', config='tune:2')
    g = torch.Generator().manual_seed(9)
    a = (torch.randn(1024, 512, generator=g) * 0.05).half()
    b = (torch.randn(512, 768, generator=g) * 0.05).half()
    got = f(a.to(dev), b.to(dev))
    want = (a.double() @ b.double()).float()
    assert torch.allclose(got.float().cpu(), want, rtol=1e-2, atol=1e-2)
    choice = f.tuned['gemm_f16.threads|1024,512,768']
    assert choice['value'] in (256, 512) and choice['us'] > 0
    assert store.load('gemm_f16_tuned')['tuned']['gemm_f16.threads|1024,512,768'] == choice
    assert torch.equal(f(a.to(dev), b.to(dev)), got)
