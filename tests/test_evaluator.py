"""The reference's own evaluator (graph_evaluator/run_graph.cpp, built unchanged into oracle/_ref/ by
oracle/Makefile) as a checker:

  * CPU: the oracle's emitted modules run under evaluator.c-mcpu, and its digests (run_graph.cpp:189-208)
    must equal what the oracle's own runtime computes from the same deterministic fill (run_graph.cpp:131-149);
  * GPU: the HIP modules written by antares_amd.lower.evaluator_emit run under evaluator.c-mi355x - the same
    evaluator compiled against include/c-mi355x/backend.hpp - and must give the digests of the CPU run.
"""
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EVAL_CPU = os.path.join(ROOT, 'oracle', '_ref', 'evaluator.c-mcpu')
EVAL_GPU = os.path.join(ROOT, 'oracle', '_ref', 'evaluator.c-mi355x')

PROGRAMS = {
    'sigmoid': ('sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))', ['data=float32[N:40960]']),
    'matmul': ('out[N, M] +=! a[N, K] * b[K, M]', ['a=float32[96, 64]', 'b=float32[64, 80]']),
    'rowmax_then_scale': ('mx[N] >=! x[N, C]; y[N, C] = x[N, C] / mx[N]', ['x=float32[33, 257]']),
    'int_mix': ('out[N] = (a[N] * 3 + b[N]) % 7', ['a=int32[N:5000]', 'b=int32[N:5000]']),
    'half_axpy': ('out[N] = a[N] * b[N] + a[N]', ['a=float16[N:12288]', 'b=float16[N:12288]']),
    'gather': ('out[N, C] = table[idx[N], C]', ['table=float32[71, 32]', 'idx=int32[50]']),
}


def run_evaluator(binary, source, tmp_path, tag):
    d = tmp_path / tag
    d.mkdir()
    (d / 'my_kernel.cc').write_text(source)
    r = subprocess.run([binary, str(d / 'my_kernel.cc')], cwd=d, capture_output=True, text=True, timeout=300,
                       env=dict(os.environ, CPU_THREADS='8'))
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    digests = [float(v) for v in re.findall(r'- K/\d+: (\S+)', r.stdout)]
    tpr = re.findall(r'- TPR: (\S+)', r.stdout)
    assert digests and tpr, r.stdout[-2000:]
    return digests, float(tpr[-1])


def oracle_digests(name):
    """The same program through the oracle's own runtime with the evaluator's fill."""
    from antares_amd.ir import parse_program
    from oracle import cpu_backend
    ir, inputs = PROGRAMS[name]
    g = parse_program(ir, inputs)
    mod = cpu_backend.CpuModule(g)
    env = mod.graph.bind_dims({})
    tensors = {}
    for i, n in enumerate(mod.graph.abi_inputs):
        t = mod.graph.tensors[n]
        arr = np.zeros(mod.graph.shape_of(n, env), dtype=cpu_backend.NP_DTYPE[t.dtype])
        tensors[n] = cpu_backend.fill(arr, t.dtype, i)
    outs = mod(**tensors)
    return mod, [cpu_backend.digest(outs[n], mod.graph.tensors[n].dtype) for n in mod.graph.abi_outputs]


@pytest.mark.skipif(not os.path.isfile(EVAL_CPU), reason='oracle/_ref/evaluator.c-mcpu is not built (needs the reference tree)')
@pytest.mark.parametrize('name', sorted(PROGRAMS))
def test_oracle_modules_run_under_the_reference_evaluator(name, tmp_path, oracle_built):
    mod, mine = oracle_digests(name)
    theirs, _ = run_evaluator(EVAL_CPU, mod.source, tmp_path, 'cpu')
    assert len(theirs) == len(mine)
    for a, b in zip(theirs, mine):
        assert a == pytest.approx(b, rel=1e-9, abs=1e-9), (name, theirs, mine)


def hip_module(name):
    from antares_amd.ir import fuse_elementwise, parse_program
    from antares_amd.lower.evaluator_emit import emit_evaluator_module
    ir, inputs = PROGRAMS[name]
    return emit_evaluator_module(fuse_elementwise(parse_program(ir, inputs)))


@pytest.mark.parametrize('name', sorted(PROGRAMS))
def test_hip_module_has_the_container_layout_and_compiles(name):
    """Layout the evaluator parses (execute_module.hpp:277-318): numeric shapes, VAMAP values, one LOCAL line and
    thread extents per kernel; and the text compiles for gfx950 as it stands."""
    from antares_amd.runtime import capi
    src = hip_module(name)
    head = src.split('\n')
    assert head[0].startswith('// GLOBALS: ') and ' -> ' in head[0]
    assert not re.search(r'\[[^\]]*[A-Za-z_][^\]]*\]', head[0]), head[0]           # every extent is a number
    assert head[1] == '// BACKEND: c-mi355x (gfx950)'
    slices = src.split('-------\n')[1:]
    assert slices
    for s in slices:
        fname = re.search(r'// LOCAL: (\S+) -- ', s).group(1)
        assert re.search(r'// \[thread_extent\] blockIdx\.x = [1-9]\d*\n', s) and '// [thread_extent] threadIdx.x = ' in s
        assert f' void {fname}(' in s
    if 'N:' in PROGRAMS[name][1][0]:
        assert re.search(r'// VAMAP: N:\d+\n', src)
    assert len(capi.compile_hip(src)) > 1000


def test_backend_shim_compiles_against_the_c_abi(tmp_path):
    """include/c-mi355x/backend.hpp stands on the C ABI alone: no HIP headers, every ab:: function the evaluator calls."""
    tu = tmp_path / 'tu.cpp'
    tu.write_text('#include "backend.hpp"\n'
                  'int main() { void* fns[] = {(void*)&ab::init, (void*)&ab::finalize, (void*)&ab::alloc, (void*)&ab::release,\n'
                  '  (void*)&ab::moduleCompile, (void*)&ab::moduleLoad, (void*)&ab::moduleGetFunction, (void*)&ab::launchKernel,\n'
                  '  (void*)&ab::memcpyHtoD, (void*)&ab::memcpyDtoH, (void*)&ab::synchronize, (void*)&ab::recordTime,\n'
                  '  (void*)&ab::convertToElapsedTime}; return fns[0] == nullptr; }\n')
    r = subprocess.run(['g++', '-std=c++17', '-fsyntax-only', '-Wall', '-I', os.path.join(ROOT, 'include', 'c-mi355x'),
                        '-I', os.path.join(ROOT, 'include'), str(tu)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert 'hip' not in open(os.path.join(ROOT, 'include', 'c-mi355x', 'backend.hpp')).read().split('#pragma once')[1].split('namespace ab')[0]


@pytest.mark.gpu
@pytest.mark.skipif(not (os.path.isfile(EVAL_GPU) and os.path.isfile(EVAL_CPU)), reason='oracle/_ref evaluators are not built')
@pytest.mark.parametrize('name', sorted(PROGRAMS))
def test_reference_evaluator_drives_the_gfx950_kernels(name, tmp_path, oracle_built):
    mod, _ = oracle_digests(name)
    cpu, _ = run_evaluator(EVAL_CPU, mod.source, tmp_path, 'cpu')
    gpu, tpr = run_evaluator(EVAL_GPU, hip_module(name), tmp_path, 'gpu')
    print(f'{name}: digests cpu={cpu} gpu={gpu} TPR={tpr:g}s', flush=True)
    assert len(gpu) == len(cpu)
    exact = name in ('int_mix', 'gather')
    for a, b in zip(gpu, cpu):
        assert a == (b if exact else pytest.approx(b, rel=2e-3 if name == 'half_axpy' else 1e-5)), (name, gpu, cpu)
    assert 0 < tpr < 1
