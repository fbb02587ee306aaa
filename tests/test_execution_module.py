"""`inject` / `forward` (the reference's pybind pair, frameworks/pytorch/main_ops.cc:17-54) over kernel containers
in the layout of antares/antares_compiler.py:179-248."""
import numpy as np
import pytest
import torch

from antares_amd.autort.execution_module import ExecutionModule, forward, inject
from antares_amd.ir import fuse_elementwise, parse_program
from antares_amd.lower.evaluator_emit import emit_evaluator_module

PROGRAMS = {
    'elementwise': ('output0[N] = input0[N] + input1[N]', {'input0': ('float32', [5000]), 'input1': ('float32', [5000])}),
    'softmax': ('temp0[N] >=! input0[N, C]; temp1[N] +=! (input0[N, C] - temp0[N]).call(`exp`); '
                'output0[N, C] = (input0[N, C] - temp0[N]).call(`exp`) / temp1[N]', {'input0': ('float32', [8, 200])}),
    'matmul': ('output0[N, M] +=! input0[N, K] * input1[K, M]', {'input0': ('float32', [48, 40]), 'input1': ('float32', [40, 56])}),
    'gather_i32': ('output0[N, F] = input0[input1[N, F]]', {'input0': ('int32', [77]), 'input1': ('int32', [4, 16])}),
}


def container(name):
    program, inputs = PROGRAMS[name]
    graph = fuse_elementwise(parse_program(program, {k: {'dtype': d, 'shape': s} for k, (d, s) in inputs.items()}, []))
    return graph, emit_evaluator_module(graph)


def test_container_is_parsed_like_the_reference_does():
    graph, text = container('softmax')
    m = ExecutionModule(text)
    assert [p[0] for p in m.global_inputs] == ['input0'] and [p[0] for p in m.global_outputs] == ['output0']
    assert m.backend == 'c-mi355x'
    assert [k['out'] for k in m.kernels] == [['temp0'], ['temp1'], ['output0']]
    assert all(k['threads']['threadIdx.x'] == 256 and k['threads']['blockIdx.x'] >= 1 for k in m.kernels)
    assert m.local_tensors['temp1'] == ('float32', [8])
    assert all(k['dynamic'] is None for k in m.kernels)
    with pytest.raises(ValueError):
        ExecutionModule('// no globals here\n')


DYNAMIC_GRID = '''// GLOBALS: a:float32[1000] -> b:float32[1000]
// BACKEND: c-mi355x (default)
// VAMAP: N:%d
// ---------------------------------------------------------------------------
// LOCAL: scale_k -- a:float32[1000] -> b:float32[1000]

extern "C" __global__ __launch_bounds__(128) void scale_k(float* __restrict__ a, float* __restrict__ b, int N) {
  // [thread_extent] threadIdx.x = 128
  // [thread_extent] $ = 2
  // [thread_extent] $$ = 1
  // [thread_extent] $0 = 128
  const int i = blockIdx.x * 128 + threadIdx.x;
  if (i < N) b[i] = a[i] * 3.0f + (float)gridDim.x;
}
'''


def test_grid_sized_at_launch_is_parsed():
    """`$` keys (backends/c-rocm/include/backend.hpp:184-194): first integer argument, constant factor, per-argument block sizes."""
    m = ExecutionModule(DYNAMIC_GRID % 1000)
    assert m.dim_values == [1000] and m.kernels[0]['dynamic'] == (2, 1, [128])
    assert m.kernels[0]['threads']['threadIdx.x'] == 128


@pytest.mark.gpu
@pytest.mark.parametrize('n', [1000, 129, 1, 0])
def test_grid_sized_at_launch_runs(n):
    """gridDim.x = $$ * ceil(N / $0) is worked out from the integer argument at launch; 0 blocks: nothing is launched."""
    import autort
    print(f'[case] run-time sized grid N={n}', flush=True)
    dev = autort.device()
    a = torch.arange(1000, dtype=torch.float32, device=dev)
    b = torch.full((1000,), -1.0, device=dev)
    ExecutionModule(DYNAMIC_GRID % n).compute([a, b])
    want = torch.full((1000,), -1.0)
    want[:n] = torch.arange(n, dtype=torch.float32) * 3 + (n + 127) // 128
    assert torch.equal(b.cpu(), want)
    with pytest.raises(ValueError):
        ExecutionModule(DYNAMIC_GRID.replace('$ = 2', '$ = 1') % n).compute([a, b])


def test_keys_count_up_and_unknown_keys_fail():
    a, b = inject(container('elementwise')[1]), inject(container('matmul')[1])
    assert b == a + 1
    with pytest.raises(KeyError):
        forward(10 ** 6, [torch.zeros(1)])


@pytest.mark.gpu
@pytest.mark.parametrize('name', sorted(PROGRAMS))
def test_forward_runs_the_container(name, oracle_built):
    import autort
    from oracle.cpu_backend import CpuModule
    print(f'[case] inject/forward {name}', flush=True)
    dev = autort.device()
    graph, text = container(name)
    g = torch.Generator().manual_seed(len(name))
    inputs = {}
    for n, (dt, shape) in PROGRAMS[name][1].items():
        if dt == 'int32':
            inputs[n] = torch.randint(0, 77, shape, generator=g, dtype=torch.int32)
        else:
            inputs[n] = torch.randn(shape, generator=g)
    want = CpuModule(parse_program(PROGRAMS[name][0], {k: {'dtype': d, 'shape': s} for k, (d, s) in PROGRAMS[name][1].items()}),
                     fast_math=False)(**{k: v.numpy() for k, v in inputs.items()})
    key = inject(text)
    out_name = graph.abi_outputs[0]
    info = graph.tensors[out_name]
    out = torch.empty([int(d) for d in info.shape], dtype=torch.int32 if info.dtype == 'int32' else torch.float32, device=dev)
    forward(key, [inputs[n].to(dev) for n in graph.abi_inputs] + [out])
    forward(key, [inputs[n].to(dev) for n in graph.abi_inputs] + [out])          # the module is kept per (key, device)
    got = out.cpu().numpy()
    if info.dtype == 'int32':
        assert np.array_equal(got, want[out_name])
    else:
        assert np.allclose(got, want[out_name], rtol=1e-5, atol=1e-5)
    with pytest.raises(ValueError):
        forward(key, [out])
