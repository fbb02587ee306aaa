"""The worked programs of AntaresIR.md:108-256: the CPU oracle against an independent numpy statement of each
program (pins parser, typing and loop-nest emission), and the gfx950 lowering against the oracle."""
import numpy as np
import pytest

from ir_examples import EXAMPLES, make_inputs

NAMES = sorted(EXAMPLES)


def oracle_run(name, inputs):
    from antares_amd.ir import parse_program
    from oracle.cpu_backend import CpuModule
    ir, input_dict, extra, _ = EXAMPLES[name]
    mod = CpuModule(parse_program(ir, dict(input_dict), extra), fast_math=False)
    tensors = {k: np.array(v) for k, v in inputs.items()}       # copies: scatter programs write into their input
    return mod, mod(**tensors)


def reference(name, inputs):
    ir, input_dict, extra, ref = EXAMPLES[name]
    if name == 'scatter4d':
        data = inputs['data'].copy()
        for b in range(inputs['indices'].shape[0]):
            i = inputs['indices'][b]
            data[i[0], i[1], i[2], i[3], :] = inputs['updates'][b]
        return {'data': data}
    return ref(**inputs)


@pytest.mark.parametrize('name', NAMES)
def test_oracle_reproduces_the_documented_semantics(name, oracle_built):
    inputs = make_inputs(name)
    mod, got = oracle_run(name, inputs)
    want = reference(name, inputs)
    assert set(want) <= set(got), (sorted(want), sorted(got))
    for k, w in want.items():
        g = got[k]
        w = np.asarray(w)
        assert tuple(g.shape) == (tuple(w.shape) if w.shape else (1,)), (k, g.shape, w.shape)
        if g.dtype.kind in 'iu':
            assert np.array_equal(g.reshape(w.shape), w), k
        else:
            assert np.allclose(g.reshape(w.shape).astype(np.float64), w.astype(np.float64), rtol=2e-5, atol=2e-5), \
                (k, np.abs(g.reshape(w.shape) - w).max())


@pytest.mark.gpu
@pytest.mark.parametrize('name', NAMES)
def test_gfx950_lowering_matches_the_oracle(name, oracle_built):
    import torch
    import autort
    ir, input_dict, extra, _ = EXAMPLES[name]
    inputs = make_inputs(name)
    print(f'[case] {name}', flush=True)
    _, want = oracle_run(name, inputs)
    specs = [f"{k}={v['dtype']}[{', '.join(map(str, v['shape']))}]" for k, v in input_dict.items()]
    op = autort.export(ir=ir, inputs=specs, extra_outputs=extra, name='doc_example_' + name)
    dev = autort.device()
    args = [torch.from_numpy(np.array(inputs[k])).to(dev) for k in input_dict]
    out = op(*args)
    torch.cuda.synchronize()
    outs = out if isinstance(out, tuple) else (out,)
    got = dict(zip(op.graph.outputs, outs))
    for k, w in want.items():
        g = got[k].cpu().numpy()
        if g.dtype.kind in 'iu':
            assert np.array_equal(g.reshape(w.shape), w), k
        else:
            assert np.allclose(g.reshape(w.shape), w, rtol=2e-5, atol=2e-5), (k, np.abs(g.reshape(w.shape) - w).max())
