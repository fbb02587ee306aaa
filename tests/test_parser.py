"""Front-end tests: the einstein_v2 grammar, typing rules and argument order
(reference: lang/einstein_v2.py, lang/generic.py:39-54, AntaresIR.md), plus the
AutoRT dialect used by the samples."""
import pytest

from antares_amd.ir import IRSyntaxError, fuse_elementwise, parse_program, to_ir


def one(ir, inputs, **kw):
    g = parse_program(ir, inputs, **kw)
    return g, g.statements[-1]


F32 = lambda *shape: {'dtype': 'float32', 'shape': list(shape)}   # noqa: E731


# ---- shapes and axis inference, the worked examples of AntaresIR.md:108-256
@pytest.mark.parametrize('ir,inputs,shape,reduce_axes', [
    ('output0[N, F, HO, WO] = input0[N] where F in 32, HO in 2, WO in 2', {'input0': F32(16)}, [16, 32, 2, 2], []),
    ('output0[N, M] +=! input0[N, K] * input1[K, M]', {'input0': F32(1024, 512), 'input1': F32(512, 512)}, [1024, 512], ['K']),
    ('output0[B, N, M] +=! input0[B, N, K] * input1[B, K, M]', {'input0': F32(3, 1024, 512), 'input1': F32(3, 512, 512)}, [3, 1024, 512], ['K']),
    ('output0[N, C, H, W] = input0[N, H, W, C]', {'input0': F32(32, 229, 229, 3)}, [32, 3, 229, 229], []),
    ('output0[A, B, C] = input0[A, B, C / 64, C % 64] where C in 128', {'input0': F32(3, 3, 2, 64)}, [3, 3, 128], []),
    ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[F, C, KH, KW] where HO in 30, WO in 30',
     {'input0': F32(16, 64, 32, 32), 'input1': F32(256, 64, 3, 3)}, [16, 256, 30, 30], ['C', 'KH', 'KW']),
    ('output0[N, C, HO, WO] >=! input0[N, C, HO * 2 + KH, WO * 2 + KW] where HO in 6, WO in 6, KW in 2, KH in 2',
     {'input0': F32(32, 3, 12, 12)}, [32, 3, 6, 6], ['KW', 'KH']),
    ('output0[N, F] = input0[N, F, 2]', {'input0': F32(1, 16, 32)}, [1, 16], []),
    ('output0[F, C] = input0[input1[F], C]', {'input0': F32(30528, 1024), 'input1': {'dtype': 'int32', 'shape': [3072]}}, [3072, 1024], []),
    ('output0[] = input0[] + input1[]', {'input0': F32(), 'input1': F32()}, [1], []),
])
def test_shapes(ir, inputs, shape, reduce_axes):
    g, st = one(ir, inputs)
    assert st.out_shape == shape
    assert [a for a, _ in st.reduce_axes] == reduce_axes
    assert g.tensors[st.output].dtype == 'float32'


def test_undetermined_axis_is_an_error():
    with pytest.raises(IRSyntaxError, match='undetermined'):
        parse_program('output0[N] = N.cast(`float32`)', {})
    g, st = one('output0[N] = N.cast(`float32`) where N in 1024', {})
    assert st.out_shape == [1024] and st.out_dtype == 'float32' and g.abi_inputs == []


# ---- typing rules
def test_comparison_is_int8_and_gt_is_swapped_lt():
    _, st = one('output0[N] = input0[N] > 0.0', {'input0': F32(8)})
    assert st.out_dtype == 'int8'
    assert to_ir(st.root) == '(const(0.0) < input0[N])'


def test_integer_division_truncates_and_float_division_does_not():
    _, st = one('output0[N] = input0[N] / 3', {'input0': {'dtype': 'int32', 'shape': [8]}})
    assert st.root.name == '//' and st.out_dtype == 'int32'
    _, st = one('output0[N] = input0[N] / 3', {'input0': F32(8)})
    assert st.root.name == '/' and st.out_dtype == 'float32'


def test_promotion_and_algebraic_simplifications():
    _, st = one('output0[N] = input0[N] * 1 + 0', {'input0': {'dtype': 'float16', 'shape': [8]}})
    assert to_ir(st.root) == 'input0[N]' and st.out_dtype == 'float16'
    _, st = one('output0[N] = input0[N] + input1[N]', {'input0': {'dtype': 'float16', 'shape': [8]}, 'input1': {'dtype': 'int32', 'shape': [8]}})
    assert st.out_dtype == 'float16'
    _, st = one('output0[N] = input0[N % 1] where N in 4', {'input0': F32(4)})
    assert to_ir(st.root) == 'input0[const(0)]'
    # an axis known to be smaller than the divisor folds to 0; smaller than the modulus stays as it is
    _, st = one('output0[N, M] = input0[N / 8, M % 8] where N in 8, M in 8', {'input0': F32(1, 8)})
    assert to_ir(st.root) == 'input0[const(0), M]'


def test_call_rewrites():
    _, st = one('output0[N] = input0[N].call(`sigmoid`)', {'input0': F32(8)})
    assert 'exp' in to_ir(st.root) and st.root.name == '/'
    _, st = one('output0[N] = input0[N].call(`floor`)', {'input0': F32(8)})
    assert st.out_dtype == 'int32'
    _, st = one('output0[N] = input0[N].call(`exp`)', {'input0': {'dtype': 'float16', 'shape': [8]}})
    assert st.root.name == 'fp16_exp'
    _, st = one('output0[N] = input0[N].call(`tanh`)', {'input0': {'dtype': 'float16', 'shape': [8]}})
    assert st.out_dtype == 'float16' and st.root.kind == 'cast' and st.root.args[0].dtype == 'float32'


def test_when_requires_matching_dtypes_and_integer_conditions():
    one('output0[N] = input0[N].when([input0[N] > 0.0], 0.0)', {'input0': F32(8)})
    with pytest.raises(TypeError):
        one('output0[N] = input0[N].when([input0[N] > 0.0], 0)', {'input0': F32(8)})
    with pytest.raises(TypeError):
        one('output0[N] = input0[N].when([input0[N]], 0.0)', {'input0': F32(8)})


def test_reduce_operators():
    for sym in ['+', '>', '<', '*', '|', '&']:
        dt = 'int8' if sym in '|&' else 'float32'
        _, st = one(f'output0[N] {sym}=! input0[N, C]', {'input0': {'dtype': dt, 'shape': [4, 6]}})
        assert st.reduce == sym and st.out_shape == [4]
    with pytest.raises(IRSyntaxError):
        parse_program('output0[N] = input0[N, C]', {'input0': F32(4, 6)})


# ---- graph level: outputs, argument order, in-out tensors, fusion
def test_argument_order_is_sorted_by_name():
    g = parse_program('output0[N] = b[N] + a[N]; output1[N] = a[N] * 2; output2[N] = b[N] + output1[N]',
                      {'b': F32(8), 'a': F32(8)}, extra_outputs=['output2', 'output0', 'output1'])
    assert g.abi_inputs == ['a', 'b'] and g.abi_outputs == ['output0', 'output1', 'output2']


def test_unused_inputs_are_dropped_and_last_statement_is_the_output():
    g = parse_program('t[N] = a[N] + 1; output0[N] = t[N] * 2', {'a': F32(8), 'unused': F32(3)})
    assert g.abi_inputs == ['a'] and g.outputs == ['output0']
    f = fuse_elementwise(g)
    assert len(f.statements) == 1 and 't' not in f.tensors


def test_scatter_makes_the_target_an_output():
    g = parse_program('data[indices[B, 0], indices[B, 1], M] =. updates[B, M]',
                      {'data': F32(32, 32, 8), 'indices': {'dtype': 'int32', 'shape': [2, 2]}, 'updates': F32(2, 8)})
    assert g.abi_inputs == ['indices', 'updates'] and g.abi_outputs == ['data'] and g.inout == ['data']
    st = g.statements[0]
    assert st.scatter and st.set_op == 'set' and sorted(a for a, _ in st.data_axes) == ['B', 'M']
    assert parse_program('data[i[B]] +=. u[B]', {'data': F32(4), 'i': {'dtype': 'int32', 'shape': [9]}, 'u': F32(9)}).statements[0].set_op == 'add'


def test_fusion_keeps_reduce_results_and_inlines_elementwise_producers():
    g = parse_program('temp0[K, N] = input0[N, K] + 100; output0[N, M] +=! temp0[K, N] * input1[K, M] where K in 10',
                      {'input0': F32(1024, 512), 'input1': F32(512, 512)})
    f = fuse_elementwise(g)
    assert len(f.statements) == 1 and 'input0[N, K]' in f.to_ir()
    g = parse_program('temp0[N] >=! input0[N, C]; temp1[N] +=! (input0[N, C] - temp0[N]).call(`exp`); '
                      'output0[N, C] = (input0[N, C] - temp0[N]).call(`exp`) / temp1[N]', {'input0': F32(32, 1024)})
    assert [s.output for s in fuse_elementwise(g).statements] == ['temp0', 'temp1', 'output0']


# ---- the AutoRT dialect (call sites: README.md:66, samples/01_sort_even_first.py:10-14, samples/05_llama2_7b_int4.py:135-139)
def test_named_dimensions_and_strs():
    g, st = one('sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))', ['data=float32[N:4096000]'])
    assert g.dims == {'N': 4096000} and st.out_shape == ['N'] and g.outputs == ['sigmoid_f32']
    assert g.bind_dims({'data': (10,)}) == {'N': 10}
    with pytest.raises(ValueError):
        g.bind_dims({'data': (2, 5)})


def test_sort_sample_programs():
    g, st = one('space[data[N] % 2, N] = 1', ['data=int32[N]', 'space=int32[2, N]'])
    assert st.scatter and g.abi_inputs == ['data'] and g.abi_outputs == ['space'] and g.dims == {'N': None}
    g, st = one('output[ids[N] - 1] = (val[N % val.size(0)]).when(ids[N] > 0)', ['ids=int32[N]', 'val=int32[M]', 'output=int32[M]'])
    assert st.scatter and st.root.kind == 'when' and len(st.root.args) == 1
    assert g.abi_inputs == ['ids', 'val'] and g.abi_outputs == ['output']
    assert g.bind_dims({'ids': (20,), 'val': (10,), 'output': (10,)}) == {'N': 20, 'M': 10}
    with pytest.raises(ValueError, match='bound to both'):
        g.bind_dims({'ids': (20,), 'val': (10,), 'output': (11,)})


def test_int4_sample_program_fuses_to_one_statement():
    ir = """
      input1[S, N] = (qweight[S / 8, N] >> (S % 8 * 4)).call(strs.bitwise_and, 15) * input0[S].like(1)
      w[S, N] = scales[S / 128, N] * (input1[S, N] - 8)
      my_result[N] +=! input0[S] * w[S, N].to(input0.dtype())
    """
    g = parse_program(ir, ['input0=float32[S:4096]', 'qweight=int32[L:512, N:12288]', 'scales=float16[K:32, N:12288]'])
    assert len(g.statements) == 3
    assert g.tensors['input1'].dtype == 'float32'          # int32 * float32 const 1 -> cast to float32
    f = fuse_elementwise(g)
    assert len(f.statements) == 1 and f.statements[0].reduce == '+' and f.statements[0].out_dtype == 'float32'
    assert f.abi_inputs == ['input0', 'qweight', 'scales'] and f.abi_outputs == ['my_result']
    assert f.dim_names == ['K', 'L', 'N', 'S']
    # names do not matter for recognising the pattern
    g2 = parse_program(ir.replace('input0', 'xx').replace('my_result', 'yy').replace('S', 'R'),
                       ['xx=float32[R:4096]', 'qweight=int32[L:512, N:12288]', 'scales=float16[K:32, N:12288]'])
    assert fuse_elementwise(g2).canonical_key() == f.canonical_key()


def test_statement_separators():
    g = parse_program('a1[N] = x[N] + 1\n  a2[N] = a1[N] *\n      2\n out[N] = a2[N]; out2[N] = out[N]', ['x=float32[N:8]'])
    assert [s.output for s in g.statements] == ['a1', 'a2', 'out', 'out2']


def test_config_strings_are_parsed_leniently():
    from antares_amd.autort.op import parse_config
    assert parse_config('tune:5') == {'tune': 5}
    assert parse_config('~N~:[256,8,32],~S~:[64,8]') == {'~N~': [256, 8, 32], '~S~': [64, 8]}
    assert parse_config(None) == {} and parse_config('whatever') == {'whatever': ''}


def test_hand_kernel_roles_follow_the_program_not_the_names():
    """A program spelled with other tensor names than the registered pattern still selects the hand-written kernel,
    and each of its tensors is bound to the part it plays in the program (first appearance in the fused statements)."""
    from antares_amd.autort import patterns
    from antares_amd.autort.op import ExportedOp
    gemm = ExportedOp('''
        mid[M, N] +=! input0[M, K].to(`float32`) * input1[K, N].to(`float32`)
        output0[M, N] = mid[M, N].to(`float16`)
    ''', ['input1=float16[K:64, N:64]', 'input0=float16[M:64, K:64]'])
    assert gemm.fast_path is patterns._gemm_f16_handler
    assert {r: gemm.fast_roles[r] for r in ('a', 'b', 'c')} == {'a': 'input0', 'b': 'input1', 'c': 'output0'}
    w4 = ExportedOp(patterns.W4A16_IR.replace('qweight', 'qw').replace('scales', 'sc').replace('qzeros', 'qz')
                    .replace('x[', 'lhs[').replace('y[', 'out[').replace('acc[', 'tmp['),
                    ['qz=int8[G:32, NH:5504]', 'lhs=float16[M:1, K:4096]', 'sc=float16[G:32, N:11008]', 'qw=int8[KH:2048, N:11008]'])
    assert w4.fast_path is patterns._w4a16_handler
    assert {r: w4.fast_roles[r] for r in ('x', 'qweight', 'scales', 'qzeros', 'y')} == \
        {'x': 'lhs', 'qweight': 'qw', 'scales': 'sc', 'qzeros': 'qz', 'y': 'out'}
    gptq = ExportedOp(patterns.GPTQ_GEMV_IR.replace('input0', 'vec').replace('qweight', 'packed').replace('scales', 'sc')
                      .replace('my_result', 'res'), ['vec=float32[S:4096]', 'packed=int32[L:512, N:12288]', 'sc=float16[K:32, N:12288]'])
    assert gptq.fast_path is patterns._gptq_handler
    assert {r: gptq.fast_roles[r] for r in ('input0', 'qweight', 'scales', 'my_result')} == \
        {'input0': 'vec', 'qweight': 'packed', 'scales': 'sc', 'my_result': 'res'}
    # the registered spelling maps to itself
    own = ExportedOp(patterns.GEMM_F16_IR, patterns.GEMM_F16_INPUTS)
    assert own.fast_roles['a'] == 'a' and own.fast_roles['c'] == 'c'


def test_programs_that_restrict_an_axis_do_not_take_a_hand_kernel():
    """The hand kernels take every size from the operands' shapes; `where K in 100` or `where M in 100` spell the same
    statements as the full product but compute a shorter sum or a smaller output, so they must go to the generic
    lowering (the canonical key alone cannot tell them apart)."""
    from antares_amd.autort import patterns
    from antares_amd.autort.op import ExportedOp
    from antares_amd.ir import fuse_elementwise, parse_program
    cases = [(patterns.GEMM_F32_IR, patterns.GEMM_F32_INPUTS), (patterns.BATCH_GEMM_F32_IR, patterns.BATCH_GEMM_F32_INPUTS),
             ('c[M, N] +=! a[K, M] * b[K, N]', ['a=float32[K:512, M:512]', 'b=float32[K:512, N:512]']),
             ('c[M, N] +=! a[M, K] * b[N, K]', ['a=float32[M:512, K:512]', 'b=float32[N:512, K:512]']),
             ('c[M, N] +=! a[K, M] * b[N, K]', ['a=float32[K:512, M:512]', 'b=float32[N:512, K:512]'])]
    for ir, inputs in cases:
        assert patterns.match(fuse_elementwise(parse_program(ir, inputs))) is not None, ir
        for clause in ('K in 100', 'M in 100', 'N in 8'):
            g = fuse_elementwise(parse_program(f'{ir} where {clause}', inputs))
            assert patterns.match(g) is None, (ir, clause)
            assert ExportedOp(f'{ir} where {clause}', list(inputs)).fast_path is None
    # the two-statement programs: a restricted reduce axis in the first statement
    f16 = patterns.GEMM_F16_IR.strip().split('\n')
    restricted = f16[0] + ' where K in 64\n' + f16[1]
    assert patterns.match(fuse_elementwise(parse_program(patterns.GEMM_F16_IR, patterns.GEMM_F16_INPUTS))) is not None
    assert patterns.match(fuse_elementwise(parse_program(restricted, patterns.GEMM_F16_INPUTS))) is None
    w4 = patterns.W4A16_IR.strip().split('\n')
    assert patterns.match(fuse_elementwise(parse_program(w4[0] + ' where N in 16\n' + w4[1] + ' where N in 16', patterns.W4A16_INPUTS))) is None
    # a `where` that only repeats the dimension, or static shapes of the full extent, still match
    assert patterns.match(fuse_elementwise(parse_program('c[M, N] +=! a[M, K] * b[K, N] where K in 4096',
                                                         ['a=float32[4096, 4096]', 'b=float32[4096, 4096]']))) is not None
