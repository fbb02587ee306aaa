"""Decisions the generic lowering takes from the text of a program alone (no GPU): which statements one row kernel
may cover, and that the generated source compiles for gfx950."""
import pytest

from antares_amd.ir import parse_program
from antares_amd.ir.graph import fuse_elementwise
from antares_amd.lower import hip_codegen

SOFTMAX = ('temp0[N] >=! input0[N, C]; temp1[N] +=! (input0[N, C] - temp0[N]).call(`exp`); '
           'output0[N, C] = (input0[N, C] - temp0[N]).call(`exp`) / temp1[N]')


def lowered(ir, inputs):
    return hip_codegen.lower_graph(fuse_elementwise(parse_program(ir, inputs)))


def test_softmax_is_one_row_group_with_kernels_for_short_and_long_rows():
    src, plans = lowered(SOFTMAX, ['input0=float32[N:32, C:1024]'])
    group = plans[0].row_group
    assert group is not None and group.count == 3 and plans[1].row_group is None and plans[2].row_group is None
    assert group.args == ['input0', 'temp0', 'temp1', 'output0']
    assert group.red_axis[0] == 'C' and [a for a, _ in group.row_axes] == ['N']
    kernels = {(team, v, e): sym for team, v, e, sym in group.cached}
    assert set(kernels) == {(64, 1, 4), (256, 1, 4), (256, 1, 16), (64, 4, 4), (256, 4, 4), (256, 4, 16)}
    assert group.vec_tensors == ['input0', 'output0']
    zero, odd = {n: 0 for n in group.args}, {**{n: 0 for n in group.args}, 'input0': 4}
    # a block per row and 16-byte vectors where the row length and the addresses allow
    assert group.choose({'N': 32, 'C': 1024}, zero) == (kernels[(256, 4, 4)], 32)
    assert group.choose({'N': 32, 'C': 1024}, odd) == (kernels[(256, 1, 4)], 32)
    assert group.choose({'N': 32, 'C': 1022}, zero) == (kernels[(256, 1, 4)], 32)
    assert group.choose({'N': 32, 'C': 4100}, zero) == (kernels[(256, 4, 16)], 32)
    assert group.choose({'N': 32, 'C': 4099}, zero) == (group.symbol, 32)           # too long for registers: walked
    assert group.choose({'N': 32, 'C': 16388}, zero) == (group.symbol, 32)
    # many short rows: a wavefront per row, four rows per block
    assert group.choose({'N': 65536, 'C': 256}, zero) == (kernels[(64, 4, 4)], hip_codegen.MAX_GRID)
    assert group.choose({'N': 10001, 'C': 250}, zero) == (kernels[(64, 1, 4)], 2501)
    # a handful of very long rows, and rows shorter than two wavefronts, are left to the per-statement kernels
    assert group.choose({'N': 8, 'C': 1 << 20}, zero)[1] == 0 and group.choose({'N': 64, 'C': 1 << 20}, zero)[1] == 64
    assert group.choose({'N': 32, 'C': 127}, zero)[1] == 0
    for sym in [group.symbol] + list(kernels.values()):
        assert f'void {sym}(' in src


@pytest.mark.parametrize('ir,inputs,covered', [
    # the map reads a result at another row's position: the reduction alone is a group
    ('t[N] +=! x[N, C]; y[N, C] = x[N, C] - t[(N + 1) % 8]', ['x=float32[N:8, C:256]'], 1),
    # the map is over other axes than the reduction
    ('t[N] +=! x[N, C]; y[N, K] = z[N, K] - t[N]', ['x=float32[N:8, C:256]', 'z=float32[N:8, K:256]'], 1),
    # a map that stores only where a condition holds
    ('t[N] +=! x[N, C]; y[N, C] = (x[N, C] - t[N]).when([x[N, C] > 0])', ['x=float32[N:8, C:256]', 'y=float32[N:8, C:256]'], 1),
    # a reduction alone; two of them; an offset in front of the reduced axis
    ('t[N] +=! x[N, C]', ['x=float32[N:8, C:256]'], 1),
    ('t[N] +=! x[N, C]; u[N] >=! x[N, C] * t[N]', ['x=float32[N:8, C:256]'], 2),
    ('t[N] +=! x[N, C] * w[C]', ['x=float32[N:8, C:256]', 'w=float32[C:256]'], 1),
    ('t[S] +=! x[S * 1024 + C] where C in 1024, S in 8', ['x=float32[N:8192]'], 1),
    # the reduction runs over the first axis: lanes of a team would read addresses a row apart
    ('t[C] +=! x[N, C]; y[N, C] = x[N, C] - t[C]', ['x=float32[N:8, C:256]'], 0),
    ('t[N] +=! x[C, N]', ['x=float32[C:256, N:8]'], 0),
    # contractions: no load is indexed by all the data axes
    ('c[N, M] +=! a[N, K] * b[K, M]', ['a=float32[N:64, K:256]', 'b=float32[K:256, M:64]'], 0),
    ('c[N, M] +=! a[N, K] * b[M, K]', ['a=float32[N:64, K:256]', 'b=float32[M:64, K:256]'], 0),
    # a map alone
    ('y[N, C] = x[N, C] * 2', ['x=float32[N:8, C:256]'], 0),
])
def test_which_statements_a_row_group_covers(ir, inputs, covered):
    _, plans = lowered(ir, inputs)
    group = plans[0].row_group
    if covered == 0:
        assert all(p.row_group is None for p in plans)
    else:
        assert group is not None and group.count == covered and group.pure
        zero = {n: 0 for n in group.args}
        # reductions alone: with enough rows to fill the chip, or when all of it is one short launch out of
        # registers; few long rows are left alone (they are sliced first)
        assert group.choose({'N': 8, 'C': 256, 'K': 256, 'S': 8}, zero)[1] > 0
        if 'S * 1024' not in ir:
            assert group.choose({'N': 8, 'C': 65536, 'K': 256}, zero)[1] == 0
            assert group.choose({'N': 100, 'C': 4096, 'K': 256}, zero)[1] == 0
            assert group.choose({'N': 512, 'C': 4096, 'K': 256}, zero)[1] == 512
    if 'S * 1024' in ir:
        assert [sym for team, v, e, sym in group.cached if (team, v, e) == (64, 4, 4)]   # the offset 1024 S keeps rows 16-byte aligned


def test_row_kernels_compile_for_gfx950(tmp_path, monkeypatch):
    monkeypatch.setenv('AUTORT_CACHE_DIR', str(tmp_path / 'cache'))
    from antares_amd.autort.op import compile_cached
    ir = ('ss[B, N] +=! x[B, N, C].to(`float32`) * x[B, N, C].to(`float32`); '
          'y[B, N, C] = (x[B, N, C].to(`float32`) * (ss[B, N] / C.val() + 1e-5).call(`rsqrt`) * w[C].to(`float32`)).to(`float16`)')
    src, plans = lowered(ir, ['x=float16[B:3, N:17, C:520]', 'w=float16[C:520]'])
    assert plans[0].row_group is not None and plans[0].row_group.count == 2
    assert len(compile_cached(src)) > 1000


PADDED_CONV = ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH - 1, WO + KW - 1].when([HO + KH - 1 >= 0, HO + KH - 1 < 56, '
               'WO + KW - 1 >= 0, WO + KW - 1 < 56], 0.0) * input1[F, C, KH, KW] where HO in 56, WO in 56')


def test_a_padded_convolution_goes_to_the_matrix_kernels_with_its_guards_tabled(tmp_path, monkeypatch):
    """AntaresIR.md:166: the zero padding is a `when` around the image operand.  Its four conditions compare two values,
    each a row part plus a k part; the kernels table those beside the addresses and never fetch outside them."""
    monkeypatch.setenv('AUTORT_CACHE_DIR', str(tmp_path / 'cache'))
    from antares_amd.autort.op import compile_cached
    graph = fuse_elementwise(parse_program(PADDED_CONV, ['input0=float32[N:8, C:64, H:56, W:56]', 'input1=float32[F:64, C:64, KH:3, KW:3]']))
    mc = hip_codegen._matrix_contraction(graph.statements[0], graph.tensors)
    # the image uses the output's last axis: it is made the second factor (columns), so that stores run along WO
    assert mc['la'].name == 'input1' and mc['lb'].name == 'input0' and mc['n'] == ['N', 'HO', 'WO'] and mc['m'] == ['F']
    assert [g[2] for g in mc['guards']['b']] == ['<=', '<', '<=', '<'] and mc['guards']['a'] == []
    assert len({(g[0], g[1]) for g in mc['guards']['b']}) == 2 and not mc['vec']['b']
    src, plans = hip_codegen.lower_graph(graph)
    # the guarded image is fetched element by element; the weights lie as rows of k = (C, KH, KW): 16-byte vectors
    assert mc['vec']['a'] and {'matrix', 'matrix64', 'matrixv', 'matrix64v'} <= set(plans[0].variants)
    assert plans[0].matrix['vec_tensors'] == ['input1']
    assert '__gmb[2][128]' in src and '__gmb[2][64]' in src
    # 25088 rows x 64 columns: tiles of 128 columns would be half padding, the small tiles take it
    env = {'N': 8, 'C': 64, 'H': 56, 'W': 56, 'F': 64, 'KH': 3, 'KW': 3}
    assert plans[0]._matrix_choice(env, {n: 0 for n in plans[0].args}) == ('matrix64v', 392)
    # 196 big blocks would be one round that is three quarters full: the small ones fill the chip; 3136 big blocks are
    # thirteen rounds of 256, less than 12544 small blocks at a 900th of a round each
    assert plans[0]._matrix_choice({**env, 'F': 128}, {n: 0 for n in plans[0].args}) == ('matrix64v', 784)
    assert plans[0]._matrix_choice({**env, 'N': 32, 'F': 512}, {n: 0 for n in plans[0].args}) == ('matrixv', 3136)
    assert plans[0]._matrix_choice(env, {**{n: 0 for n in plans[0].args}, 'input1': 4}) == ('matrix64', 392)
    assert len(compile_cached(src)) > 1000
    # a guard that mixes rows and k in a product, or reads a tensor, leaves the statement to the other variants
    for cond in ('HO * KH < 56', 'input1[F, C, KH, KW] > 0'):
        ir = f'output0[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW].when([{cond}], 0.0) * input1[F, C, KH, KW] where HO in 54, WO in 54'
        g2 = fuse_elementwise(parse_program(ir, ['input0=float32[N:8, C:64, H:56, W:56]', 'input1=float32[F:64, C:64, KH:3, KW:3]']))
        assert hip_codegen._matrix_contraction(g2.statements[0], g2.tensors) is None


def test_graph_rewrites_for_one_call_keep_the_program_on_the_oracle():
    """Two rewrites made per set of dimension values: a reduction over (N, H, W) with few outputs is sliced along all of
    N, and reduce extents of a few named elements become constants.  Both leave the oracle's results where they were."""
    import numpy as np
    from antares_amd.ir.graph import bake_small_reduce_extents, split_wide_reductions
    from oracle.cpu_backend import CpuModule
    rng = np.random.default_rng(5)
    # channel sums: 24 outputs, the outermost reduce axis has 16 values and is sliced into 16
    prog = parse_program('output0[C] +=! input0[N, C, H, W]', ['input0=float32[N:16, C:24, H:20, W:20]'])
    env = {'N': 16, 'C': 24, 'H': 20, 'W': 20}
    sliced = split_wide_reductions(fuse_elementwise(prog), env)
    assert len(sliced.statements) == 2 and sliced.statements[0].data_axes[0][1] == 16
    assert [e for _, e in sliced.statements[0].reduce_axes] == [1, 'H', 'W']
    x = rng.standard_normal((16, 24, 20, 20)).astype(np.float32)
    assert np.allclose(CpuModule(sliced, fast_math=False)(input0=x)['output0'], x.astype(np.float64).sum((0, 2, 3)), rtol=1e-5, atol=1e-3)
    # a single reduce axis is never sliced into slices of one element
    one = split_wide_reductions(fuse_elementwise(parse_program('output0[C] +=! input0[N, C]', ['input0=float32[N:16, C:24]'])), {'N': 16, 'C': 24})
    assert len(one.statements) == 1
    # a depthwise filter of named size 3 x 3; a filter of 9 x 9 stays symbolic
    ir = 'output0[N, C, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[C, KH, KW] where HO in 6, WO in 6'
    inputs = ['input0=float32[N:2, C:3, H:8, W:8]', 'input1=float32[C:3, KH:3, KW:3]']
    g = fuse_elementwise(parse_program(ir, inputs))
    env = {'N': 2, 'C': 3, 'H': 8, 'W': 8, 'KH': 3, 'KW': 3}
    baked = bake_small_reduce_extents(g, env)
    assert baked is not g and baked.statements[0].reduce_axes == [('KH', 3), ('KW', 3)] and baked.tensors['input1'].shape == ['C', 3, 3]
    assert baked.dim_names == g.dim_names                  # the kernels keep every dimension as an argument
    assert bake_small_reduce_extents(g, {**env, 'KH': 9, 'KW': 9}) is g
    a, w = rng.standard_normal((2, 3, 8, 8)).astype(np.float32), rng.standard_normal((3, 3, 3)).astype(np.float32)
    assert np.array_equal(CpuModule(baked, fast_math=False)(input0=a, input1=w)['output0'], CpuModule(g, fast_math=False)(input0=a, input1=w)['output0'])
    src, plans = hip_codegen.lower_graph(baked)
    assert 'const int __ext_KH = 3;' in src and 'int __dim_KH' in src


def test_contractions_with_few_tiles_are_sliced_along_k_and_keep_their_vector_fetches():
    """512 x 512 outputs are 64 tiles of 64 x 64: over 8192 values of k the contraction is cut into 8 slices that run as
    a batch (slices in front, so the statement is still a contraction) and a sum over the slices; each operand is rows
    of k inside a slice too.  Enough tiles, or a short k, and nothing is cut."""
    import numpy as np
    from antares_amd.ir.graph import split_wide_reductions
    from antares_amd.lower import contraction_slices
    from oracle.cpu_backend import CpuModule
    ir, inputs = 'output0[N, M] +=! input0[N, K] * input1[M, K]', ['input0=float32[N:512, K:8192]', 'input1=float32[M:512, K:8192]']
    g = fuse_elementwise(parse_program(ir, inputs))
    env = {'N': 512, 'M': 512, 'K': 8192}
    cut = split_wide_reductions(g, env, wanted=contraction_slices(g.tensors))
    assert len(cut.statements) == 2
    s1, s2 = cut.statements
    assert s1.data_axes[0] == ('KS', 8) and s1.reduce_axes == [('KC', 1024)] and cut.tensors[s1.output].shape == [8, 'N', 'M']
    assert [a for a, _ in s2.reduce_axes] == ['KS'] and s2.output == 'output0'
    assert split_wide_reductions(cut, env, wanted=contraction_slices(cut.tensors)) is cut          # not cut twice
    mc = hip_codegen._matrix_contraction(s1, cut.tensors)
    assert mc['batch'] == ['KS'] and mc['vec'] == {'a': True, 'b': True} and mc['pitch'] == {'a': ['K'], 'b': ['K']}
    src, plans = hip_codegen.lower_graph(cut)
    zero = {n: 0 for n in plans[0].args}
    assert plans[0]._matrix_choice(env, zero) == ('matrix64v', 512)
    # a row of the tensor that is no whole number of vectors: element-wise fetches (never the case for a sliced K, but the
    # launcher checks what it is given)
    plans[0].matrix['vec_pitch'] = [[8190], ['K']]
    assert plans[0]._matrix_choice(env, zero) == ('matrix64', 512)
    for e in ({'N': 2048, 'M': 2048, 'K': 8192}, {'N': 512, 'M': 512, 'K': 512}, {'N': 16, 'M': 4096, 'K': 8192}):
        assert split_wide_reductions(g, e, wanted=contraction_slices(g.tensors)) is g
    # the two-statement form computes the same thing
    small = fuse_elementwise(parse_program(ir, ['input0=float32[N:64, K:2048]', 'input1=float32[M:64, K:2048]']))
    cut = split_wide_reductions(small, {'N': 64, 'M': 64, 'K': 2048}, wanted=lambda st, value: None if '__part' in st.output else 4)
    assert len(cut.statements) == 2
    rng = np.random.default_rng(3)
    a, b = rng.standard_normal((64, 2048)).astype(np.float32), rng.standard_normal((64, 2048)).astype(np.float32)
    got = CpuModule(cut, fast_math=False)(input0=a, input1=b)['output0']
    assert np.allclose(got, a.astype(np.float64) @ b.astype(np.float64).T, rtol=1e-5, atol=1e-3)


def test_the_programs_of_the_lowering_benchmark_lower_and_take_the_kernels_they_are_listed_for():
    """`bench.py --lowering` times these programs on the GPU; here: each parses and lowers, the contractions have
    matrix-instruction kernels, the two row programs are one row group each, and the fused tail is one launch."""
    import bench
    for name, ir, inputs, shapes, (kind, count) in bench.LOWERING_CASES:
        graph = fuse_elementwise(parse_program(ir, inputs))
        src, plans = hip_codegen.lower_graph(graph)
        assert len(plans) == len(graph.statements) and src
        if kind == 'flop':
            assert 'matrix' in plans[0].variants, name
        if 'AntaresIR.md:226' in name or 'AntaresIR.md:232' in name:
            assert plans[0].row_group is not None and plans[0].row_group.count == 3, name
        if 'one launch' in name:
            assert plans[0].covers == 2, name


def test_a_zero_padded_factor_is_copied_into_a_padded_tensor_once():
    """`x[.., HO * 2 + KH - 1, WO + KW - 1].when([bounds], 0) * w[...]`: the guards are evaluated once per element of a
    padded copy, the contraction reads the copy unguarded; the rewrite is refused when it cannot prove what it needs."""
    import numpy as np
    from antares_amd.ir.graph import pad_guarded_factors
    from oracle.cpu_backend import CpuModule
    conv = ('output0[N, F, HO, WO] +=! input0[N, C, HO * 2 + KH - 1, WO + KW - 1].when([HO * 2 + KH - 1 >= 0, HO * 2 + KH - 1 < 32, '
            'WO + KW - 1 >= 0, WO + KW - 1 < 32], 0.0) * input1[F, C, KH, KW] where HO in 16, WO in 32')
    inputs = ['input0=float32[N:2, C:8, H:32, W:32]', 'input1=float32[F:8, C:8, KH:3, KW:3]']
    g = fuse_elementwise(parse_program(conv, inputs))
    env = {'N': 2, 'C': 8, 'H': 32, 'W': 32, 'F': 8, 'KH': 3, 'KW': 3}
    padded = pad_guarded_factors(g, env)
    assert [s.output for s in padded.statements] == ['input0__pad', 'output0'] and padded.tensors['input0__pad'].shape == [2, 8, 33, 34]
    assert pad_guarded_factors(padded, env) is padded and pad_guarded_factors(g, {}) is g        # once; and not without the extents
    mc = hip_codegen._matrix_contraction(padded.statements[1], padded.tensors)
    assert mc is not None and mc['guards'] == {'a': [], 'b': []}
    rng = np.random.default_rng(1)
    x, w = rng.standard_normal((2, 8, 32, 32)).astype(np.float32), rng.standard_normal((8, 8, 3, 3)).astype(np.float32)
    assert np.array_equal(CpuModule(padded, fast_math=False)(input0=x, input1=w)['output0'], CpuModule(g, fast_math=False)(input0=x, input1=w)['output0'])
    refused = [
        # a condition on something that is no index of the load; an unguarded index that may leave the tensor; too few terms
        conv.replace('WO + KW - 1 < 32]', 'WO + KW - 1 < 32, HO < 9]'),
        conv.replace('input0[N, C,', 'input0[N + 1, C,').replace('WO in 32', 'WO in 32, N in 2'),
        'output0[N, M] +=! input0[N, K + 5].when([K + 5 < 40], 0.0) * input1[K, M] where K in 40',
    ]
    for ir in refused[:2]:
        g2 = fuse_elementwise(parse_program(ir, inputs))
        assert pad_guarded_factors(g2, env) is g2, ir
    g3 = fuse_elementwise(parse_program(refused[2], ['input0=float32[N:64, J:40]', 'input1=float32[K:40, M:64]']))
    assert pad_guarded_factors(g3, {'N': 64, 'J': 40, 'K': 40, 'M': 64}) is g3


def test_the_padding_rewrite_leaves_guarded_values_that_do_not_map_zero_to_zero():
    """`g(x[..]).when(conds, 0) * w`: the border contributes 0, not g(0) * w.  The rewrite into a padded copy is only
    taken for a bare load or casts of it; whatever the rewrite returns must compute what the program as written does
    (both run through the CPU oracle, before and after)."""
    import numpy as np
    from antares_amd.ir.graph import pad_guarded_factors
    from oracle.cpu_backend import CpuModule
    guards = '.when([HO + KH - 1 >= 0, HO + KH - 1 < 16, WO + KW - 1 >= 0, WO + KW - 1 < 16], 0.0)'
    idx = 'input0[N, C, HO + KH - 1, WO + KW - 1]'
    env = {'N': 2, 'C': 8, 'H': 16, 'W': 16, 'F': 4, 'KH': 3, 'KW': 3}
    rng = np.random.default_rng(2)
    w = rng.standard_normal((4, 8, 3, 3)).astype(np.float32)
    cases = [
        (f'({idx} + 1.0)', 'float32', False),                        # g(0) = 1
        (f'{idx}.call(`exp`)', 'float32', False),                    # g(0) = 1
        (f'({idx} * 2.0)', 'float32', False),                        # maps 0 to 0, but not proved: left alone
        (idx, 'float32', True),
        (f'{idx}.cast(`float32`)', 'float16', True),                 # a cast stays around the padded load
    ]
    for factor, dt, rewritten in cases:
        ir = f'output0[N, F, HO, WO] +=! {factor}{guards} * input1[F, C, KH, KW] where HO in 16, WO in 16'
        g = fuse_elementwise(parse_program(ir, [f'input0={dt}[N:2, C:8, H:16, W:16]', 'input1=float32[F:4, C:8, KH:3, KW:3]']))
        after = pad_guarded_factors(g, env)
        assert (after is not g) == rewritten, factor
        x = rng.standard_normal((2, 8, 16, 16)).astype(np.float16 if dt == 'float16' else np.float32)
        want = CpuModule(g, fast_math=False)(input0=x, input1=w)['output0']
        got = CpuModule(after, fast_math=False)(input0=x, input1=w)['output0']
        assert np.array_equal(got, want), factor
    # what the refused rewrite would have done wrong: the border of the `+ 1.0` case is not the interior's formula
    ir = f'output0[N, F, HO, WO] +=! ({idx} + 1.0){guards} * input1[F, C, KH, KW] where HO in 16, WO in 16'
    g = fuse_elementwise(parse_program(ir, ['input0=float32[N:2, C:8, H:16, W:16]', 'input1=float32[F:4, C:8, KH:3, KW:3]']))
    x = rng.standard_normal((2, 8, 16, 16)).astype(np.float32)
    out = CpuModule(g, fast_math=False)(input0=x, input1=w)['output0']
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1))) + 1.0                 # the wrong reading: g applied to the padding
    wrong = np.einsum('nchw,fc->nfhw', xp[:, :, 0:16, 0:16], w[:, :, 0, 0])
    for kh in range(3):
        for kw in range(3):
            if kh or kw:
                wrong += np.einsum('nchw,fc->nfhw', xp[:, :, kh:kh + 16, kw:kw + 16], w[:, :, kh, kw])
    assert np.abs(out - wrong)[:, :, 0, :].max() > 0.5 and np.allclose(out[:, :, 1:15, 1:15], wrong[:, :, 1:15, 1:15], atol=1e-4)
