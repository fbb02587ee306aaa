"""Worked programs of the reference's IR documentation (AntaresIR.md:108-256) at reduced sizes, each with an
independent numpy statement of what it computes.  Used as fixtures by test_ir_examples.py: the CPU oracle must
reproduce the numpy result, the gfx950 lowering must reproduce the oracle."""
import numpy as np


def _f32(*shape):
    return {'dtype': 'float32', 'shape': list(shape)}


def _i32(*shape):
    return {'dtype': 'int32', 'shape': list(shape)}


def _i8(*shape):
    return {'dtype': 'int8', 'shape': list(shape)}


def _conv_nopad(x, w):
    n, c, h, wd = x.shape
    f, _, kh, kw = w.shape
    out = np.zeros((n, f, h - kh + 1, wd - kw + 1), np.float64)
    for i in range(kh):
        for j in range(kw):
            out += np.einsum('nchw,fc->nfhw', x[:, :, i:i + out.shape[2], j:j + out.shape[3]].astype(np.float64), w[:, :, i, j].astype(np.float64))
    return out


def _pool(x, k, s, fn):
    n, c, h, w = x.shape
    ho, wo = (h - k) // s + 1, (w - k) // s + 1
    win = np.stack([x[:, :, i:i + s * ho:s, j:j + s * wo:s] for i in range(k) for j in range(k)], 0)
    return fn(win, 0)


# name -> (program, input_dict, extra_outputs, reference(**inputs) -> {output name: array})
EXAMPLES = {
    'broadcast': ('output0[N, F, HO, WO] = input0[N] where F in 32, HO in 2, WO in 2', {'input0': _f32(16)}, [],
                  lambda input0: {'output0': np.broadcast_to(input0[:, None, None, None], (16, 32, 2, 2))}),
    'broadcast_all': ('output0[N, F, HO, WO] = input0[0] where N in 8, F in 32, HO in 2, WO in 2', {'input0': _f32(1)}, [],
                      lambda input0: {'output0': np.full((8, 32, 2, 2), input0[0])}),
    'matmul': ('output0[N, M] +=! input0[N, K] * input1[K, M]', {'input0': _f32(48, 40), 'input1': _f32(40, 56)}, [],
               lambda input0, input1: {'output0': input0.astype(np.float64) @ input1.astype(np.float64)}),
    'matmul_bias_add': ('output0[N, M] +=! input0[N, K] * input1[K, M] + input2[M] / K.val()',
                        {'input0': _f32(24, 32), 'input1': _f32(32, 16), 'input2': _f32(16)}, [],
                        lambda input0, input1, input2: {'output0': input0.astype(np.float64) @ input1.astype(np.float64) + input2}),
    'batch_matmul': ('output0[B, N, M] +=! input0[B, N, K] * input1[B, K, M]', {'input0': _f32(3, 20, 24), 'input1': _f32(3, 24, 12)}, [],
                     lambda input0, input1: {'output0': np.einsum('bnk,bkm->bnm', input0.astype(np.float64), input1.astype(np.float64))}),
    'elementwise': ('output0[N] = input0[N] + input1[N]', {'input0': _f32(5000), 'input1': _f32(5000)}, [],
                    lambda input0, input1: {'output0': input0 + input1}),
    'scalar': ('output0[] = input0[] + input1[]', {'input0': _f32(), 'input1': _f32()}, [],
               lambda input0, input1: {'output0': input0 + input1}),
    'multiple_outputs': ('output0[N] = input0[N] + input1[N]; output1[N] = input0[N] * 2; output2[N] = input1[N] + output1[N];',
                         {'input0': _f32(3000), 'input1': _f32(3000)}, ['output0', 'output1', 'output2'],
                         lambda input0, input1: {'output0': input0 + input1, 'output1': input0 * 2, 'output2': input1 + input0 * 2}),
    'transpose': ('output0[N, C, H, W] = input0[N, H, W, C]', {'input0': _f32(2, 9, 7, 3)}, [],
                  lambda input0: {'output0': input0.transpose(0, 3, 1, 2)}),
    'reshape': ('output0[A, B, C] = input0[A, B, C / 64, C % 64] where C in 128', {'input0': _f32(3, 3, 2, 64)}, [],
                lambda input0: {'output0': input0.reshape(3, 3, 128)}),
    'reduce_sum': ('output0[N] +=! input0[N, C]', {'input0': _f32(32, 300)}, [], lambda input0: {'output0': input0.astype(np.float64).sum(1)}),
    'reduce_min': ('output0[N] <=! input0[N, C]', {'input0': _f32(32, 300)}, [], lambda input0: {'output0': input0.min(1)}),
    'reduce_all': ('output0[N] &=! input0[N, C]', {'input0': _i8(32, 100)}, [], lambda input0: {'output0': (input0 != 0).all(1).astype(np.int8)}),
    'reduce_any': ('output0[N] |=! input0[N, C]', {'input0': _i8(32, 100)}, [], lambda input0: {'output0': (input0 != 0).any(1).astype(np.int8)}),
    'cast_range': ('output0[N] = N.cast(`float32`) where N in 1024', {}, [], lambda: {'output0': np.arange(1024, dtype=np.float32)}),
    'relu': ('output0[N, C] = input0[N, C].when([input0[N, C] > 0.0], 0.0)', {'input0': _f32(40, 33)}, [],
             lambda input0: {'output0': np.maximum(input0, 0)}),
    'relu_dynamic_dtype': ('output0[N, C] = input0[N, C].when([input0[N, C] > const(0.0).cast(input0[N, C].dtype())], const(0.0).cast(input0[N, C].dtype()))',
                           {'input0': _f32(40, 33)}, [], lambda input0: {'output0': np.maximum(input0, 0)}),
    'range_tanh': ('output0[N] = N.cast(`float32`).call(`tanh`) where N in 64', {}, [],
                   lambda: {'output0': np.tanh(np.arange(64, dtype=np.float64))}),
    'conv_nopad': ('output0[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[F, C, KH, KW] where HO in 6, WO in 6',
                   {'input0': _f32(2, 5, 8, 8), 'input1': _f32(4, 5, 3, 3)}, [],
                   lambda input0, input1: {'output0': _conv_nopad(input0, input1)}),
    'depth_to_space': ('output0[N, H, C0, W, C1, C2] = input0[N, H, W, C0, C1, C2]', {'input0': _f32(1, 6, 5, 2, 2, 4)}, [],
                       lambda input0: {'output0': input0.transpose(0, 1, 3, 2, 4, 5)}),
    'depthwise_conv': ('output0[N, C, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[KH, KW, C, 0] where HO in 6, WO in 6',
                       {'input0': _f32(2, 4, 8, 8), 'input1': _f32(3, 3, 4, 1)}, [],
                       lambda input0, input1: {'output0': sum(input0[:, :, i:i + 6, j:j + 6].astype(np.float64) * input1[i, j, :, 0][None, :, None, None]
                                                               for i in range(3) for j in range(3))}),
    'slice': ('output0[N, F] = input0[N, F, 2]', {'input0': _f32(1, 16, 32)}, [], lambda input0: {'output0': input0[:, :, 2]}),
    'concat': ('output0[N, F] = input0[N, F].when([F < 128], input1[N, F - 128]) where F in 256', {'input0': _f32(4, 128), 'input1': _f32(4, 128)}, [],
               lambda input0, input1: {'output0': np.concatenate([input0, input1], 1)}),
    'one_hot': ('output0[N, F] = const(1.0).when([input0[N] == F], const(0.0)) where F in 128', {'input0': _i32(4)}, [],
                lambda input0: {'output0': (input0[:, None] == np.arange(128)[None]).astype(np.float32)}),
    'take': ('output0[F, C] = input0[input1[F], C]', {'input0': _f32(71, 24), 'input1': _i32(50)}, [],
             lambda input0, input1: {'output0': input0[input1]}),
    'gather': ('output0[N, F] = input0[input1[N, F]]', {'input0': _f32(71), 'input1': _i32(4, 16)}, [],
               lambda input0, input1: {'output0': input0[input1]}),
    'pad': ('output0[N, C, HO, WO] = input0[N, C, -1 + HO, -1 + WO].when([-1 + HO >= 0, -1 + HO < 8, -1 + WO >= 0, -1 + WO < 8], 0.0) where HO in 10, WO in 10',
            {'input0': _f32(2, 3, 8, 8)}, [], lambda input0: {'output0': np.pad(input0, ((0, 0), (0, 0), (1, 1), (1, 1)))}),
    'div_no_nan': ('output0[N] = (input0[N] / input1[N]).when([input1[N] != 0], 0.0)', {'input0': _f32(1000), 'input1': _f32(1000)}, [],
                   lambda input0, input1: {'output0': np.where(input1 != 0, input0 / np.where(input1 != 0, input1, 1), 0)}),
    'max_pool': ('output0[N, C, HO, WO] >=! input0[N, C, HO * 2 + KH, WO * 2 + KW] where HO in 6, WO in 6, KW in 2, KH in 2',
                 {'input0': _f32(4, 3, 12, 12)}, [], lambda input0: {'output0': _pool(input0, 2, 2, np.max)}),
    'avg_pool': ('output0[NC, HO, WO] +=! input0[NC, HO * 3 + KH, WO * 3 + KW] / 9.0 where HO in 5, WO in 5, KW in 3, KH in 3',
                 {'input0': _f32(6, 15, 15)}, [], lambda input0: {'output0': _pool(input0[None].astype(np.float64), 3, 3, np.mean)[0]}),
    'tile': ('output0[ON, OC] = input0[ON % 2, OC % 16] where ON in 64, OC in 96', {'input0': _f32(2, 16)}, [],
             lambda input0: {'output0': np.tile(input0, (32, 6))}),
    'softmax': ('temp0[N] >=! input0[N, C]; temp1[N] +=! (input0[N, C] - temp0[N]).call(`exp`); output0[N, C] = (input0[N, C] - temp0[N]).call(`exp`) / temp1[N]',
                {'input0': _f32(8, 200)}, [],
                lambda input0: {'output0': np.exp(input0.astype(np.float64) - input0.max(1, keepdims=True)) /
                                np.exp(input0.astype(np.float64) - input0.max(1, keepdims=True)).sum(1, keepdims=True)}),
    'batch_norm': ('output0[N, C, H, W] = bias[C] + scale[C] * (input0[N, C, H, W] - mean[C]) * (variance[C] + 1e-5).call(`rsqrt`)',
                   {'input0': _f32(2, 6, 4, 4), 'mean': _f32(6), 'variance': _f32(6), 'scale': _f32(6), 'bias': _f32(6)}, [],
                   lambda input0, mean, variance, scale, bias: {'output0': bias[None, :, None, None] + scale[None, :, None, None] *
                                                                (input0 - mean[None, :, None, None]) / np.sqrt(np.abs(variance)[None, :, None, None] + 1e-5)}),
    'layer_norm': ('temp0[N] +=! input0[N, C]; temp1[N] +=! input0[N, C] * input0[N, C]; output0[N, C] = (input0[N, C] * C.val() - temp0[N]) * (temp1[N] * C.val() - temp0[N] * temp0[N] + 1e-5).call(`rsqrt`)',
                   {'input0': _f32(8, 64)}, [],
                   lambda input0: {'output0': (input0.astype(np.float64) * 64 - input0.astype(np.float64).sum(1, keepdims=True)) /
                                   np.sqrt((input0.astype(np.float64) ** 2).sum(1, keepdims=True) * 64 - input0.astype(np.float64).sum(1, keepdims=True) ** 2 + 1e-5)}),
    'logical': ('output0[N, M] = input0[N, M] & ~input1[N, M]', {'input0': _i8(30, 20), 'input1': _i8(30, 20)}, [],
                lambda input0, input1: {'output0': ((input0 != 0) & (input1 == 0)).astype(np.int8)}),   # logical, not bitwise (default_codegen.py:73-79)
    'sigmoid': ('output0[N, M] = 1.0 / (1.0 + (-input0[N, M]).call(`exp`))', {'input0': _f32(30, 20)}, [],
                lambda input0: {'output0': 1 / (1 + np.exp(-input0.astype(np.float64)))}),
    'add_matmul_head_fusion': ('temp0[K, N] = input0[N, K] + 100; output0[N, M] +=! temp0[K, N] * input1[K, M] where K in 10',
                               {'input0': _f32(24, 16), 'input1': _f32(16, 12)}, [],
                               lambda input0, input1: {'output0': (input0[:, :10].astype(np.float64) + 100) @ input1[:10].astype(np.float64)}),
    'conv_bias_relu_tail_fusion': ('conv_out[N, F, HO, WO] +=! input0[N, C, HO + KH, WO + KW] * input1[KH, KW, C, F] where HO in 6, WO in 6; '
                                   'conv_bias[N, F, HO, WO] = conv_out[N, F, HO, WO] + input2[0, 0, 0, F]; '
                                   'output0[N, F, HO, WO] = conv_bias[N, F, HO, WO].when(conv_bias[N, F, HO, WO] > 0.0, 0.0)',
                                   {'input0': _f32(2, 5, 8, 8), 'input1': _f32(3, 3, 5, 4), 'input2': _f32(1, 1, 1, 4)}, [],
                                   lambda input0, input1, input2: {'output0': np.maximum(_conv_nopad(input0, input1.transpose(3, 2, 0, 1)) + input2[0, 0, 0][None, :, None, None], 0)}),
    'scatter4d': ('data[indices[B, 0], indices[B, 1], indices[B, 2], indices[B, 3], M] =. updates[B, M]',
                  {'data': _f32(4, 4, 4, 4, 8), 'indices': _i32(2, 4), 'updates': _f32(2, 8)}, [], None),   # reference built in the test (in-out tensor)
    'vectorized_bool_check': ('output0[N] = ((input0[N, 0] == 0).cast(`int32`) << 24) + ((input0[N, 1] == 0).cast(`int32`) << 16) + ((input0[N, 2] == 0).cast(`int32`) << 8) + (input0[N, 3] == 0).cast(`int32`)',
                              {'input0': _i32(100, 4)}, [],
                              lambda input0: {'output0': ((input0[:, 0] == 0).astype(np.int32) << 24) + ((input0[:, 1] == 0).astype(np.int32) << 16) +
                                              ((input0[:, 2] == 0).astype(np.int32) << 8) + (input0[:, 3] == 0).astype(np.int32)}),
}


def make_inputs(name, seed=0):
    """Deterministic inputs of the declared shapes: floats in [-2, 2), indices inside the tensors they address."""
    _, input_dict, _, _ = EXAMPLES[name]
    rng = np.random.default_rng(seed + sum(map(ord, name)))
    out = {}
    for k, spec in input_dict.items():
        shape = tuple(spec['shape'])
        if spec['dtype'] == 'float32':
            a = (rng.random(shape) * 4 - 2).astype(np.float32)
            if name == 'div_no_nan' and k == 'input1':
                a[::7] = 0
            if name == 'batch_norm' and k == 'variance':
                a = np.abs(a)
        elif spec['dtype'] == 'int8':
            a = rng.integers(0, 2, shape).astype(np.int8) if name.startswith('reduce') else rng.integers(-1, 3, shape).astype(np.int8)
            if name == 'reduce_all':
                a[::3] = 1
        else:
            hi = {'one_hot': 128, 'take': 71, 'gather': 71, 'scatter4d': 4, 'vectorized_bool_check': 3}[name]
            a = rng.integers(0, hi, shape).astype(np.int32)
        out[k] = a
    if name == 'scatter4d':
        out['indices'] = np.array([[0, 1, 2, 3], [3, 2, 1, 0]], np.int32)     # distinct destinations
    return out
