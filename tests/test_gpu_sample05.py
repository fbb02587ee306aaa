"""The decode step of samples/05_llama2_7b_int4.py written the way the sample writes it - fp32 activations, the
GPTQ int32 weight layout, `autort.export` of the sample's own three-statement program, `autort.ops.rmsnorm_f32 /
rotary_f32 / attention_f32` on views of the caches, torch for the glue - on a small random model, against the
same step computed by the CPU oracle's operators.  What it pins: the sample's calling conventions work unchanged
(outputs written through views with `out=`, scalars through `extra=`, the fused v|q|k projection that parks q and k
in the value cache, lines :146-177)."""
import math

import numpy as np
import pytest
import torch

from antares_amd import workloads

pytestmark = pytest.mark.gpu

LAYERS, HEADS, HEAD, HIDDEN, VOCAB, SEQ = 2, 4, 128, 1024, 512, 12
DIM = HEADS * HEAD
SAMPLE_IR = """
  input1[S, N] = (qweight[S / 8, N] >> (S % 8 * 4)).call(strs.bitwise_and, 15) * input0[S].like(1)
  w[S, N] = scales[S / 128, N] * (input1[S, N] - 8)
  my_result[N] +=! input0[S] * w[S, N].to(input0.dtype())
"""


def gptq_linear(g, K, N):
    q = torch.randint(0, 16, (K, N), generator=g)
    return {'qweight': workloads.pack_gptq(q), 'scales': torch.rand(K // 128, N, generator=g) * 0.019 + 0.001}


def make_model(seed=5):
    g = torch.Generator().manual_seed(seed)
    m = {'embed': torch.randn(VOCAB, DIM, generator=g) * 0.5, 'classify': torch.randn(VOCAB, DIM, generator=g) * 0.05,
         'rms_end': 1 + 0.1 * torch.randn(DIM, generator=g), 'layers': []}
    for _ in range(LAYERS):
        m['layers'].append({'rms_att': 1 + 0.1 * torch.randn(DIM, generator=g), 'rms_ffn': 1 + 0.1 * torch.randn(DIM, generator=g),
                            'vqk': gptq_linear(g, DIM, 3 * DIM), 'o': gptq_linear(g, DIM, DIM), 'f1': gptq_linear(g, DIM, HIDDEN),
                            'f3': gptq_linear(g, DIM, HIDDEN), 'f2': gptq_linear(g, HIDDEN, DIM)})
    return m


def inv_frequencies():
    inv = 1.0 / (10000.0 ** (torch.arange(0, HEAD, 2).float() / HEAD))
    return torch.cat([inv, inv]).view(HEAD)


class OracleStep:
    """The same step out of the oracle's operators, fp32 throughout."""

    def __init__(self, m):
        from oracle import hot_ops
        self.ops, self.m = hot_ops, m
        self.key = np.zeros((LAYERS, SEQ + 2, DIM), np.float32)
        self.val = np.zeros((LAYERS, SEQ + 2, DIM), np.float32)
        self.inv = inv_frequencies().numpy()

    def linear(self, x, lin):
        return self.ops.gemv_gptq_f32(x.astype(np.float32), lin['qweight'].numpy(), lin['scales'].numpy())

    def norm(self, x, w):
        vsum = np.array([(x * x).sum(dtype=np.float32)], np.float32)
        return self.ops.rmsnorm(x, vsum, w.numpy(), 1.0 / x.size, 1e-5, np.float32)

    def forward(self, token, pos):
        x = self.m['embed'][token].numpy().copy()
        for l, lw in enumerate(self.m['layers']):
            vqk = self.linear(self.norm(x, lw['rms_att']), lw['vqk'])
            v, q, k = vqk[:DIM], vqk[DIM:2 * DIM], vqk[2 * DIM:]
            self.val[l, pos] = v
            q = self.ops.rotary(q.reshape(HEADS, 2, -1), self.inv, pos)
            self.key[l, pos] = self.ops.rotary(k.reshape(HEADS, 2, -1), self.inv, pos).reshape(-1)
            att = self.ops.attention(q, self.key[l, :pos + 1].reshape(pos + 1, HEADS, HEAD), self.val[l, :pos + 1].reshape(pos + 1, HEADS, HEAD),
                                     1 / math.sqrt(HEAD))
            x = x + self.linear(att.reshape(-1), lw['o'])
            xb = self.norm(x, lw['rms_ffn'])
            gate, up = self.linear(xb, lw['f1']), self.linear(xb, lw['f3'])
            x = x + self.linear(gate / (1 + np.exp(-gate)) * up, lw['f2'])
        return self.norm(x, self.m['rms_end']) @ self.m['classify'].numpy().T


def test_sample_decode_step_as_the_sample_writes_it(oracle_built):
    import autort
    device = autort.device()
    m = make_model()
    dev = lambda t: t.to(device)
    layers = [{k: ({kk: dev(vv) for kk, vv in v.items()} if isinstance(v, dict) else dev(v)) for k, v in lw.items()} for lw in m['layers']]
    embed, classify, rms_end = dev(m['embed']), dev(m['classify']), dev(m['rms_end'])
    key_cache = torch.zeros([LAYERS, SEQ + 2, DIM], dtype=torch.float32, device=device)
    val_cache = torch.zeros([LAYERS, SEQ + 2, DIM], dtype=torch.float32, device=device)     # two spare rows: q and k park at pos+1, pos+2
    att_f = torch.tensor([1 / math.sqrt(HEAD)], dtype=torch.float32, device=device)
    inv_freq = dev(inv_frequencies())

    my_custom_fn = autort.export(ir=SAMPLE_IR, inputs=["input0=float32[S:4096]", "qweight=int32[L:512, N:12288]", "scales=float32[K:32, N:12288]"],
                                 config='~N~:[256,8,32],~S~:[64,8]')
    assert my_custom_fn.fast_path is not None          # the sample's program runs on the hand-written kernel

    def rmsnorm(x, weight):
        x = x.float()
        vsum = (x * x).sum().view(1)
        return autort.ops.rmsnorm_f32(x.view(-1), vsum, weight.float(), extra=[1.0 / int(x.numel())])

    def matmul_dequat(x, lin, memory_out=None):
        x = x.view(-1)
        memory_out = memory_out if memory_out is not None else torch.empty([lin['qweight'].size(-1)], dtype=x.dtype, device=x.device)
        return my_custom_fn(x, lin['qweight'], lin['scales'], out=memory_out.view(-1))

    def forward(token, pos):
        x = embed.select(0, token).view(1, DIM)
        for l in range(LAYERS):
            lw = layers[l]
            xb = rmsnorm(x, lw['rms_att'])
            local_cache = val_cache.select(0, l).narrow(0, pos, 3)
            matmul_dequat(xb, lw['vqk'], memory_out=local_cache.view(-1, 3 * xb.size(-1)))
            sq, sk = local_cache[1], local_cache[2]
            sq_out = torch.empty_like(sq).view(HEADS, HEAD)
            sk_out = key_cache.select(0, l).narrow(0, pos, 1).view(HEADS, HEAD)
            autort.ops.rotary_f32(sq.view(HEADS, 2, -1), inv_freq, sq_out, extra=[pos, ])
            autort.ops.rotary_f32(sk.view(HEADS, 2, -1), inv_freq, sk_out, extra=[pos, ])
            b_sk = key_cache.select(0, l).view(SEQ + 2, HEADS, HEAD).narrow(0, 0, pos + 1)
            b_sv = val_cache.select(0, l).view(SEQ + 2, HEADS, HEAD).narrow(0, 0, pos + 1)
            xb = autort.ops.attention_f32(sq_out, b_sk, b_sv, att_f)
            x = x + matmul_dequat(xb, lw['o'])
            xb = rmsnorm(x, lw['rms_ffn'])
            xb = torch.nn.functional.silu(matmul_dequat(xb, lw['f1'])) * matmul_dequat(xb, lw['f3'])
            x = x + matmul_dequat(xb, lw['f2'])
        x = rmsnorm(x, rms_end)
        return torch.matmul(x, classify.t())

    ref = OracleStep(m)
    token = 3
    with torch.no_grad():
        for pos in range(SEQ):
            print(f'[case] sample step pos={pos} token={token}', flush=True)
            want = ref.forward(token, pos)
            got = forward(token, pos).float().cpu().numpy().reshape(-1)
            assert np.allclose(got, want, rtol=2e-4, atol=2e-4), (pos, np.abs(got - want).max())
            token = int(np.argmax(want))


def test_programs_spelled_with_other_names_run_on_the_hand_kernels(oracle_built):
    """The same three programs with tensor names other than the registered ones: the hand-written kernel must be
    selected and fed the right operands (a rectangular, non-symmetric case so that a swapped operand cannot pass)."""
    import autort
    from antares_amd import workloads
    from antares_amd.autort import patterns
    from oracle import hot_ops
    dev = autort.device()
    print('[case] fp16 GEMM as input0/input1/output0', flush=True)
    f = autort.export(ir='''
        mid[M, N] +=! input0[M, K].to(`float32`) * input1[K, N].to(`float32`)
        output0[M, N] = mid[M, N].to(`float16`)
    ''', inputs=['input0=float16[M:4096, K:4096]', 'input1=float16[K:4096, N:4096]'], name='gemm_f16_renamed')
    assert f.fast_path is not None
    g = torch.Generator().manual_seed(2)
    a = (torch.randn(96, 128, generator=g) * 0.1).half()
    b = (torch.randn(128, 72, generator=g) * 0.1).half()
    got = f(a.to(dev), b.to(dev)).cpu()
    assert torch.allclose(got.float(), (a.double() @ b.double()).float(), rtol=1e-2, atol=1e-2)

    print('[case] int4 GEMV as lhs/qw/sc/qz', flush=True)
    ir = (patterns.W4A16_IR.replace('qweight', 'qw').replace('scales', 'sc').replace('qzeros', 'qz')
          .replace('x[', 'lhs[').replace('y[', 'out[').replace('acc[', 'tmp['))
    h = autort.export(ir=ir, inputs=['lhs=float16[M:1, K:4096]', 'qw=int8[KH:2048, N:11008]', 'sc=float16[G:32, N:11008]',
                                     'qz=int8[G:32, NH:5504]'], name='gemv_w4a16_renamed')
    assert h.fast_path is not None
    p = workloads.w4_problem(21, 1, 1024, 272)
    y = h(p['x'].to(dev), p['qweight'].to(dev), p['scales'].to(dev), p['qzeros'].to(dev)).cpu().numpy()
    want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    assert np.allclose(y.astype(np.float32), want.astype(np.float32), rtol=1e-2, atol=1e-2)

    print('[case] GPTQ GEMV as vec/packed/sc', flush=True)
    ir = SAMPLE_IR.replace('input0', 'vec').replace('qweight', 'packed').replace('scales', 'sc').replace('my_result', 'res')
    k = autort.export(ir=ir, inputs=['vec=float32[S:4096]', 'packed=int32[L:512, N:12288]', 'sc=float32[K:32, N:12288]'],
                      name='gemv_gptq_renamed')
    assert k.fast_path is not None
    lin = gptq_linear(g, 2048, 192)
    x = torch.randn(2048, generator=g)
    y = k(x.to(dev), lin['qweight'].to(dev), lin['scales'].to(dev)).cpu().numpy()
    want = hot_ops.gemv_gptq_f32(x.numpy(), lin['qweight'].numpy(), lin['scales'].numpy())
    assert np.allclose(y, want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize('K,N', [(2048, 192), (4096, 4096), (11008, 512)])
def test_gptq_fp32_results_keep_fp32_precision_at_any_magnitude(oracle_built, K, N):
    """The K-splits of an fp32 result meet exactly: outputs around 1e-7 are as accurate relative to their size as
    outputs around 1, outputs around 1e6 do not turn into NaN, and a second call gives the same bits."""
    import autort
    from oracle import hot_ops
    dev = autort.device()
    f = autort.export(ir=SAMPLE_IR, inputs=["input0=float32[S:4096]", "qweight=int32[L:512, N:12288]", "scales=float32[K:32, N:12288]"])
    g = torch.Generator().manual_seed(K + N)
    lin = gptq_linear(g, K, N)
    x = torch.randn(K, generator=g)
    for name, xs, ss in [('unit', 1.0, 1.0), ('tiny', 1e-3, 1e-4), ('huge', 1e3, 1e3)]:
        print(f'[case] gptq fp32 magnitudes K={K} N={N} {name}', flush=True)
        xv, sv = x * xs, lin['scales'] * ss
        got = f(xv.to(dev), lin['qweight'].to(dev), sv.to(dev))
        again = f(xv.to(dev), lin['qweight'].to(dev), sv.to(dev))
        assert torch.equal(got, again)
        got = got.cpu().numpy()
        want = hot_ops.gemv_gptq_f32(xv.numpy(), lin['qweight'].numpy(), sv.numpy())
        assert np.isfinite(got).all()
        # relative to the size of the sums involved: an fp32 sum of K terms is good to about sqrt(K) * 2^-24 of the
        # magnitude of its terms, whatever that magnitude is
        scale = float(np.abs(want).mean())
        assert np.abs(got - want).max() < 2e-4 * scale, (name, np.abs(got - want).max(), scale)
