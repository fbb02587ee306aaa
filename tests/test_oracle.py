"""Pins the CPU oracle: README known answers, closed forms, special cases that
a dropped term / wrong nibble order / transposed operand would break, and the
agreement of its two independent halves (plain-C hot_ops vs the loop nests
emitted from the IR)."""
import math

import numpy as np
import pytest
import torch

from antares_amd import workloads
from antares_amd.autort import patterns
from antares_amd.ir import parse_program

pytestmark = pytest.mark.usefixtures('oracle_built')

README_SIGMOID = [0.5000, 0.7311, 0.8808, 0.9526, 0.9820, 0.9933, 0.9975, 0.9991, 0.9997, 0.9999]   # README.md:68
README_SORT_IN = [101, 102, 208, 99, 1, 127, 62, 8, 336, 336]                                       # samples/01_sort_even_first.py:36
README_SORT_OUT = [102, 208, 62, 8, 336, 336, 101, 99, 1, 127]                                      # README.md:95-99


def cpu_module(ir, inputs, **kw):
    from oracle.cpu_backend import CpuModule
    return CpuModule(parse_program(ir, inputs), **kw)


def test_sigmoid_known_answer():
    from oracle import hot_ops
    x = np.arange(10, dtype=np.float32)
    assert np.allclose(hot_ops.sigmoid_f32(x), README_SIGMOID, atol=5e-5)
    m = cpu_module('sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))', ['data=float32[N:4096000]'])
    assert np.allclose(m(data=x)['sigmoid_f32'], README_SIGMOID, atol=5e-5)


def test_sigmoid_matches_float64_closed_form():
    from oracle import hot_ops
    x = workloads.sigmoid_input(1, 100_000).numpy()
    want = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    assert np.allclose(hot_ops.sigmoid_f32(x), want, rtol=1e-5, atol=1e-6)
    m = cpu_module('sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))', ['data=float32[N:4096000]'])
    assert np.allclose(m(data=x)['sigmoid_f32'], want, rtol=1e-5, atol=1e-6)


def sort_pipeline_via_ir(x: np.ndarray) -> np.ndarray:
    """The sample's three steps with the two exported programs run by the IR oracle."""
    m1 = cpu_module('space[data[N] % 2, N] = 1', ['data=int32[N]', 'space=int32[2, N]'])
    m2 = cpu_module('output[ids[N] - 1] = (val[N % val.size(0)]).when(ids[N] > 0)',
                    ['ids=int32[N]', 'val=int32[M]', 'output=int32[M]'])
    space = np.zeros((2, x.size), np.int32)
    m1(data=x, space=space)
    ids = (np.cumsum(space.reshape(-1), dtype=np.int32) * space.reshape(-1)).astype(np.int32)
    out = np.zeros_like(x)
    m2(ids=ids, val=x, output=out)
    return out


def test_sort_known_answer():
    from oracle import hot_ops
    x = np.array(README_SORT_IN, dtype=np.int32)
    assert hot_ops.sort_even_first_i32(x).tolist() == README_SORT_OUT
    assert sort_pipeline_via_ir(x).tolist() == README_SORT_OUT


@pytest.mark.parametrize('n', [1, 2, 63, 64, 65, 4095, 4096, 4097, 100_003])
def test_sort_is_stable_partition(n):
    from oracle import hot_ops
    x = workloads.partition_input(n, n).numpy()
    want = np.concatenate([x[x % 2 == 0], x[x % 2 == 1]])
    assert np.array_equal(hot_ops.sort_even_first_i32(x), want)
    if n <= 4097:
        assert np.array_equal(sort_pipeline_via_ir(x), want)


def test_sort_all_even_all_odd():
    from oracle import hot_ops
    ev = np.arange(0, 2000, 2, dtype=np.int32)
    od = ev + 1
    assert np.array_equal(hot_ops.sort_even_first_i32(ev), ev)
    assert np.array_equal(hot_ops.sort_even_first_i32(od), od)


# ---------------------------------------------------------------- int4 products
def dequant_f64(p):
    q, z, s = p['q'].numpy().astype(np.float64), p['z'].numpy().astype(np.float64), p['scales'].numpy().astype(np.float64)
    return (q - np.repeat(z, 128, axis=0)) * np.repeat(s, 128, axis=0)


def test_w4a16_against_float64():
    from oracle import hot_ops
    p = workloads.w4_problem(3, 2, 256, 64)
    got = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    want = p['x'].numpy().astype(np.float64) @ dequant_f64(p)
    assert np.allclose(got.astype(np.float64), want, rtol=4e-3, atol=4e-3)


def test_w4a16_special_cases_pin_layout():
    from oracle import hot_ops
    K, N = 256, 32
    ones = np.ones((K // 128, N), np.float16)
    # q == z everywhere -> y == 0
    q = torch.full((K, N), 7, dtype=torch.uint8)
    z = torch.full((K // 128, N), 7, dtype=torch.uint8)
    x = np.random.default_rng(0).standard_normal((1, K)).astype(np.float16)
    y = hot_ops.gemm_w4a16(x, workloads.pack_w4(q).numpy(), ones, workloads.pack_z4(z).numpy())
    assert np.all(y == 0)
    # scales 1, z 0, q 1 -> y = sum(x)
    q = torch.ones((K, N), dtype=torch.uint8)
    z = torch.zeros((K // 128, N), dtype=torch.uint8)
    y = hot_ops.gemm_w4a16(x, workloads.pack_w4(q).numpy(), ones, workloads.pack_z4(z).numpy())
    assert np.allclose(y.astype(np.float32), x.astype(np.float32).sum(), atol=2e-2)
    # a single nibble q[k0, n0] = 9 and x one-hot at k0: y[n0] = 9, zero elsewhere (pins nibble order along K)
    for k0, n0 in [(0, 0), (1, 5), (130, 17), (255, 31)]:
        q = torch.zeros((K, N), dtype=torch.uint8)
        q[k0, n0] = 9
        xx = np.zeros((1, K), np.float16)
        xx[0, k0] = 1
        y = hot_ops.gemm_w4a16(xx, workloads.pack_w4(q).numpy(), ones, workloads.pack_z4(z).numpy())
        want = np.zeros(N)
        want[n0] = 9
        assert np.array_equal(y[0].astype(np.float64), want)
    # a single zero point z[g0, n0] = 5 with q = 5 at one k of that group and x all ones (pins nibble order along N)
    for g0, n0 in [(0, 0), (1, 1), (1, 30)]:
        z = torch.zeros((K // 128, N), dtype=torch.uint8)
        z[g0, n0] = 5
        q = torch.zeros((K, N), dtype=torch.uint8)
        xx = np.ones((1, K), np.float16)
        y = hot_ops.gemm_w4a16(xx, workloads.pack_w4(q).numpy(), ones, workloads.pack_z4(z).numpy())
        want = np.zeros(N)
        want[n0] = -5 * 128
        assert np.array_equal(y[0].astype(np.float64), want)


def test_w4a16_ir_program_agrees_with_plain_c():
    from oracle import hot_ops
    p = workloads.w4_problem(5, 3, 256, 64)
    m = cpu_module(patterns.W4A16_IR, patterns.W4A16_INPUTS, fast_math=False)
    got = m(x=p['x'].numpy(), qweight=p['qweight'].numpy(), scales=p['scales'].numpy(), qzeros=p['qzeros'].numpy())['y']
    want = hot_ops.gemm_w4a16(p['x'].numpy(), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy())
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize('scales_dtype', [np.float32, np.float16])
def test_gptq_program(scales_dtype):
    from oracle import hot_ops
    K, N = 512, 96
    g = torch.Generator().manual_seed(11)
    q = torch.randint(0, 16, (K, N), generator=g)
    s = (torch.rand(K // 128, N, generator=g) * 0.019 + 0.001).numpy().astype(scales_dtype)
    x = torch.randn(K, generator=g).numpy()
    qw = workloads.pack_gptq(q).numpy()
    got = hot_ops.gemv_gptq_f32(x, qw, s)
    want = x.astype(np.float64) @ ((q.numpy().astype(np.float64) - 8) * np.repeat(s.astype(np.float64), 128, axis=0))
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4)
    sd = 'float32' if scales_dtype == np.float32 else 'float16'
    m = cpu_module(patterns.GPTQ_GEMV_IR, patterns._gptq_inputs('float32', sd), fast_math=False)
    got_ir = m(input0=x, qweight=qw, scales=s)['my_result']
    assert np.allclose(got_ir, got, rtol=1e-6, atol=1e-6)
    # nibble j of a word is k % 8 == j: one-hot check
    q1 = torch.full((K, N), 8)
    q1[13, 7] = 15
    x1 = np.zeros(K, np.float32)
    x1[13] = 1
    y = hot_ops.gemv_gptq_f32(x1, workloads.pack_gptq(q1).numpy(), np.ones((K // 128, N), scales_dtype))
    want1 = np.zeros(N)
    want1[7] = 7
    assert np.array_equal(y, want1)


# ---------------------------------------------------------------- harness
def test_fill_and_digest_closed_form():
    from oracle.cpu_backend import digest, fill
    a = fill(np.zeros(1000, np.float32), 'float32', 2)
    assert np.array_equal(a, (np.arange(1000) + 3) % 71)
    assert np.array_equal(fill(np.ones(10, np.int32), 'int32', 0), np.zeros(10))
    # the harness converts with bare bit moves (execute_module.hpp:46-55): exact for 1..70, but a float 0.0
    # becomes the half 0x4000 = 2.0, and a half 0x0000 is read back as 2^-15 by the digest
    h = fill(np.zeros(100, np.float16), 'float16', 0)
    want16 = ((np.arange(100) + 1) % 71).astype(np.float32)
    want16[want16 == 0] = 2.0
    assert np.array_equal(h.astype(np.float32), want16) and h[70] == 2.0
    assert digest(np.zeros(10, np.float16), 'float16') == pytest.approx(sum(range(1, 11)) * 2.0 ** -15, rel=1e-12)
    assert digest(np.full(4, 1.5, np.float16), 'float16') == pytest.approx(1.5 * (1 + 2 + 3 + 4), rel=1e-12)
    out = np.linspace(-1, 1, 500).astype(np.float32)
    want = float(np.sum(((np.arange(500) + 1) % 83) * out.astype(np.float64)))
    assert digest(out, 'float32') == pytest.approx(want, rel=1e-12)


def test_reduce_identities_and_ops():
    x = np.random.default_rng(1).standard_normal((8, 33)).astype(np.float32)
    inp = {'input0': {'dtype': 'float32', 'shape': [8, 33]}}
    assert np.allclose(cpu_module('output0[N] +=! input0[N, C]', dict(inp))(input0=x)['output0'], x.sum(1), rtol=1e-5, atol=1e-5)
    assert np.array_equal(cpu_module('output0[N] >=! input0[N, C]', dict(inp))(input0=x)['output0'], x.max(1))
    assert np.array_equal(cpu_module('output0[N] <=! input0[N, C]', dict(inp))(input0=x)['output0'], x.min(1))
    b = (np.random.default_rng(2).random((8, 33)) > 0.9).astype(np.int8)
    inp8 = {'input0': {'dtype': 'int8', 'shape': [8, 33]}}
    assert np.array_equal(cpu_module('output0[N] |=! input0[N, C]', dict(inp8))(input0=b)['output0'], b.any(1))
    assert np.array_equal(cpu_module('output0[N] &=! input0[N, C]', dict(inp8))(input0=b)['output0'], b.all(1))


# ---------------------------------------------------------------- llama operators
def test_rmsnorm_closed_forms():
    from oracle import hot_ops
    rng = np.random.default_rng(5)
    n = 4096
    x, w = rng.standard_normal(n).astype(np.float32), (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    vsum = np.array([(x.astype(np.float64) ** 2).sum()], np.float32)
    out = hot_ops.rmsnorm(x, vsum, w, 1.0 / n)
    want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean() + 1e-5) * w
    assert np.allclose(out, want, rtol=1e-5, atol=1e-6)
    # invariant: sum (out/w)^2 = N / (1 + eps N / sum x^2)
    lhs = ((out.astype(np.float64) / w) ** 2).sum()
    assert lhs == pytest.approx(n / (1 + 1e-5 * n / float(vsum[0])), rel=1e-5)
    # computing the sum of squares inside gives the same thing
    assert np.allclose(hot_ops.rmsnorm(x, None, w), out, rtol=1e-5, atol=1e-6)
    # eps matters: a tiny input is damped, not blown up
    tiny = hot_ops.rmsnorm(x * 1e-4, None, w)
    assert np.abs(tiny).max() < np.abs(out).max()


def test_rotary_closed_forms():
    from oracle import hot_ops
    rng = np.random.default_rng(6)
    H, D = 4, 128
    x = rng.standard_normal((H, 2, D // 2)).astype(np.float32)
    f = (1.0 / (10000.0 ** (np.arange(0, D, 2, dtype=np.float64) / D))).astype(np.float32)
    inv_freq = np.concatenate([f, f])
    assert np.array_equal(hot_ops.rotary(x, inv_freq, 0), x.reshape(H, D))          # pos 0 = identity
    for pos in (1, 7, 383):
        out = hot_ops.rotary(x, inv_freq, pos).astype(np.float64)
        # HF Llama: x*cos + rotate_half(x)*sin, rotate_half(x) = cat(-x2, x1)
        xf = x.reshape(H, D).astype(np.float64)
        ang = pos * inv_freq.astype(np.float32).astype(np.float64)
        rot = np.concatenate([-xf[:, D // 2:], xf[:, :D // 2]], axis=1)
        assert np.allclose(out, xf * np.cos(ang) + rot * np.sin(ang), atol=2e-4)   # fp32 sin/cos of angles up to 383 rad
        # each (j, j + D/2) pair keeps its norm
        n_in = xf[:, :D // 2] ** 2 + xf[:, D // 2:] ** 2
        n_out = out[:, :D // 2] ** 2 + out[:, D // 2:] ** 2
        assert np.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)


def test_rotate_interleaved():
    from oracle import hot_ops
    rng = np.random.default_rng(7)
    dim = 64
    data = rng.standard_normal(dim).astype(np.float32)
    coef = rng.random(dim // 2).astype(np.float32)
    assert np.array_equal(hot_ops.rotate(coef, data, 0), data)
    out = hot_ops.rotate(coef, data, 5).astype(np.float64)
    z = (data[0::2] + 1j * data[1::2]) * np.exp(1j * 5 * coef.astype(np.float64))       # complex multiplication form
    assert np.allclose(out[0::2], z.real, atol=1e-5) and np.allclose(out[1::2], z.imag, atol=1e-5)


def test_attention_closed_forms():
    from oracle import hot_ops
    rng = np.random.default_rng(8)
    S, H, D = 37, 4, 128
    q = rng.standard_normal((H, D)).astype(np.float32)
    k = rng.standard_normal((S, H, D)).astype(np.float32)
    v = rng.standard_normal((S, H, D)).astype(np.float32)
    f = 1.0 / np.sqrt(D)
    out = hot_ops.attention(q, k, v, f)
    att = np.einsum('hm,shm->hs', q.astype(np.float64), k.astype(np.float64)) * f
    att = np.exp(att - att.max(1, keepdims=True))
    att /= att.sum(1, keepdims=True)
    assert np.allclose(out, np.einsum('hs,shm->hm', att, v.astype(np.float64)), rtol=1e-5, atol=1e-5)
    # q = 0 -> uniform weights -> mean of v ; S = 1 -> v[0]
    assert np.allclose(hot_ops.attention(np.zeros_like(q), k, v, f), v.mean(0), rtol=1e-5, atol=1e-5)
    assert np.allclose(hot_ops.attention(q, k[:1], v[:1], f), v[0], rtol=1e-6, atol=1e-6)


# ---------------------------------------------------------------- decode step
def _dense_f64(lin):
    """Packed int4 linear -> dense float64 [K, N] with plain torch indexing (no oracle code)."""
    qw, s, qz = lin['qweight'], lin['scales'].double(), lin['qzeros']
    K, N = qw.shape[0] * 2, qw.shape[1]
    q = torch.empty(K, N, dtype=torch.float64)
    q[0::2] = (qw & 15).double()
    q[1::2] = (qw >> 4).double()
    z = torch.empty(K // 128, N, dtype=torch.float64)
    z[:, 0::2] = (qz & 15).double()
    z[:, 1::2] = (qz >> 4).double()
    return (q - z.repeat_interleave(128, 0)) * s.repeat_interleave(128, 0)


class TorchDecodeF64:
    """The forward pass of samples/05_llama2_7b_int4.py:146-177 written from the sample's text with torch float64
    tensors and library routines (dense matmul, torch.nn.functional.silu, torch.softmax, the Hugging Face
    x*cos + rotate_half(x)*sin), sharing no code with oracle/llama_ref.py or oracle/hot_ops.c."""

    def __init__(self, cfg, w):
        self.cfg = cfg
        self.embed = w['embed'].double()
        self.final_norm = w['final_norm'].double()
        self.lm_head = _dense_f64(w['lm_head'])
        self.layers = [{'att_norm': lw['att_norm'].double(), 'ffn_norm': lw['ffn_norm'].double(),
                        'qkv': _dense_f64(lw['qkv']), 'o': _dense_f64(lw['o']),
                        'gate_up': _dense_f64(lw['gate_up']), 'down': _dense_f64(lw['down'])} for lw in w['layers']]
        D = cfg.head_dim
        inv = (1.0 / (cfg.rope_base ** (torch.arange(0, D, 2).float() / D))).to(torch.float16)     # sample :125
        self.inv_freq = torch.cat([inv, inv]).double()                                             # sample :126
        self.keys = torch.zeros(cfg.n_layers, cfg.max_seq, cfg.n_heads, D, dtype=torch.float64)
        self.vals = torch.zeros_like(self.keys)

    def norm(self, x, w):                                         # sample :128-131
        return x * torch.rsqrt((x * x).mean() + self.cfg.rms_eps) * w

    def rope(self, x, pos):                                       # [H, D]
        half = x.shape[-1] // 2
        ang = pos * self.inv_freq
        rotate_half = torch.cat([-x[:, half:], x[:, :half]], dim=-1)
        return x * torch.cos(ang) + rotate_half * torch.sin(ang)

    def forward(self, token, pos):
        cfg = self.cfg
        d, H, D = cfg.dim, cfg.n_heads, cfg.head_dim
        x = self.embed[token]                                      # :147
        for l, lw in enumerate(self.layers):
            xb = self.norm(x, lw['att_norm'])                      # :150
            q, k, v = (xb @ lw['qkv']).split(d)                    # :151-153, columns q | k | v in this build
            self.keys[l, pos] = self.rope(k.view(H, D), pos)       # :158
            self.vals[l, pos] = v.view(H, D)
            q = self.rope(q.view(H, D), pos)                       # :157
            ks, vs = self.keys[l, :pos + 1], self.vals[l, :pos + 1]                      # :162-163
            att = torch.softmax(torch.einsum('hd,shd->hs', q, ks) / math.sqrt(D), dim=-1)   # samples/03_llama_tiny.py:94-99
            xb = torch.einsum('hs,shd->hd', att, vs).reshape(d)    # :165
            x = x + xb @ lw['o']                                   # :167-168
            xb = self.norm(x, lw['ffn_norm'])                      # :169
            gate, up = (xb @ lw['gate_up']).split(cfg.ffn)         # f1 = gate_proj, f3 = up_proj
            x = x + (torch.nn.functional.silu(gate) * up) @ lw['down']                   # :171-173
        return self.norm(x, self.final_norm) @ self.lm_head        # :175-176


def test_decode_oracle_against_independent_float64_restatement():
    """LlamaRef.forward (the checker of the decode parity tests) against TorchDecodeF64 over 10 positions of a
    prompt-then-greedy run.  A swapped gate/up, a residual in the wrong place, a missing final norm, a wrong
    rotary pairing or cache row would each move the logits by O(1)."""
    from antares_amd.llama import LlamaConfig, random_weights
    from oracle.llama_ref import LlamaRef
    cfg = LlamaConfig(n_layers=2, dim=512, n_heads=4, ffn=1024, vocab=1024, max_seq=32)
    w = random_weights(cfg, seed=3)
    ref, ind = LlamaRef(cfg, w), TorchDecodeF64(cfg, w)
    prompt = [5, 77, 901]
    token = prompt[0]
    worst = 0.0
    for pos in range(10):
        got = ref.forward(token, pos).astype(np.float64)
        want = ind.forward(token, pos).numpy()
        assert want.std() > 0.3                                     # the logits are not degenerate
        worst = max(worst, np.abs(got - want).max())
        # the oracle rounds every operator output to fp16; the restatement rounds nothing
        assert np.allclose(got, want, rtol=2e-2, atol=2e-2), (pos, np.abs(got - want).max())
        top2 = np.sort(want)[-2:]
        if top2[1] - top2[0] > 0.05:
            assert int(np.argmax(got)) == int(np.argmax(want)), pos
        token = prompt[pos + 1] if pos + 1 < len(prompt) else int(np.argmax(want))
        for l in range(cfg.n_layers):                               # the cache rows both sides wrote at this position
            assert np.allclose(ref.key_cache[l, pos].astype(np.float64), ind.keys[l, pos].reshape(-1).numpy(), rtol=2e-2, atol=2e-2)
            assert np.allclose(ref.val_cache[l, pos].astype(np.float64), ind.vals[l, pos].reshape(-1).numpy(), rtol=2e-2, atol=2e-2)
    assert worst < 2e-2


def test_decode_oracle_restatement_detects_plausible_mistakes():
    """The check above has teeth: each of these mis-readings of the sample moves the logits far outside its tolerance."""
    from antares_amd.llama import LlamaConfig, random_weights
    cfg = LlamaConfig(n_layers=2, dim=512, n_heads=4, ffn=1024, vocab=1024, max_seq=32)
    w = random_weights(cfg, seed=3)
    good = TorchDecodeF64(cfg, w)
    base = [good.forward(t, p).numpy() for p, t in enumerate([5, 77, 901])]

    class SwappedGate(TorchDecodeF64):
        def forward(self, token, pos):
            for lw in self.layers:
                gu = lw['gate_up']
                lw['gate_up'] = torch.cat([gu[:, self.cfg.ffn:], gu[:, :self.cfg.ffn]], dim=1)
            try:
                return super().forward(token, pos)
            finally:
                for lw in self.layers:
                    gu = lw['gate_up']
                    lw['gate_up'] = torch.cat([gu[:, self.cfg.ffn:], gu[:, :self.cfg.ffn]], dim=1)

    class NoFinalNorm(TorchDecodeF64):
        def norm(self, x, w):
            return x if w is self.final_norm else super().norm(x, w)

    class InterleavedRope(TorchDecodeF64):
        def rope(self, x, pos):
            H, D = x.shape
            z = torch.view_as_complex(x.reshape(H, D // 2, 2).contiguous()) * torch.polar(torch.ones(D // 2, dtype=torch.float64), pos * self.inv_freq[:D // 2])
            return torch.view_as_real(z).reshape(H, D)

    for cls in (SwappedGate, NoFinalNorm, InterleavedRope):
        bad = cls(cfg, w)
        outs = [bad.forward(t, p).numpy() for p, t in enumerate([5, 77, 901])]
        assert max(np.abs(a - b).max() for a, b in zip(outs, base)) > 0.1, cls.__name__
