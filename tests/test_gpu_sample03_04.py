"""The decode steps of samples/03_llama_tiny.py (fp32, `rmsnorm_f32` + `rotate_f32`, attention spelled in torch)
and samples/04_llama2_7b_fp16.py (fp16, `rmsnorm_f16` on an fp32 copy of x, `rotary_f16`, `attention_f16`, the
linears through `torch.matmul(out=...)` into cache views) written the way the samples write them, on small random
models, against the same steps out of the CPU oracle's operators.  The linears are torch's in the samples too;
what is pinned here is that the operators take the samples' tensors as they come (views of the caches as outputs,
fp32 x with fp16 weights, `extra=[pos]`) and that a sequence of positions stays on the oracle's trajectory."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

LAYERS, HEADS, HEAD, HIDDEN, VOCAB, SEQ = 2, 4, 128, 1024, 512, 10
DIM = HEADS * HEAD


def make_model(seed, dtype):
    g = torch.Generator().manual_seed(seed)

    def w(rows, cols, scale):
        return (torch.randn(rows, cols, generator=g) * scale).to(dtype)
    m = {'embed': w(VOCAB, DIM, 0.5), 'classify': w(VOCAB, DIM, 0.05), 'rms_end': (1 + 0.1 * torch.randn(DIM, generator=g)).to(dtype),
         'layers': []}
    for _ in range(LAYERS):
        m['layers'].append({'rms_att': (1 + 0.1 * torch.randn(DIM, generator=g)).to(dtype),
                            'rms_ffn': (1 + 0.1 * torch.randn(DIM, generator=g)).to(dtype),
                            'q': w(DIM, DIM, 0.03), 'k': w(DIM, DIM, 0.03), 'v': w(DIM, DIM, 0.03), 'o': w(DIM, DIM, 0.03),
                            'f1': w(HIDDEN, DIM, 0.03), 'f3': w(HIDDEN, DIM, 0.03), 'f2': w(DIM, HIDDEN, 0.03)})
    return m


class OracleStep:
    """Both samples' steps out of the oracle's operators.  `half` rounds where the fp16 sample rounds: every linear
    (fp32 accumulation, fp16 result), every operator output, the residual stream."""

    def __init__(self, m, half, interleaved):
        from oracle import hot_ops
        self.ops, self.m, self.half, self.interleaved = hot_ops, m, half, interleaved
        self.dt = np.float16 if half else np.float32
        self.key = np.zeros((LAYERS, SEQ + 2, DIM), self.dt)
        self.val = np.zeros((LAYERS, SEQ + 2, DIM), self.dt)
        inv = 1.0 / (10000.0 ** (torch.arange(0, HEAD, 2).float() / HEAD))
        if half:
            inv = inv.half()                                   # samples/04:79 rounds the frequencies to fp16
        self.inv = torch.cat([inv, inv]).view(HEAD).numpy()
        # samples/03:60: one coefficient per pair over the whole hidden size
        self.coef = (1 / torch.pow(1e4, torch.arange(0, DIM, 2, dtype=torch.int64) % HEAD / HEAD)).view(1, -1).float().numpy()

    def linear(self, x, w):
        return (x.astype(np.float32) @ w.numpy().astype(np.float32).T).astype(self.dt)

    def norm(self, x, w):
        xf = x.astype(np.float32)
        vsum = np.array([(xf * xf).sum(dtype=np.float32)], np.float32)
        return self.ops.rmsnorm(xf, vsum, w.numpy(), 1.0 / x.size, 1e-5, self.dt)

    def rope(self, t, pos):
        if self.interleaved:
            return self.ops.rotate(self.coef, t, pos)
        return self.ops.rotary(t.reshape(HEADS, 2, -1), self.inv, pos).reshape(-1)

    def forward(self, token, pos):
        x = self.m['embed'][token].numpy().copy()
        for l, lw in enumerate(self.m['layers']):
            xb = self.norm(x, lw['rms_att'])
            self.val[l, pos] = self.linear(xb, lw['v'])
            q = self.rope(self.linear(xb, lw['q']), pos)
            self.key[l, pos] = self.rope(self.linear(xb, lw['k']), pos)
            att = self.ops.attention(q.reshape(HEADS, HEAD), self.key[l, :pos + 1].reshape(pos + 1, HEADS, HEAD),
                                     self.val[l, :pos + 1].reshape(pos + 1, HEADS, HEAD), 1 / math.sqrt(HEAD))
            x = (x + self.linear(att.reshape(-1), lw['o'])).astype(self.dt)
            xb = self.norm(x, lw['rms_ffn'])
            gate, up = self.linear(xb, lw['f1']).astype(np.float32), self.linear(xb, lw['f3'])
            hb = (gate / (1 + np.exp(-gate))).astype(self.dt) * up
            x = (x + self.linear(hb.astype(self.dt), lw['f2'])).astype(self.dt)
        return self.linear(self.norm(x, self.m['rms_end']), self.m['classify']).astype(np.float32)


def _to_device(m, device):
    out = {k: v.to(device) for k, v in m.items() if k != 'layers'}
    out['layers'] = [{k: v.to(device) for k, v in lw.items()} for lw in m['layers']]
    return out


def _run(forward, ref, tol):
    token = 3
    with torch.no_grad():
        for pos in range(SEQ):
            print(f'[case] sample step pos={pos} token={token}', flush=True)
            want = ref.forward(token, pos)
            got = forward(token, pos).float().cpu().numpy().reshape(-1)
            assert np.allclose(got, want, rtol=tol, atol=tol), (pos, np.abs(got - want).max())
            token = int(np.argmax(want))


def test_tiny_llama_step_as_sample_03_writes_it(oracle_built):
    """samples/03_llama_tiny.py:62-113: fp32, interleaved-pair rotation over the whole hidden vector."""
    import autort
    device = autort.device()
    m = make_model(11, torch.float32)
    d = _to_device(m, device)
    key_cache = torch.zeros([LAYERS, SEQ + 2, DIM], dtype=torch.float32, device=device)
    val_cache = torch.zeros_like(key_cache)
    ceof = (1 / torch.pow(1e4, torch.arange(0, DIM, 2, dtype=torch.int64) % HEAD / HEAD)).view(1, -1).float().to(device)
    att_f = torch.tensor([1 / math.sqrt(HEAD)], dtype=torch.float32, device=device)

    def rmsnorm(x, weight):
        x = x.float()
        vsum = (x * x).sum()
        return autort.ops.rmsnorm_f32(x.view(-1), vsum, weight, extra=[1.0 / int(x.numel())])

    def rotate(data, ceof, pos, out):
        autort.ops.rotate_f32(ceof, data.view(-1), out.view(-1), extra=[pos, ])
        return out

    def forward(token, pos):
        x = d['embed'].select(0, token).view(1, DIM)
        for l in range(LAYERS):
            lw = d['layers'][l]
            xb = rmsnorm(x, lw['rms_att']).view(1, DIM)
            sq = torch.matmul(xb, lw['q'].t())
            sk = torch.matmul(xb, lw['k'].t())
            sv = val_cache.select(0, l).narrow(0, pos, 1)
            torch.matmul(xb, lw['v'].t(), out=sv)
            sq_out = torch.empty_like(sq)
            sk_out = key_cache.select(0, l).narrow(0, pos, 1)
            rotate(sq, ceof, pos, out=sq_out)
            rotate(sk, ceof, pos, out=sk_out)
            b_sq = sq_out.view(HEADS, HEAD)
            b_sk = key_cache.select(0, l).view(SEQ + 2, HEADS, HEAD).narrow(0, 0, pos + 1)
            att = torch.nn.functional.softmax(torch.einsum('hm,shm->hs', b_sq, b_sk) * att_f, dim=-1)
            b_sv = val_cache.select(0, l).view(SEQ + 2, HEADS, HEAD).narrow(0, 0, pos + 1)
            xb = torch.einsum('hs,shm->hm', att, b_sv).reshape(1, DIM)
            x = x + torch.matmul(xb, lw['o'].t())
            xb = rmsnorm(x, lw['rms_ffn']).view(1, DIM)
            hb = torch.nn.functional.silu(torch.matmul(xb, lw['f1'].t())) * torch.matmul(xb, lw['f3'].t())
            x = x + torch.matmul(hb, lw['f2'].t())
        x = rmsnorm(x, d['rms_end']).view(1, DIM)
        return torch.matmul(x, d['classify'].t())

    _run(forward, OracleStep(m, half=False, interleaved=True), 2e-4)


def test_fp16_llama_step_as_sample_04_writes_it(oracle_built):
    """samples/04_llama2_7b_fp16.py:84-116: fp16 weights and caches, the fused v|q|k projection written into three
    rows of the value cache, rmsnorm_f16 fed an fp32 copy of x, fp16-rounded frequencies."""
    import autort
    device = autort.device()
    m = make_model(12, torch.float16)
    d = _to_device(m, device)
    vqk = [torch.cat([lw['v'], lw['q'], lw['k']]) for lw in d['layers']]
    key_cache = torch.zeros([LAYERS, SEQ + 2, DIM], dtype=torch.float16, device=device)
    val_cache = torch.zeros([LAYERS, SEQ + 2, DIM], dtype=torch.float16, device=device)
    att_f = torch.tensor([1 / math.sqrt(HEAD)], dtype=torch.float32, device=device)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, HEAD, 2).float() / HEAD)).half())
    inv_freq = torch.cat([inv_freq, inv_freq]).view(HEAD).to(device)

    def rmsnorm(x, weight):
        x = x.float()
        vsum = (x * x).sum().view(1)
        return autort.ops.rmsnorm_f16(x.view(-1), vsum, weight, extra=[1.0 / int(x.numel())])

    def forward(token, pos):
        x = d['embed'].select(0, token).view(1, DIM)
        for l in range(LAYERS):
            lw = d['layers'][l]
            xb = rmsnorm(x, lw['rms_att']).view(1, DIM)
            local_cache = val_cache.select(0, l).narrow(0, pos, 3)
            torch.matmul(xb, vqk[l].t(), out=local_cache.view(-1, 3 * xb.size(-1)))
            sq, sk = local_cache[1], local_cache[2]
            sq_out = torch.empty_like(sq).view(HEADS, HEAD)
            sk_out = key_cache.select(0, l).narrow(0, pos, 1).view(HEADS, HEAD)
            autort.ops.rotary_f16(sq.view(HEADS, 2, -1), inv_freq, sq_out, extra=[pos, ])
            autort.ops.rotary_f16(sk.view(HEADS, 2, -1), inv_freq, sk_out, extra=[pos, ])
            b_sk = key_cache.select(0, l).view(SEQ + 2, HEADS, HEAD).narrow(0, 0, pos + 1)
            b_sv = val_cache.select(0, l).view(SEQ + 2, HEADS, HEAD).narrow(0, 0, pos + 1)
            xb = autort.ops.attention_f16(sq_out, b_sk, b_sv, att_f)
            x = x + torch.matmul(xb.view(1, DIM), lw['o'].t())
            xb = rmsnorm(x, lw['rms_ffn']).view(1, DIM)
            xb = torch.nn.functional.silu(torch.matmul(xb, lw['f1'].t())) * torch.matmul(xb, lw['f3'].t())
            x = x + torch.matmul(xb, lw['f2'].t())
        x = rmsnorm(x, d['rms_end']).view(1, DIM)
        return torch.matmul(x, d['classify'].t())

    _run(forward, OracleStep(m, half=True, interleaved=False), 2e-2)
