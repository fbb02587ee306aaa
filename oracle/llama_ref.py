"""TEST INFRASTRUCTURE ONLY — CPU oracle of the int4 Llama decode step.  Only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.

Restates the forward pass of samples/05_llama2_7b_int4.py:146-177 for the
benchmark configuration (packed int4 linears with zero points, fp16 everything
else) out of the oracle's own operators (hot_ops.c).  Every operator output is
rounded to fp16, as each GPU operator rounds its output.

Pinned by tests/test_oracle.py::test_decode_oracle_against_independent_float64_restatement:
ten positions against a torch float64 forward pass written from the sample's text
with library routines only (dense matmul, silu, softmax, rotate_half), logits,
greedy tokens and cache rows.
"""
from __future__ import annotations

import math

import numpy as np

from . import hot_ops


def _np(t):
    return t.numpy() if hasattr(t, 'numpy') else np.asarray(t)


class LlamaRef:
    def __init__(self, cfg, weights, linear=None):
        """``linear(x_fp16[1,K], lin) -> fp16[1,N]`` may be replaced (the threaded
        loop-nest module is used for the full-size timing run)."""
        self.cfg, self.w = cfg, weights
        d, D = cfg.dim, cfg.head_dim
        self.key_cache = np.zeros((cfg.n_layers, cfg.max_seq, d), np.float16)
        self.val_cache = np.zeros((cfg.n_layers, cfg.max_seq, d), np.float16)
        inv = (1.0 / (cfg.rope_base ** (np.arange(0, D, 2, dtype=np.float32) / np.float32(D)))).astype(np.float16)
        self.inv_freq = np.concatenate([inv, inv])
        self.att_f = np.float32(1 / math.sqrt(D))
        self.linear = linear or self._linear

    @staticmethod
    def _linear(x, lin):
        return hot_ops.gemm_w4a16(x, _np(lin['qweight']), _np(lin['scales']), _np(lin['qzeros']))

    def forward(self, token: int, pos: int) -> np.ndarray:
        cfg = self.cfg
        d, H, D = cfg.dim, cfg.n_heads, cfg.head_dim
        x = _np(self.w['embed'])[token].astype(np.float16)                                   # :147
        for l, lw in enumerate(self.w['layers']):
            xb = hot_ops.rmsnorm(x, None, _np(lw['att_norm']), 1.0 / d, cfg.rms_eps, np.float16)   # :150
            qkv = self.linear(xb.reshape(1, d), lw['qkv']).reshape(-1)                        # :151-152
            q, k, v = qkv[:d], qkv[d:2 * d], qkv[2 * d:]
            q_rot = hot_ops.rotary(q.reshape(H, 2, D // 2), self.inv_freq, pos)               # :157
            self.key_cache[l, pos] = hot_ops.rotary(k.reshape(H, 2, D // 2), self.inv_freq, pos).reshape(-1)   # :158
            self.val_cache[l, pos] = v
            ks = self.key_cache[l, :pos + 1].reshape(pos + 1, H, D)                           # :162-163
            vs = self.val_cache[l, :pos + 1].reshape(pos + 1, H, D)
            att = hot_ops.attention(q_rot, ks, vs, float(self.att_f))                         # :165
            x = (x + self.linear(att.reshape(1, d), lw['o']).reshape(-1)).astype(np.float16)  # :167-168
            xb = hot_ops.rmsnorm(x, None, _np(lw['ffn_norm']), 1.0 / d, cfg.rms_eps, np.float16)
            gu = self.linear(xb.reshape(1, d), lw['gate_up']).reshape(2, -1).astype(np.float32)
            hb = (gu[0] / (np.float32(1) + np.exp(-gu[0])) * gu[1]).astype(np.float16)        # silu(gate) * up, :171
            x = (x + self.linear(hb.reshape(1, -1), lw['down']).reshape(-1)).astype(np.float16)
        xb = hot_ops.rmsnorm(x, None, _np(self.w['final_norm']), 1.0 / d, cfg.rms_eps, np.float16)   # :175
        return self.linear(xb.reshape(1, d), self.w['lm_head']).reshape(-1)                   # :176
