"""Llama-2-shaped int4 decode driven through ``autort.ops`` — the host-side glue of
the reference's samples/05_llama2_7b_int4.py:109-200 for the benchmark
configuration: every linear layer in the packed int4 group-128 format with
per-group zero points, fp16 embeddings / norm weights / activations / KV cache,
batch 1, one token per step.

Differences from the sample's ``forward`` that do not change results:
* the sum of squares of RMSNorm is computed inside the operator (``vsum=None``);
* q, k, v are projected into a scratch vector; k is rotated straight into its
  cache row and v copied into its row by kernels that read the position from a
  1-element device tensor, so one recorded HIP graph serves every position;
* residual add, SiLU*up and the embedding row select are einstein_v2 programs
  exported through ``autort.export`` (the sample uses torch ops for them).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from . import workloads
from .autort import patterns


@dataclass
class LlamaConfig:
    n_layers: int = 32
    dim: int = 4096
    n_heads: int = 32
    ffn: int = 11008
    vocab: int = 32000
    max_seq: int = 384
    rms_eps: float = 1e-5
    rope_base: float = 10000.0

    @property
    def head_dim(self) -> int:
        return self.dim // self.n_heads

    def weight_bytes_per_token(self) -> int:
        """Bytes of packed weights, scales and zero points one decode step streams."""
        per_layer = sum(workloads.w4_bytes(0, k, n) for k, n in self.layer_shapes())
        return self.n_layers * per_layer + workloads.w4_bytes(0, self.dim, self.vocab)

    def layer_shapes(self):
        return [(self.dim, 3 * self.dim), (self.dim, self.dim), (self.dim, 2 * self.ffn), (self.ffn, self.dim)]


def random_int4_linear(gen: torch.Generator, K: int, N: int) -> Dict[str, torch.Tensor]:
    """Packed weights drawn directly as bytes: a uniform byte is two independent uniform nibbles."""
    qweight = torch.empty(K // 2, N, dtype=torch.uint8).random_(0, 256, generator=gen)
    qzeros = torch.empty(K // 128, N // 2, dtype=torch.uint8).random_(0, 256, generator=gen)
    scales = (torch.rand(K // 128, N, generator=gen, dtype=torch.float32) * 0.019 + 0.001).to(torch.float16)
    return {'qweight': qweight, 'qzeros': qzeros, 'scales': scales}


def random_weights(cfg: LlamaConfig, seed: int = 0) -> Dict[str, object]:
    """Random-init weights of the architecture on the CPU (one generator per matrix,
    seeded from ``seed``), so the GPU path and the CPU oracle share bits."""
    def g(i):
        return torch.Generator().manual_seed(seed * 100003 + i)
    w: Dict[str, object] = {
        'embed': (torch.randn(cfg.vocab, cfg.dim, generator=g(1)) * 0.02).to(torch.float16),
        'final_norm': (1 + 0.1 * torch.randn(cfg.dim, generator=g(2))).to(torch.float16),
        'lm_head': random_int4_linear(g(3), cfg.dim, cfg.vocab),
        'layers': [],
    }
    for l in range(cfg.n_layers):
        base = 1000 + 10 * l
        w['layers'].append({
            'att_norm': (1 + 0.1 * torch.randn(cfg.dim, generator=g(base))).to(torch.float16),
            'ffn_norm': (1 + 0.1 * torch.randn(cfg.dim, generator=g(base + 1))).to(torch.float16),
            'qkv': random_int4_linear(g(base + 2), cfg.dim, 3 * cfg.dim),          # columns: q | k | v
            'o': random_int4_linear(g(base + 3), cfg.dim, cfg.dim),
            'gate_up': random_int4_linear(g(base + 4), cfg.dim, 2 * cfg.ffn),      # columns: gate | up
            'down': random_int4_linear(g(base + 5), cfg.ffn, cfg.dim),
        })
    return w


def _to_device(obj, dev):
    if isinstance(obj, torch.Tensor):
        return obj.to(dev)
    if isinstance(obj, dict):
        return {k: _to_device(v, dev) for k, v in obj.items()}
    if isinstance(obj, list):
        return [_to_device(v, dev) for v in obj]
    return obj


class LlamaInt4Decoder:
    """One-token-per-step decoder.  ``step()`` enqueues a whole forward pass on the
    current stream; ``capture()`` records it once in a HIP graph."""

    def __init__(self, cfg: LlamaConfig, weights: Dict[str, object], device=None, fused: bool = True, att_parts: int = 8,
                 packed: Optional[bool] = None):
        """``packed`` (default: with ``fused``): the projections whose input needs no merging (q|k|v, gate|up, down,
        lm_head) run over weights repacked once here (``autort.ops.w4_prepack``, the counterpart of the sample's
        load-time repacking, samples/05_llama2_7b_int4.py:34-66) with ``autort.ops.gemv_w4p``: one block per 16
        columns over all of K, no K-splits.  The benchmark-format tensors stay for the o-projection (which merges the
        split attention's records while it loads x) and for the batched passes of ``prefill``."""
        import autort
        self.fused = fused
        self.packed = fused if packed is None else bool(packed)
        if self.packed and not fused:
            raise ValueError('the packed projections come with the fused decoder')
        self.att_parts = att_parts if fused else 1     # blocks per head in the decode attention (1 = unsplit)
        self.autort = autort
        self.cfg = cfg
        self.dev = device or autort.device()
        self.w = _to_device(weights, self.dev)
        d, H, D = cfg.dim, cfg.n_heads, cfg.head_dim
        f16 = dict(dtype=torch.float16, device=self.dev)
        self.key_cache = torch.zeros(cfg.n_layers, cfg.max_seq, d, **f16)
        self.val_cache = torch.zeros(cfg.n_layers, cfg.max_seq, d, **f16)
        inv = (1.0 / (cfg.rope_base ** (torch.arange(0, D, 2).float() / D))).to(torch.float16)
        self.inv_freq = torch.cat([inv, inv]).view(D).to(self.dev)
        self.att_f = torch.tensor([1 / math.sqrt(D)], dtype=torch.float32, device=self.dev)
        # sum(x^2) of the residual stream, handed from the projection that writes it to the one that normalises it
        # (the packed projections own all of K and sum the squares of x themselves)
        self.hand_sumsq = fused and d <= 8192 and not self.packed
        self.sumsq = torch.zeros(2, 256, dtype=torch.int64, device=self.dev)
        # device-side step state
        self.token = torch.zeros(1, dtype=torch.int32, device=self.dev)
        self.pos = torch.zeros(1, dtype=torch.int32, device=self.dev)
        # activations (fixed addresses: the step can be recorded in a graph)
        self.x = torch.empty(d, **f16)
        self.xb = torch.empty(d, **f16)
        self.qkv = torch.empty(3 * d, **f16)
        self.q_rot = torch.empty(H, D, **f16)
        self.att_partial = torch.zeros(H, max(self.att_parts, 2), 132, dtype=torch.float32, device=self.dev)
        self.att = torch.empty(H, D, **f16)
        self.proj = torch.empty(d, **f16)
        self.gu = torch.empty(2 * cfg.ffn, **f16)
        self.hb = torch.empty(cfg.ffn, **f16)
        self.logits = torch.empty(cfg.vocab, **f16)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self._prefill_cache: Dict[int, Dict[str, object]] = {}      # prompt length -> operators of `prefill`
        self._prefill_graphs: Dict[int, tuple] = {}                  # prompt length -> (recorded pass, its token buffer)
        self._stream: Optional[torch.cuda.Stream] = None             # the one side stream recordings are made on
        self._ops()
        self.pw: Dict[str, object] = {}
        if self.packed:
            self._prepack()

    def _prepack(self):
        """One-time repacking of the matrices the packed GEMV reads; gate and up are interleaved in blocks of 8
        columns first, so that a block of the GEMV holds matching gate / up columns and can apply SwiGLU itself."""
        from .autort.builtin_ops import interleave_gate_up
        pack = self.autort.ops.w4_prepack
        F = self.cfg.ffn

        def packed(lin):
            return pack(lin['qweight'], lin['scales'], lin['qzeros'])
        layers = []
        for lw in self.w['layers']:
            gu = lw['gate_up']
            gate = {'qweight': gu['qweight'][:, :F].contiguous(), 'scales': gu['scales'][:, :F].contiguous(),
                    'qzeros': gu['qzeros'][:, :F // 2].contiguous()}
            up = {'qweight': gu['qweight'][:, F:].contiguous(), 'scales': gu['scales'][:, F:].contiguous(),
                  'qzeros': gu['qzeros'][:, F // 2:].contiguous()}
            layers.append({'qkv': packed(lw['qkv']), 'gate_up': packed(interleave_gate_up(gate, up)), 'down': packed(lw['down']),
                           'o': packed(lw['o'])})      # used when the attention runs as one block per head
        self.pw = {'layers': layers, 'lm_head': packed(self.w['lm_head'])}

    def _ops(self):
        a = self.autort
        self.gemv = a.export(ir=patterns.W4A16_IR, inputs=patterns.W4A16_INPUTS, name='gemv_w4a16')
        self.embed = a.export(ir='emb[D] = table[tok[0], D]', inputs=['table=float16[V, D]', 'tok=int32[1]'], name='embed_row_f16')
        self.add = a.export(ir='acc[N] = acc[N] + delta[N]', inputs=['acc=float16[N]', 'delta=float16[N]'], name='residual_add_f16')
        self.silu_mul = a.export(
            ir='hidden[N] = (gu[0, N].to(`float32`) / (1.0 + (0.0 - gu[0, N].to(`float32`)).call(strs.exp)) * gu[1, N].to(`float32`)).to(`float16`)',
            inputs=['gu=float16[2, N]'], name='silu_mul_f16')
        self.store_row = a.export(ir='cache[pos[0], D] = row[D]', inputs=['cache=float16[S, D]', 'pos=int32[1]', 'row=float16[D]'],
                                  name='store_row_f16')

    def _linear(self, x: torch.Tensor, lin: Dict[str, torch.Tensor], out: torch.Tensor):
        self.gemv(x.view(1, -1), lin['qweight'], lin['scales'], lin['qzeros'], out=out.view(1, -1))

    def step(self, embed: bool = True) -> torch.Tensor:
        """Forward pass for (self.token, self.pos); leaves fp16 logits in self.logits.  ``embed=False`` skips the
        embedding lookup: self.x already holds the row (the fused ``advance`` leaves it there)."""
        return self.step_fused(embed) if self.fused else self.step_plain()

    def step_fused(self, embed: bool = True) -> torch.Tensor:
        """Five launches per layer: RMSNorm, SwiGLU and the residual adds ride inside the projections; rotary of
        q and k and both cache writes ride inside the attention.  Same roundings as ``step_plain``."""
        cfg, ops = self.cfg, self.autort.ops
        H, D = cfg.n_heads, cfg.head_dim
        gemv = ops.gemv_w4a16_fused
        if embed:
            self.embed(self.w['embed'], self.token, out=self.x)
        if self.packed:
            return self._step_packed()
        # The projections that write the residual stream (o, down) leave sum(x^2) of what they wrote in a buffer, and the
        # projection that normalises the stream next reads it there instead of re-reading x in every block.  Two
        # buffers alternate: a writer adds into one and zeroes the other for the writer after it.  Only the first
        # projection of a step computes its own sum (its x is an embedding row).
        after_o, after_down = self.sumsq if self.hand_sumsq else (None, None)
        for l, lw in enumerate(self.w['layers']):
            a, o, gu, dn = lw['qkv'], lw['o'], lw['gate_up'], lw['down']
            gemv(self.x, a['qweight'], a['scales'], a['qzeros'], self.qkv, norm_weight=lw['att_norm'], eps=cfg.rms_eps,
                 sumsq_in=after_down if l > 0 else None)
            if self.att_parts > 1:      # attention over several blocks per head, merged by the o-projection as it loads x
                ops.attention_rope_split_f16(self.qkv, self.inv_freq, self.key_cache[l], self.val_cache[l], self.att_f,
                                             self.att_partial, extra=[self.pos])
                ops.gemv_w4a16_attn(self.att_partial, o['qweight'], o['scales'], o['qzeros'], self.x, residual=self.x,
                                    sumsq_out=after_o, sumsq_clear=after_down)
            else:
                ops.attention_rope_f16(self.qkv, self.inv_freq, self.key_cache[l], self.val_cache[l], self.att_f, self.att,
                                       extra=[self.pos])
                gemv(self.att.view(-1), o['qweight'], o['scales'], o['qzeros'], self.x, residual=self.x,
                     sumsq_out=after_o, sumsq_clear=after_down)
            gemv(self.x, gu['qweight'], gu['scales'], gu['qzeros'], self.gu, norm_weight=lw['ffn_norm'], eps=cfg.rms_eps,
                 sumsq_in=after_o)
            gemv(self.gu, dn['qweight'], dn['scales'], dn['qzeros'], self.x, residual=self.x, swiglu=True,
                 sumsq_out=after_down, sumsq_clear=after_o)
        h = self.w['lm_head']
        gemv(self.x, h['qweight'], h['scales'], h['qzeros'], self.logits, norm_weight=self.w['final_norm'], eps=cfg.rms_eps,
             sumsq_in=after_down)
        return self.logits

    def _step_packed(self) -> torch.Tensor:
        """The fused step over repacked weights: q|k|v (RMSNorm folded in), attention, o (merge + residual, benchmark
        layout), gate|up (RMSNorm in, SwiGLU out), down (residual), five launches per layer."""
        cfg, ops = self.cfg, self.autort.ops
        d, F = cfg.dim, cfg.ffn
        gemv = ops.gemv_w4p
        for l, (lw, pw) in enumerate(zip(self.w['layers'], self.pw['layers'])):
            o = lw['o']
            gemv(self.x, pw['qkv'], self.qkv, norm_weight=lw['att_norm'], eps=cfg.rms_eps, shape=(d, 3 * d))
            if self.att_parts > 1:
                ops.attention_rope_split_f16(self.qkv, self.inv_freq, self.key_cache[l], self.val_cache[l], self.att_f,
                                             self.att_partial, extra=[self.pos])
                ops.gemv_w4a16_attn(self.att_partial, o['qweight'], o['scales'], o['qzeros'], self.x, residual=self.x)
            else:
                ops.attention_rope_f16(self.qkv, self.inv_freq, self.key_cache[l], self.val_cache[l], self.att_f, self.att,
                                       extra=[self.pos])
                gemv(self.att.view(-1), pw['o'], self.x, residual=self.x, shape=(d, d))
            gemv(self.x, pw['gate_up'], self.hb, norm_weight=lw['ffn_norm'], eps=cfg.rms_eps, swiglu_out=True, shape=(d, 2 * F))
            gemv(self.hb, pw['down'], self.x, residual=self.x, shape=(F, d))
        gemv(self.x, self.pw['lm_head'], self.logits, norm_weight=self.w['final_norm'], eps=cfg.rms_eps, shape=(d, cfg.vocab))
        return self.logits

    def step_plain(self) -> torch.Tensor:
        """One launch per operator of the sample's forward pass (thirteen per layer)."""
        cfg, ops = self.cfg, self.autort.ops
        d, H, D = cfg.dim, cfg.n_heads, cfg.head_dim
        self.embed(self.w['embed'], self.token, out=self.x)
        for l, lw in enumerate(self.w['layers']):
            ops.rmsnorm_f16(self.x, None, lw['att_norm'], self.xb, extra=[1.0 / d, cfg.rms_eps])
            self._linear(self.xb, lw['qkv'], self.qkv)
            q, k, v = self.qkv[:d], self.qkv[d:2 * d], self.qkv[2 * d:]
            ops.rotary_f16(q.view(H, 2, -1), self.inv_freq, self.q_rot, extra=[self.pos])
            ops.rotary_f16(k.view(H, 2, -1), self.inv_freq, self.key_cache[l], extra=[self.pos])
            self.store_row(self.val_cache[l], self.pos, v)
            ops.attention_f16(self.q_rot, self.key_cache[l].view(cfg.max_seq, H, D), self.val_cache[l].view(cfg.max_seq, H, D),
                              self.att_f, self.att, extra=[self.pos])
            self._linear(self.att.view(-1), lw['o'], self.proj)
            self.add(self.x, self.proj)
            ops.rmsnorm_f16(self.x, None, lw['ffn_norm'], self.xb, extra=[1.0 / d, cfg.rms_eps])
            self._linear(self.xb, lw['gate_up'], self.gu)
            self.silu_mul(self.gu.view(2, -1), out=self.hb)
            self._linear(self.hb, lw['down'], self.proj)
            self.add(self.x, self.proj)
        ops.rmsnorm_f16(self.x, None, self.w['final_norm'], self.xb, extra=[1.0 / d, cfg.rms_eps])
        self._linear(self.xb, self.w['lm_head'], self.logits)
        return self.logits

    # -- whole-prompt ingestion ------------------------------------------------
    def _prefill_ops(self, T: int):
        """Operators of `prefill` for a prompt of T tokens: einstein_v2 programs at static sizes (compiled once per
        T and kept in the code-object cache) around the batched int4 projections."""
        ops = self._prefill_cache.get(T)
        if ops is not None:
            return ops
        from .autort.op import ExportedOp

        def program(ir, inputs, name):
            # the operator autort.export would make, but neither listed in autort.ops nor written to a module file:
            # there is one set of these per prompt length
            return ExportedOp(ir, list(inputs), name=name)
        cfg = self.cfg
        d, H, D, F, V = cfg.dim, cfg.n_heads, cfg.head_dim, cfg.ffn, cfg.vocab
        f32 = '.to(`float32`)'
        ops = {
            'embed': program(ir='emb[T, D] = table[tok[T], D]', inputs=[f'table=float16[{V}, {d}]', f'tok=int32[{T}]'],
                              name=f'prefill_embed_{T}'),
            'silu_mul': program(
                ir=f'hid[T, N] = (gu[T, N]{f32} / (1.0 + (0.0 - gu[T, N]{f32}).call(`exp`)) * gu[T, {F} + N]{f32}).to(`float16`) where N in {F}',
                inputs=[f'gu=float16[{T}, {2 * F}]'], name=f'prefill_silu_mul_{T}'),
        }
        self._prefill_cache[T] = ops
        return ops

    def prefill(self, tokens: torch.Tensor, graph: bool = True) -> torch.Tensor:
        """Ingests a whole prompt (int32 [T] on the device, T >= 4, positions 0..T-1) in one pass: the projections
        run as batched int4 GEMMs on the matrix cores (`gemv_w4a16` with T rows), attention is causal over the
        prompt (`attention_causal_f16`, matrix cores), keys and values land in cache rows 0..T-1.  Leaves the step
        state at the last prompt position (self.pos = T - 1, self.x = its hidden state, self.logits = its logits), so
        `advance()` and the recorded decode step continue from there.  Same operators and roundings as the one-token
        step, applied to T rows.  With ``graph`` the pass is recorded once per prompt length in a HIP graph (about 420
        launches) and replayed on later calls with the new tokens copied into the recorded input."""
        T = int(tokens.numel())
        if not 4 <= T <= self.cfg.max_seq:
            raise ValueError(f'prefill takes 4..{self.cfg.max_seq} tokens, got {T}')
        if not graph or torch.cuda.is_current_stream_capturing():
            return self._prefill_eager(tokens)
        rec = self._prefill_graphs.get(T)
        if rec is None:
            static_tokens = tokens.view(T).clone()
            stream = self._side_stream()
            stream.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(stream):
                self._prefill_eager(static_tokens)          # loads every module and workspace outside the capture
                stream.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    self._prefill_eager(static_tokens)
            torch.cuda.current_stream().wait_stream(stream)
            rec = self._prefill_graphs[T] = (g, static_tokens)
        g, static_tokens = rec
        static_tokens.copy_(tokens.view(T))
        g.replay()
        return self.logits

    def _side_stream(self):
        if self._stream is None:
            self._stream = torch.cuda.Stream()
        return self._stream

    def _prefill_eager(self, tokens: torch.Tensor) -> torch.Tensor:
        cfg = self.cfg
        T = int(tokens.numel())
        d, H, D, F = cfg.dim, cfg.n_heads, cfg.head_dim, cfg.ffn
        ops = self._prefill_ops(T)
        f16 = dict(dtype=torch.float16, device=self.dev)
        x = ops['embed'](self.w['embed'], tokens.view(T))
        qkv = torch.empty(T, 3 * d, **f16)
        gu = torch.empty(T, 2 * F, **f16)
        qr = torch.empty(T, H, D, **f16)

        def linear(inp, lin, out):
            self.gemv(inp, lin['qweight'], lin['scales'], lin['qzeros'], out=out)

        def gemm_res(inp, lin, acc):    # acc += inp @ W, the residual add folded into the projection
            self.autort.ops.gemm_w4a16_residual(inp, lin['qweight'], lin['scales'], lin['qzeros'], acc, residual=acc)

        def rms(inp, weight):           # the built-in operator takes rows: one launch for the T positions
            return self.autort.ops.rmsnorm_f16(inp, None, weight, extra=[1.0 / d, cfg.rms_eps])

        for l, lw in enumerate(self.w['layers']):
            xb = rms(x, lw['att_norm'])
            linear(xb, lw['qkv'], qkv)
            self.autort.ops.rope_qkv_store_rows_f16(qkv, self.inv_freq, qr, self.key_cache[l], self.val_cache[l])
            att = self.autort.ops.attention_causal_f16(qr, self.key_cache[l].view(cfg.max_seq, H, D),
                                                       self.val_cache[l].view(cfg.max_seq, H, D), self.att_f)
            gemm_res(att.view(T, d), lw['o'], x)
            xb = rms(x, lw['ffn_norm'])
            linear(xb, lw['gate_up'], gu)
            hid = ops['silu_mul'](gu)
            gemm_res(hid, lw['down'], x)
        self.x.copy_(x[T - 1])
        self.pos.fill_(T - 1)
        self.token.copy_(tokens.view(T)[T - 1:T])
        h = self.w['lm_head']
        self.autort.ops.gemv_w4a16_fused(self.x, h['qweight'], h['scales'], h['qzeros'], self.logits,
                                         norm_weight=self.w['final_norm'], eps=cfg.rms_eps)
        return self.logits

    def tune_att_parts(self, pos: int, candidates=(8, 4, 2, 1), runs: int = 20) -> Dict[str, object]:
        """The decode attention's launch parameter - blocks per head - for a cache filled up to `pos`: times the
        attention + o-projection pair of every layer for each candidate and keeps the fastest in `self.att_parts`
        (call before `capture`; the caches are used as scratch only in row `pos`, which a real step rewrites)."""
        if not self.fused:
            raise RuntimeError('the unfused decoder has no split attention to tune')
        from .runtime import capi
        ops = self.autort.ops
        saved_pos = self.pos.clone()
        self.pos.fill_(pos)
        best = None
        stream = torch.cuda.current_stream().cuda_stream
        for parts in candidates:
            partial = torch.zeros(self.cfg.n_heads, max(parts, 2), 132, dtype=torch.float32, device=self.dev)

            def pair(l, lw):
                o = lw['o']
                if parts > 1:
                    ops.attention_rope_split_f16(self.qkv, self.inv_freq, self.key_cache[l], self.val_cache[l], self.att_f,
                                                 partial, extra=[self.pos])
                    ops.gemv_w4a16_attn(partial, o['qweight'], o['scales'], o['qzeros'], self.proj)
                else:
                    ops.attention_rope_f16(self.qkv, self.inv_freq, self.key_cache[l], self.val_cache[l], self.att_f, self.att,
                                           extra=[self.pos])
                    ops.gemv_w4a16_fused(self.att.view(-1), o['qweight'], o['scales'], o['qzeros'], self.proj)
            pair(0, self.w['layers'][0])
            start, stop = capi.Event(), capi.Event()
            start.record(stream)
            n = 0
            while n < runs:
                for l, lw in enumerate(self.w['layers']):
                    pair(l, lw)
                    n += 1
            stop.record(stream)
            us = start.elapsed_ms(stop) * 1e3 / n
            if best is None or us < best['us']:
                best = {'value': parts, 'us': round(us, 3)}
        self.pos.copy_(saved_pos)
        self.att_parts = best['value']
        self.att_partial = torch.zeros(self.cfg.n_heads, max(self.att_parts, 2), 132, dtype=torch.float32, device=self.dev)
        self.graph = None
        return best

    def advance(self, prompt: Optional[torch.Tensor] = None):
        """pos <- pos + 1; token <- prompt[pos] while the prompt lasts, else argmax(logits).
        All on the device, so it can be part of the recorded graph.  The fused decoder does it in one launch,
        which also leaves the embedding row of the new token in self.x."""
        if self.fused:
            self.autort.ops.greedy_next_f16(self.logits, prompt, self.token, self.pos, self.w['embed'], self.x)
            return
        nxt = torch.argmax(self.logits).to(torch.int32).view(1)
        self.pos.add_(1)
        if prompt is not None and prompt.numel() > 0:
            L = prompt.numel()
            idx = torch.clamp(self.pos, max=L - 1).long()
            nxt = torch.where(self.pos < L, prompt[idx], nxt)
        self.token.copy_(nxt)

    def capture(self, greedy: bool = True, prompt: Optional[torch.Tensor] = None):
        """Record one step (+ advance) in a HIP graph.  ``prompt`` (int32 on the device)
        is fed token by token before greedy decoding takes over."""
        stream = self._side_stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            self.step()                       # loads every module outside the capture
            stream.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                self.step(embed=not (greedy and self.fused))     # the fused advance has already fetched the row
                if greedy:
                    self.advance(prompt)
        torch.cuda.synchronize()
        self.graph = g
        return g

    def reset(self, token: int = 0, pos: int = 0):
        self.token.fill_(token)
        self.pos.fill_(pos)
        self.embed(self.w['embed'], self.token, out=self.x)      # a recorded greedy graph starts from self.x
