"""Exported operators: the callable objects behind ``autort.export`` and
``autort.ops.<name>``.

The calling convention follows the call sites of the reference's samples:
tensors are passed positionally in the order of the ``inputs=`` list
(samples/01_sort_even_first.py:22,27); a tensor of that list which the program
writes is updated in place; an output that is not in the list is allocated, or
taken from a trailing positional argument (samples/05_llama2_7b_int4.py:157) or
from ``out=`` (samples/05_llama2_7b_int4.py:144), and returned.  Outputs may be
views into larger tensors as long as the view itself is contiguous.  Kernels are
enqueued on torch's current stream and never synchronise.
"""
from __future__ import annotations

import hashlib
import os
from typing import Dict, List, Optional, Sequence

import torch

from ..ir import Graph, bake_small_reduce_extents, fuse_elementwise, pad_guarded_factors, parse_program, split_wide_reductions
from ..lower import contraction_slices, lower_graph
from ..runtime import capi

TORCH_DTYPE = {'float64': torch.float64, 'float32': torch.float32, 'float16': torch.float16,
               'int64': torch.int64, 'int32': torch.int32, 'int16': torch.int16, 'int8': torch.int8,
               'uint8': torch.uint8}
_COMPATIBLE = {('int8', torch.uint8), ('uint8', torch.int8)}     # same bits, reinterpreted

_CACHE_DIR = os.environ.get('AUTORT_CACHE_DIR') or os.path.join(
    os.path.dirname(os.path.dirname(os.path.abspath(__file__))), '_cache')


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def current_stream_handle(device_index: Optional[int] = None) -> int:
    """hipStream_t of torch's current stream (what a HIP graph capture records on).  The raw getter skips the
    Stream object torch.cuda.current_stream() builds on every call (about 2.5 us of an operator call)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device() if device_index is None else device_index)
    return torch.cuda.current_stream().cuda_stream


def compile_cached(source: str) -> bytes:
    """HIP source -> code object.  Code objects are cached on disk by the hash
    of their source, so a process only compiles what no earlier process has
    compiled.  Needs no GPU."""
    key = hashlib.sha256(source.encode()).hexdigest()[:24]
    path = os.path.join(_CACHE_DIR, key + '.hsaco')
    if os.path.exists(path):
        with open(path, 'rb') as f:
            image = f.read()
    else:
        image = capi.compile_hip(source)
        try:
            os.makedirs(_CACHE_DIR, exist_ok=True)
            tmp = f'{path}.tmp{os.getpid()}'
            with open(tmp, 'wb') as f:
                f.write(image)
            os.replace(tmp, path)
        except OSError:
            pass                     # a read-only tree only costs the recompilation next time
    return image


class ExportedOp:
    """One einstein_v2 program bound to gfx950 kernels."""

    def __init__(self, ir: str, inputs, config: Optional[str] = None, name: Optional[str] = None,
                 extra_outputs: Sequence[str] = (), tuned: Optional[Dict[str, object]] = None):
        self.ir = ir
        self.input_specs = list(inputs)
        self.config_text = config
        self.extra_outputs = list(extra_outputs)
        self.tuned: Dict[str, object] = dict(tuned or {})    # choices of a tuning run, keyed by kernel
        self.config = parse_config(config)
        self.graph: Graph = parse_program(ir, inputs, extra_outputs)
        self.fused: Graph = fuse_elementwise(self.graph)
        self.name = name or self.graph.outputs[-1]
        self.declared = list(self.graph.declared)
        self.inout = list(self.graph.inout)
        # outputs the caller does not pass among the declared tensors
        self.fresh_outputs = [o for o in self.graph.outputs if o not in self.declared]
        # what the generic lowering compiles: wide reductions with few outputs become two statements (statically
        # sized ones here; programs with named dimensions get a variant per set of values at call time)
        padded = pad_guarded_factors(self.fused)
        self.lowered: Graph = split_wide_reductions(padded, wanted=contraction_slices(padded.tensors))
        self.source, self.plans = lower_graph(self.lowered, prefix='autort_' + _ident(self.name))
        self._variants: Dict[tuple, dict] = {}
        self._module: Optional[capi.Module] = None
        self._image: Optional[bytes] = None
        from . import patterns
        hit = patterns.match(self.fused)
        # hand-written kernel for this program, if any, and which of the caller's tensors plays which part in it
        self.fast_path, self.fast_roles = hit if hit is not None else (None, {})
        # per-call bookkeeping that does not depend on the call
        self._wanted_dtype = {}
        for n in list(self.declared) + list(self.fresh_outputs):
            info = self.fused.tensors.get(n) or self.graph.tensors[n]
            self._wanted_dtype[n] = (TORCH_DTYPE[info.dtype], info.dtype)
        self._declared_in_graph = [n for n in self.declared if n in self.fused.tensors]
        self._shape_cache: Dict[tuple, tuple] = {}     # shapes of the declared tensors -> (dimension values, output shapes)

    # -- persistence ---------------------------------------------------------
    def persist(self) -> Optional[str]:
        """Writes the operator's module file (see store.py); returns its path, or
        None when the directory is not writable (the operator still works)."""
        from . import store
        try:
            return store.save(self.name, self.ir, self.input_specs, self.config_text, self.extra_outputs,
                              tuned=self.tuned, source=self.source)
        except OSError:
            return None

    # -- compilation ---------------------------------------------------------
    def compile(self) -> 'ExportedOp':
        """Builds the generic kernels (or finds them in the cache).  Needs no GPU."""
        if self._image is None:
            self._image = compile_cached(self.source)
        return self

    def _load(self) -> capi.Module:
        if self._module is None:
            self.compile()
            self._module = capi.Module(self._image)
        return self._module

    # -- calling -------------------------------------------------------------
    def __call__(self, *tensors, extra=None, out=None):
        g = self.fused
        nd = len(self.declared)
        if len(tensors) < nd:
            raise TypeError(f'{self.name}() takes {nd} tensor(s) {self.declared}, got {len(tensors)}')
        bound: Dict[str, torch.Tensor] = dict(zip(self.declared, tensors[:nd]))
        trailing = list(tensors[nd:])
        if len(trailing) > len(self.fresh_outputs):
            raise TypeError(f'{self.name}() got {len(tensors)} tensors but declares {nd} inputs and '
                            f'{len(self.fresh_outputs)} output(s)')
        for n, t in zip(self.fresh_outputs, trailing):
            bound[n] = t
        if out is not None:
            if not self.fresh_outputs:
                raise TypeError(f'{self.name}() has no separate output tensor to pass as out=')
            bound[self.fresh_outputs[-1]] = out
        dev = None
        for n, t in bound.items():
            self._check_tensor(n, t)
            dev = dev or t.device
        if dev is None:
            dev = torch.device('cuda', torch.cuda.current_device())
        if dev.type != 'cuda':
            raise RuntimeError(f'{self.name}(): tensors must live on the GPU (got {dev}); there is no CPU fallback')
        # dimension values and output shapes depend on the shapes of the declared tensors only: worked out once per
        # combination of shapes (a decode loop calls with the same shapes every time)
        key = tuple([bound[n].shape for n in self._declared_in_graph])
        hit = self._shape_cache.get(key)
        if hit is None:
            env = g.bind_dims({n: tuple(bound[n].shape) for n in self._declared_in_graph})
            hit = (env, {n: g.shape_of(n, env) for n in self.fresh_outputs})
            if len(self._shape_cache) < 64:
                self._shape_cache[key] = hit
        env, wants = hit
        for n in self.fresh_outputs:
            want = wants[n]
            if n in bound:
                if bound[n].numel() != _numel(want):
                    raise ValueError(f'output `{n}` expects {want} ({_numel(want)} elements), got {list(bound[n].shape)}')
            else:
                bound[n] = torch.empty(want, dtype=self._wanted_dtype[n][0], device=dev)
        capi.init(dev.index or 0)
        stream = current_stream_handle(dev.index)
        if self.fast_path is None or not self.fast_path(self, bound, env, stream):
            self._run_generic(bound, env, dev, stream)
        outs = [bound[o] for o in self.graph.outputs]
        return outs[0] if len(outs) == 1 else tuple(outs)

    def _check_tensor(self, name: str, t: torch.Tensor):
        if not isinstance(t, torch.Tensor):
            raise TypeError(f'argument `{name}` must be a torch.Tensor, got {type(t).__name__}')
        want, ir_dtype = self._wanted_dtype[name]
        if t.dtype != want and (ir_dtype, t.dtype) not in _COMPATIBLE:
            raise TypeError(f'tensor `{name}` must be {ir_dtype}, got {t.dtype}')
        if not t.is_contiguous():
            raise ValueError(f'tensor `{name}` must be contiguous (views are fine if they are dense)')

    def _variant(self, env: Dict[str, int]) -> dict:
        """Graph, plans and module for these values of the named dimensions: the default ones, unless a reduction
        of the program is worth slicing at these sizes (split_wide_reductions), runs over a window of a few elements
        given by named dimensions (bake_small_reduce_extents) or multiplies a zero-padded operand
        (pad_guarded_factors), which need their own kernels."""
        key = tuple(env[d] for d in self.fused.dim_names)
        v = self._variants.get(key)
        if v is not None and len(self._variants) > 1:
            self._variants[key] = self._variants.pop(key)      # most recently used last
        if v is None:
            # rows that one row kernel reduces and maps in a single launch are not sliced
            in_rows = any(p.row_group is not None and p.row_group.choose(env, {n: 0 for n in p.row_group.args})[1] for p in self.plans)
            g = bake_small_reduce_extents(self.lowered, env) if self.fused.dims else self.lowered
            g = pad_guarded_factors(g, env) if self.fused.dims else g
            g = split_wide_reductions(g, env, wanted=contraction_slices(g.tensors)) if self.fused.dims and not in_rows else g
            if g is not self.lowered:      # kernels of this call's own anyway: every reduce extent a constant (divisions by constants)
                g = bake_small_reduce_extents(g, env, limit=1 << 30)
            if g is self.lowered:
                v = {'graph': self.lowered, 'plans': self.plans, 'module': None, 'source': None}
            else:
                source, plans = lower_graph(g, prefix='autort_' + _ident(self.name) + '_s' + '_'.join(str(k) for k in key))
                v = {'graph': g, 'plans': plans, 'module': None, 'source': source}
            if len(self._variants) >= 64:          # the set of values used longest ago goes; its code object stays loaded
                self._variants.pop(next(iter(self._variants)))      # (capi.shared_module) and is found again by its text
            self._variants[key] = v
        if v['module'] is None:
            v['module'] = self._load() if v['source'] is None else capi.shared_module(compile_cached(v['source']))
        return v

    def plans_for(self, env: Dict[str, int]) -> list:
        """The kernel plans (one per statement of the lowered graph) that a call with these values of the named
        dimensions launches from."""
        return self._variant(env)['plans']

    def _run_generic(self, bound: Dict[str, torch.Tensor], env: Dict[str, int], dev, stream: int):
        variant = self._variant(env)
        module, g, plans_ = variant['module'], variant['graph'], variant['plans']
        dims = [env[d] for d in g.dim_names]
        trials = self.config.get('tune')
        trials = trials if isinstance(trials, int) and trials > 0 else 0
        skip = 0
        for plan in plans_:
            if skip:                       # computed by the row kernel of an earlier statement
                skip -= 1
                continue
            group = plan.row_group
            if group is not None:
                for n in group.args:
                    if n not in bound:
                        bound[n] = torch.empty(g.shape_of(n, env), dtype=TORCH_DTYPE[g.tensors[n].dtype], device=dev)
                sym, grid = group.choose(env, {n: bound[n].data_ptr() for n in group.args})
                if grid:
                    capi.launch(module.function(sym), (grid, 1, 1), (256, 1, 1), stream, [bound[n].data_ptr() for n in group.args] + dims)
                    skip = group.count - 1
                    continue
            for n in plan.args:
                if n not in bound:         # intermediate (reduce result) of a multi-kernel program
                    bound[n] = torch.empty(g.shape_of(n, env), dtype=TORCH_DTYPE[g.tensors[n].dtype], device=dev)
            ptrs = {n: bound[n].data_ptr() for n in plan.args}
            key = plan.name + '|' + ','.join(str(v) for v in dims) + '|' + ''.join('a' if ptrs[n] % 16 == 0 else 'u' for n in plan.args)
            saved = self.tuned.get(key)
            if saved is None and trials and not torch.cuda.is_current_stream_capturing():
                saved = self._tune(plan, key, bound, dims, ptrs, env, module, trials)
            if saved is not None and saved['variant'] in plan.variants:
                sym, grid, block = plan.variants[saved['variant']], int(saved['grid']), 256
            else:
                sym, grid, block = plan.choose(env, ptrs)
            skip = plan.covers - 1         # a map applied at this reduction's stores
            if grid == 0:
                continue
            capi.launch(module.function(sym), (grid, 1, 1), (block, 1, 1), stream,
                        [ptrs[n] for n in plan.args] + dims)

    def _tune(self, plan, key: str, bound, dims, ptrs, env, module, trials: int):
        """``config="tune:N"``: times up to N launch configurations of one kernel for the extents of this call
        (the reference searches its schedule space with OpEvo, tuner/OpEvo/main.py:467-616, N steps at a time;
        the space here is small - kernel variant x grid size - so the walk is: the heuristic choice first, then
        its neighbours, best first).  Written tensors are replaced by scratch copies while timing, so programs
        that accumulate into their output are not disturbed.  The winner is kept in the module file."""
        cands = plan.candidates(env, ptrs)
        if len(cands) <= 1:
            return None
        base_sym, base_grid, _ = plan.choose(env, ptrs)
        cands.sort(key=lambda c: (c[1] != base_sym, abs(c[2] - base_grid)))      # heuristic first, then nearest
        # Timed on rotating copies of the tensors (up to 512 MiB in all): one buffer launched over and over would
        # be served by the 256 MiB memory-side cache and favour configurations that do not stream well.
        per_launch = sum(bound[n].numel() * bound[n].element_size() for n in plan.args)
        copies = max(1, min(8, (512 << 20) // max(per_launch, 1)))
        sets, keep = [], []
        for c in range(copies):
            scratch = {n: (torch.empty_like(bound[n]) if n == plan.output or n in self.inout else (bound[n] if c == 0 else bound[n].clone()))
                       for n in plan.args}
            keep.append(scratch)                                                  # the copies live until the timing is over
            sets.append([scratch[n].data_ptr() for n in plan.args] + dims)
        stream = current_stream_handle()
        best = None
        for tag, sym, grid in cands[:trials]:
            fn = module.function(sym)
            capi.launch(fn, (grid, 1, 1), (256, 1, 1), stream, sets[0])           # warm-up
            start, stop = capi.Event(), capi.Event()
            start.record(stream)
            runs = max(5, copies)
            for i in range(runs):
                capi.launch(fn, (grid, 1, 1), (256, 1, 1), stream, sets[i % copies])
            stop.record(stream)
            us = start.elapsed_ms(stop) * 1e3 / runs
            if best is None or us < best['us']:
                best = {'variant': tag, 'grid': grid, 'us': round(us, 3)}
        del keep            # elapsed_ms waited for the last launch: nothing reads the copies any more
        self.tuned[key] = best
        self.persist()
        return best

    def __repr__(self):
        return f'<autort op {self.name}: {" ".join(self.ir.split())[:80]}>'


def parse_config(config: Optional[str]) -> Dict[str, object]:
    """Tuning hints such as ``"tune:5"`` or ``"~N~:[256,8,32],~S~:[64,8]"``
    (README.md:66, samples/05_llama2_7b_int4.py:139).  The grammar is not
    documented; unknown keys are kept verbatim and never rejected."""
    out: Dict[str, object] = {}
    if not config:
        return out
    depth, cur, parts = 0, '', []
    for ch in config:
        if ch in '[(':
            depth += 1
        elif ch in '])':
            depth -= 1
        if ch == ',' and depth == 0:
            parts.append(cur)
            cur = ''
        else:
            cur += ch
    if cur.strip():
        parts.append(cur)
    for p in parts:
        k, _, v = p.partition(':')
        k, v = k.strip(), v.strip()
        if not k:
            continue
        try:
            import json
            out[k] = json.loads(v)
        except Exception:
            out[k] = v
    return out


def _ident(name: str) -> str:
    return ''.join(c if c.isalnum() else '_' for c in name)


def _numel(shape) -> int:
    n = 1
    for s in shape:
        n *= s
    return n
