"""TEST INFRASTRUCTURE ONLY — CPU oracle.  Only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may use this module; the shipped GPU path never
imports it.

Restates what the reference's multi-thread CPU backend (c-mcpu) computes for an
einstein_v2 program: every statement becomes the plain loop nest that
AntaresIR.md:6-67 prescribes — initialise the output with the identity of the
reduce operator, then accumulate over the reduce axes in the r-value's dtype,
then store with a cast to the output dtype (antares/default_codegen.py:105-141).
Kernels use the CPU kernel ABI ``extern "C" void f(const int __rank__, void**
__args)`` with tensors first (inputs sorted by name, then outputs sorted by
name) and named run-time dimensions as trailing integer-valued slots
(backends/c-scpu/config.py:22-49, lang/generic.py:53-54), and the text is packed
in the evaluator's container format with ``// GLOBALS`` / ``// LOCAL`` /
``// [thread_extent]`` headers (antares/antares_compiler.py:183-232) so that the
reference's own evaluator binary can run it as well.

Indexing is row-major over the declared extents (as in the reference's direct
C emitter, backends/c-ipu/config.py:38-42).  Each ``__rank__`` computes one
contiguous slice of the flattened output space.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

CTYPE = {'float64': 'double', 'float32': 'float', 'float16': 'half', 'int64': 'long long', 'int32': 'int',
         'int16': 'short', 'int8': 'signed char', 'uint8': 'unsigned char'}

import os as _os

with open(_os.path.join(_os.path.dirname(_os.path.abspath(__file__)), 'ref_half.h')) as _f:
    _HALF_H = _f.read().replace('#pragma once', '')

# ref_half.h is pasted in rather than #included: the reference's evaluator
# compiles kernel text from a temporary directory.
PRELUDE = r'''
#include <math.h>
#include <stdint.h>
#include <algorithm>
''' + _HALF_H + r'''
#define rsqrt(x)  (1.0f / sqrt(x))
template <class T, class U> static inline T bitwise_and(T a, U b) { return (T)(a & (T)b); }
template <class T, class U> static inline T bitwise_or(T a, U b) { return (T)(a | (T)b); }
template <class T, class U> static inline T bitwise_xor(T a, U b) { return (T)(a ^ (T)b); }
static inline float normcdf(float x) { return 0.5f * erfcf(-x * 0.70710678118654752440f); }
static inline double normcdf(double x) { return 0.5 * erfc(-x * 0.70710678118654752440); }
static inline half fp16_exp(half x) { return half(expf((float)x)); }
static inline half fp16_log(half x) { return half(logf((float)x)); }
static inline half fp16_sqrt(half x) { return half(sqrtf((float)x)); }
static inline half fp16_rsqrt(half x) { return half(1.0f / sqrtf((float)x)); }
static inline half fp16_sin(half x) { return half(sinf((float)x)); }
static inline half fp16_cos(half x) { return half(cosf((float)x)); }
static inline half fp16_floor(half x) { return half(floorf((float)x)); }
static inline half fp16_ceil(half x) { return half(ceilf((float)x)); }
static inline half fp16_max(half a, half b) { return (float)a < (float)b ? b : a; }
static inline half fp16_min(half a, half b) { return (float)b < (float)a ? b : a; }
'''

# identity of every reduce operator (antares/default_codegen.py:113-128)
def reduce_identity(op: str, dtype: str) -> str:
    ct = CTYPE[dtype]
    if op == '+' or op == '|':
        return f'({ct})0'
    if op == '*' or op == '&':
        return f'({ct})1'
    lim = {'float64': '1.7976931348623157e308', 'float32': '3.402823466e38f', 'float16': '65504.0f',
           'int64': '9223372036854775807LL', 'int32': '2147483647', 'int16': '32767', 'int8': '127', 'uint8': '255'}[dtype]
    low = {'int64': '(-9223372036854775807LL-1)', 'int32': '(-2147483647-1)', 'int16': '-32768', 'int8': '-128',
           'uint8': '0'}.get(dtype, '-' + lim)
    if op == '>':
        return f'({ct})({low})'
    if op == '<':
        return f'({ct})({lim})'
    raise ValueError(f'unknown reduce operator {op}')


def _dim(d) -> str:
    # run-time dimensions live in their own name space: an axis may share its name
    return str(d) if isinstance(d, int) else f'__dim_{d}'


def _const(value, dtype: str) -> str:
    if dtype == 'float32':
        return repr(float(value)) + 'f'
    if dtype == 'float64':
        return repr(float(value))
    if dtype == 'float16':
        return f'half({float(value)!r}f)'
    return f'(({CTYPE[dtype]}){int(value)})'


class _Emit:
    def __init__(self, tensors):
        self.tensors = tensors

    def offset(self, name: str, idx: List[str]) -> str:
        shape = self.tensors[name].shape
        terms = []
        for i, ix in enumerate(idx):
            stride = ' * '.join(f'(long long){_dim(d)}' for d in shape[i + 1:])
            terms.append(f'({ix}) * {stride}' if stride else f'({ix})')
        return ' + '.join(terms) if terms else '0'

    def expr(self, n) -> str:
        k = n.kind
        ct = CTYPE[n.dtype]
        if k == 'const':
            return _const(n.value, n.dtype)
        if k == 'axis':
            return n.name
        if k == 'axis_range':
            return f'__ext_{n.name}'
        if k == 'dim':
            return _dim(n.value)
        if k == 'load':
            return f'{n.name}[{self.offset(n.name, [self.expr(a) for a in n.args])}]'
        if k == 'cast':
            return f'(({ct})({self.expr(n.args[0])}))'
        if k == 'op':
            if n.name == '~':
                return f'(({ct})(!({self.expr(n.args[0])})))'
            a, b = self.expr(n.args[0]), self.expr(n.args[1])
            sym = {'//': '/', '&': '&&', '|': '||'}.get(n.name, n.name)
            return f'(({ct})({a} {sym} {b}))'
        if k == 'call':
            args = ', '.join(self.expr(a) for a in n.args)
            fn = {'max': 'std::max', 'min': 'std::min'}.get(n.name, n.name)
            return f'(({ct}){fn}({args}))'
        if k == 'when':
            rel = ' && ' if n.merge == 'all' else ' || '
            cond = rel.join(f'({self.expr(c)})' for c in n.conds) or '1'
            if len(n.args) == 1:
                raise ValueError('one-armed when() is only valid at the root of a statement')
            return f'(({cond}) ? ({self.expr(n.args[0])}) : ({self.expr(n.args[1])}))'
        raise ValueError(f'unhandled node kind {k}')


def _combine(op: str, acc: str, val: str, dtype: str) -> str:
    ct = CTYPE[dtype]
    if op == '+':
        return f'{acc} = ({ct})({acc} + {val});'
    if op == '*':
        return f'{acc} = ({ct})({acc} * {val});'
    if op == '>':
        return f'{{ {ct} __v = {val}; if ({acc} < __v) {acc} = __v; }}'
    if op == '<':
        return f'{{ {ct} __v = {val}; if (__v < {acc}) {acc} = __v; }}'
    if op == '|':
        return f'{acc} = ({ct})(({acc} != 0) || ({val} != 0));'
    if op == '&':
        return f'{acc} = ({ct})(({acc} != 0) && ({val} != 0));'
    raise ValueError(op)


def emit_statement(st, graph, kernel_name: str, args: List[str], nranks: int) -> str:
    """One CPU kernel for one statement.  ``args`` is the tensor ABI order of
    this kernel; named dimensions follow in sorted order."""
    em = _Emit(graph.tensors)
    lines: List[str] = []
    for i, name in enumerate(args):
        ct = CTYPE[graph.tensors[name].dtype]
        lines.append(f'  {ct}* __restrict {name} = ({ct}*)__args[{i}];')
    for j, d in enumerate(graph.dim_names):
        lines.append(f'  const int {_dim(d)} = *(int*)&__args[{len(args) + j}]; (void){_dim(d)};')
    for ax, ext in st.data_axes + st.reduce_axes:
        lines.append(f'  const int __ext_{ax} = {_dim(ext)}; (void)__ext_{ax};')
    total = ' * '.join(f'(long long)__ext_{ax}' for ax, _ in st.data_axes) or '1LL'
    lines.append(f'  const long long __total = {total};')
    lines.append(f'  const long long __begin = __total * __rank__ / {nranks}, __end = __total * (__rank__ + 1) / {nranks};')
    lines.append('  for (long long __i = __begin; __i < __end; ++__i) {')
    # decompose the flat index into the data axes (last axis fastest)
    lines.append('    long long __r = __i;')
    for ax, _ in reversed(st.data_axes):
        lines.append(f'    const int {ax} = (int)(__r % __ext_{ax}); __r /= __ext_{ax};')
    root = st.root
    cond = None
    if root.kind == 'when' and len(root.args) == 1:
        rel = ' && ' if root.merge == 'all' else ' || '
        cond = rel.join(f'({em.expr(c)})' for c in root.conds)
        root = root.args[0]
    oct_ = CTYPE[st.out_dtype]
    dst = f'{st.output}[{em.offset(st.output, [em.expr(i) for i in st.out_index])}]'
    ind = '    '
    if st.reduce_axes:
        act = CTYPE[root.dtype]
        lines.append(f'{ind}{act} __acc = {reduce_identity(st.reduce, root.dtype)};')
        for ax, _ in st.reduce_axes:
            lines.append(f'{ind}for (int {ax} = 0; {ax} < __ext_{ax}; ++{ax}) {{')
            ind += '  '
        lines.append(f'{ind}{_combine(st.reduce, "__acc", em.expr(root), root.dtype)}')
        for _ in st.reduce_axes:
            ind = ind[:-2]
            lines.append(f'{ind}}}')
        value = '__acc'
    else:
        value = em.expr(root)
    store = {None: f'{dst} = ({oct_})({value});', 'set': f'{dst} = ({oct_})({value});',
             'add': f'{dst} = ({oct_})({dst} + ({oct_})({value}));',
             'min': f'{{ {oct_} __v = ({oct_})({value}); if (__v < {dst}) {dst} = __v; }}',
             'max': f'{{ {oct_} __v = ({oct_})({value}); if ({dst} < __v) {dst} = __v; }}'}[st.set_op]
    if st.reduce and not st.reduce_axes:
        # a reduce operator without reduce axes degenerates to a plain store
        pass
    lines.append(f'{ind}if ({cond}) {{ {store} }}' if cond else f'{ind}{store}')
    lines.append('  }')
    body = '\n'.join(lines)
    return (f'extern "C" void {kernel_name}(const int __rank__, void** __args) {{\n'
            f'  // [thread_extent] __rank__ = {nranks}\n{body}\n}}\n')


def _display(name: str, graph, env: Dict[str, int]) -> str:
    t = graph.tensors[name]
    shape = [d if isinstance(d, int) else env[d] for d in t.shape]
    return f'{name}:{t.dtype}{shape}'


def emit_module(graph, nranks: int = 64, env: Dict[str, int] = None) -> Tuple[str, List[dict]]:
    """Whole program -> (source text in evaluator container format, kernel table).

    Scatter statements run on one rank: the reference's semantics for colliding
    destinations are "last writer in loop order wins", which a single ordered
    loop reproduces deterministically.
    """
    from antares_amd.ir import fuse_elementwise
    g = fuse_elementwise(graph)
    env = dict(env or {d: (v if v is not None else 1) for d, v in g.dims.items()})
    ins, outs = g.abi_inputs, g.abi_outputs
    head = '// GLOBALS: ' + ', '.join(_display(n, g, env) for n in ins) + ' -> ' + \
        ', '.join(_display(n, g, env) for n in outs) + '\n// BACKEND: c-mcpu (default)\n'
    if g.dims:
        head += '// VAMAP: ' + ','.join(f'{d}:{env[d]}' for d in g.dim_names) + '\n'
    head += f'// CONFIG: \n// COMPUTE_V1: - einstein_v2({g.source.strip()!r})\n'
    parts, kernels = [head + PRELUDE], []
    for i, st in enumerate(g.statements):
        name = f'template_op_kernel{i}'
        k_in = sorted(n for n in st.reads if n != st.output)
        last = i + 1 == len(g.statements)
        k_out = outs if last else [st.output]
        if st.output not in k_out:
            k_out = sorted(set(k_out) | {st.output})
        args = k_in + [o for o in k_out if o not in k_in]
        r = 1 if st.scatter else nranks
        src = emit_statement(st, g, name, args, r)
        parts.append(f'// LOCAL: {name} -- ' + ', '.join(_display(n, g, env) for n in k_in) + ' -> ' +
                     ', '.join(_display(n, g, env) for n in args[len(k_in):]) + '\n\n' + src)
        kernels.append({'name': name, 'args': args, 'nranks': r, 'output': st.output})
    sep = '\n// ---------------------------------------------------------------------------\n'
    return sep.join(parts), kernels
