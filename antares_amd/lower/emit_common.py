"""What every kernel family of the generic lowering shares: C spellings of types and constants, the expression
emitter, kernel signatures (the reference's HIP kernel ABI, backends/c-rocm/config.py:25-85: tensor pointers first, then
the named run-time dimensions as ``int``), and small helpers over index expressions."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

from ..ir.nodes import Expr, ITEMSIZE, walk


HIP_TYPE = {'float64': 'double', 'float32': 'float', 'float16': 'half_t', 'int64': 'long long', 'int32': 'int',
            'int16': 'short', 'int8': 'signed char', 'uint8': 'unsigned char'}

BLOCK = 256
MAX_GRID = 256 * 32       # 256 CUs, enough resident blocks each to hide HBM latency

_CALLS = {'max': 'art_max', 'min': 'art_min', 'abs': 'art_abs', 'rsqrt': 'art_rsqrt', 'normcdf': 'art_normcdf'}
_REDUCE_OP = {'+': 'OpAdd', '*': 'OpMul', '>': 'OpMax', '<': 'OpMin', '|': 'OpAny', '&': 'OpAll'}


def dim_c(d) -> str:
    return str(d) if isinstance(d, int) else f'__dim_{d}'


def reduce_identity(op: str, dtype: str) -> str:
    """Start value of each reduce operator (antares/default_codegen.py:113-128)."""
    ct = HIP_TYPE[dtype]
    if op in ('+', '|'):
        return f'({ct})0'
    if op in ('*', '&'):
        return f'({ct})1'
    hi = {'float64': '1.7976931348623157e308', 'float32': '3.402823466e38f', 'float16': '65504.0f',
          'int64': '9223372036854775807LL', 'int32': '2147483647', 'int16': '32767', 'int8': '127', 'uint8': '255'}[dtype]
    lo = {'int64': '(-9223372036854775807LL-1)', 'int32': '(-2147483647-1)', 'int16': '-32768', 'int8': '-128',
          'uint8': '0'}.get(dtype, '-' + hi)
    return f'({ct})({lo if op == ">" else hi})'


def const_c(value, dtype: str) -> str:
    if dtype == 'float32':
        return repr(float(value)) + 'f'
    if dtype == 'float64':
        return repr(float(value))
    if dtype == 'float16':
        return f'((half_t){float(value)!r}f)'
    return f'(({HIP_TYPE[dtype]}){int(value)})'


class ExprEmitter:
    """IR expression -> HIP C++ text.  ``load_override`` lets the vector kernels
    replace tensor loads by lanes of a register vector."""

    def __init__(self, tensors, load_override: Optional[Callable[[Expr], Optional[str]]] = None):
        self.tensors = tensors
        self.load_override = load_override

    def offset(self, name: str, idx: List[str]) -> str:
        shape = self.tensors[name].shape
        terms = []
        for i, ix in enumerate(idx):
            stride = ' * '.join(f'(long long){dim_c(d)}' for d in shape[i + 1:])
            terms.append(f'({ix}) * {stride}' if stride else f'({ix})')
        return ' + '.join(terms) if terms else '0'

    def expr(self, n: Expr) -> str:
        k, ct = n.kind, HIP_TYPE[n.dtype]
        if k == 'const':
            return const_c(n.value, n.dtype)
        if k == 'axis':
            return n.name
        if k == 'axis_range':
            return f'__ext_{n.name}'
        if k == 'dim':
            return dim_c(n.value)
        if k == 'load':
            if self.load_override is not None:
                o = self.load_override(n)
                if o is not None:
                    return o
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
            return f'(({ct}){_CALLS.get(n.name, n.name)}({args}))'
        if k == 'when':
            if len(n.args) == 1:
                raise ValueError('one-armed when() is only valid at the root of a statement')
            rel = ' && ' if n.merge == 'all' else ' || '
            cond = rel.join(f'({self.expr(c)})' for c in n.conds) or '1'
            return f'(({cond}) ? ({self.expr(n.args[0])}) : ({self.expr(n.args[1])}))'
        raise ValueError(f'unhandled node kind {k}')


def _signature(name: str, args: List[str], tensors, dims: List[str], written: List[str]) -> str:
    ps = []
    for a in args:
        ct = HIP_TYPE[tensors[a].dtype]
        ps.append(f'{ct}* __restrict__ {a}' if a in written else f'const {ct}* __restrict__ {a}')
    ps += [f'int {dim_c(d)}' for d in dims]
    return f'extern "C" __global__ __launch_bounds__({BLOCK}) void {name}({", ".join(ps)})'


def _extents(st) -> List[str]:
    return [f'  const int __ext_{ax} = {dim_c(e)}; (void)__ext_{ax};' for ax, e in st.data_axes + st.reduce_axes]


def _decompose(var: str, axes, indent: str, bound: Optional[str] = None, tmp: str = '__r') -> List[str]:
    """The axis values of flat position `var`, last axis fastest.  With `bound` (C text of an exclusive upper limit of
    `var`) the divisions are 32-bit whenever that limit fits: a 64-bit division by a run-time value costs this part
    some hundred instructions, and a thread-per-output kernel makes one per axis and output."""
    if bound is None or not axes:
        out = [f'{indent}long long {tmp} = {var};']
        for ax, _ in reversed(axes):
            out.append(f'{indent}const int {ax} = (int)({tmp} % __ext_{ax}); {tmp} /= __ext_{ax};')
        return out
    out = [f'{indent}int ' + ', '.join(ax for ax, _ in axes) + ';',
           f'{indent}if ({bound} <= 0x7fffffffLL) {{', f'{indent}  unsigned int {tmp} = (unsigned int)({var});']
    for ax, _ in reversed(axes):
        out.append(f'{indent}  {ax} = (int)({tmp} % (unsigned int)__ext_{ax}); {tmp} /= (unsigned int)__ext_{ax};')
    out += [f'{indent}}} else {{', f'{indent}  long long {tmp} = {var};']
    for ax, _ in reversed(axes):
        out.append(f'{indent}  {ax} = (int)({tmp} % __ext_{ax}); {tmp} /= __ext_{ax};')
    out.append(f'{indent}}}')
    out.append(indent + ' '.join(f'(void){ax};' for ax, _ in axes))
    return out


def _root_and_cond(st, em: ExprEmitter):
    root, cond = st.root, None
    if root.kind == 'when' and len(root.args) == 1:
        rel = ' && ' if root.merge == 'all' else ' || '
        cond = rel.join(f'({em.expr(c)})' for c in root.conds)
        root = root.args[0]
    return root, cond



def _axes_of(e: Expr) -> set:
    return {m.name for m in walk(e) if m.kind == 'axis'}


def _axes_of_all(load: Expr) -> set:
    return set().union(*[_axes_of(a) for a in load.args]) if load.args else set()


def _multiple_of(n: Expr, v: int, free_of: str) -> bool:
    """True when the integer expression is provably a multiple of v and does not involve axis `free_of`."""
    if any(m.kind == 'axis' and m.name == free_of for m in walk(n)):
        return False
    if n.kind == 'const':
        return isinstance(n.value, int) and n.value % v == 0
    if n.kind == 'op' and n.name == '*':
        return any(_multiple_of(a, v, free_of) for a in n.args)
    if n.kind == 'op' and n.name in ('+', '-') and len(n.args) == 2:
        return all(_multiple_of(a, v, free_of) for a in n.args)
    return False
