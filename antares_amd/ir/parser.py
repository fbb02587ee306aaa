"""Parser for einstein_v2 statements (legacy Antares syntax + the AutoRT dialect).

What is accepted follows the reference front-end (lang/einstein_v2.py:259-404,
519-578 and lang/generic.py:15-57) and the call sites of the AutoRT samples
(samples/01_sort_even_first.py:10-14, samples/05_llama2_7b_int4.py:135-139,
README.md:66).  How it is done differs: the r-value is parsed with Python's
``ast`` module and walked by a small interpreter, so no user text is ever
``eval``-ed, and tensor extents may stay symbolic (named run-time dimensions).
"""
from __future__ import annotations

import ast as pyast
import re
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from .nodes import (Dim, Expr, Typing, as_expr, cast, const, is_int_dtype, up_cast, walk, ITEMSIZE)


class IRSyntaxError(Exception):
    pass


@dataclass
class TensorInfo:
    dtype: str
    shape: List[Dim]


@dataclass
class Statement:
    output: str
    out_index: Tuple[Expr, ...]          # l-value index expressions
    root: Expr                           # r-value
    reduce: Optional[str]                # '+', '>', '<', '*', '|', '&' or None
    set_op: Optional[str]                # 'set' | 'add' | 'min' | 'max' for scatter statements
    data_axes: List[Tuple[str, Dim]]
    reduce_axes: List[Tuple[str, Dim]]
    out_dtype: str
    out_shape: List[Dim]
    scatter: bool
    reads: List[str] = field(default_factory=list)

    @property
    def axes(self) -> Dict[str, Dim]:
        return dict(self.data_axes + self.reduce_axes)


_AXIS_RE = re.compile(r'\b[A-Z][a-zA-Z0-9]*')
_STMT_START_RE = re.compile(r'^\s*[a-z_][A-Za-z0-9_]*\s*\[')
_REDUCE_CHARS = ('<', '>', '+', '*', '|', '&')
_SET_OPS = {'=.': 'set', '+=.': 'add', '<=.': 'min', '>=.': 'max'}


def find_axis_names(text: str) -> List[str]:
    """Upper-case-initial identifiers outside quoted strings, in order of first
    appearance (reference: lang/einstein_v2.py:259-269)."""
    seen, out = set(), []
    for i, section in enumerate(text.split('"')):
        if i % 2 == 1:
            continue
        for m in _AXIS_RE.finditer(section):
            w = m.group(0)
            if w not in seen:
                seen.add(w)
                out.append(w)
    return out


def split_where(text: str):
    """``expr where A in 8, B in n:16`` -> (expr, {A: 8, B: 'n'})
    (reference: lang/einstein_v2.py:272-294)."""
    at = text.rfind(' where ')
    ranges: Dict[str, Dim] = {}
    defaults: Dict[str, int] = {}
    if at < 0:
        return text, ranges, defaults
    desc, text = text[at + len(' where '):], text[:at]
    for item in desc.split(','):
        item = item.strip()
        if not item:
            continue
        if ' in ' not in item:
            raise IRSyntaxError(f'Bad range item in where clause: `{item}`')
        k, v = item.split(' in ')
        k, v = k.strip(), v.strip()
        if ':' in v:
            n, d = v.split(':')
            ranges[k] = n.strip()
            defaults[n.strip()] = int(d)
        else:
            ranges[k] = int(v)
    return text, ranges, defaults


def split_statements(program: str) -> List[str]:
    """Statements are separated by ';' or, in the AutoRT dialect, by newlines.
    A line that does not start like ``name[`` continues the previous one."""
    out: List[str] = []
    for piece in program.split(';'):
        cur = ''
        for line in piece.split('\n'):
            if not line.strip():
                continue
            if cur and _STMT_START_RE.match(line) and _balanced(cur):
                out.append(cur.strip())
                cur = line
            else:
                cur = (cur + ' ' + line.strip()) if cur else line
        if cur.strip():
            out.append(cur.strip())
    return out


def _balanced(s: str) -> bool:
    return s.count('(') == s.count(')') and s.count('[') == s.count(']')


def _top_level_assign(text: str) -> int:
    """Index of the first '=' that is outside any bracket pair and is not part
    of ``==``, ``!=``."""
    depth = 0
    for i, ch in enumerate(text):
        if ch in '([':
            depth += 1
        elif ch in ')]':
            depth -= 1
        elif ch == '=' and depth == 0:
            if text[i + 1:i + 2] == '=' or text[i - 1:i] in ('!', '='):
                continue
            return i
    raise IRSyntaxError(f'No assignment found in statement: `{text}`')


class _TensorRef:
    def __init__(self, name: str, info: TensorInfo):
        self.name, self.info = name, info


class _Strs:
    """``strs.exp`` -> 'exp' (reference call site: README.md:66)."""


class _Bound:
    def __init__(self, obj, attr):
        self.obj, self.attr = obj, attr


class _Interp:
    """Evaluates the Python-grammar r-value into IR nodes, in Python's own
    evaluation order so that axis extents are discovered at the same moments
    the reference discovers them."""

    def __init__(self, tensors: Dict[str, TensorInfo], ranges: Dict[str, Optional[Dim]]):
        self.tensors = tensors
        self.ranges = ranges
        self.reads: List[str] = []
        self.t = Typing(lambda name: self.ranges.get(name))

    # -- helpers ------------------------------------------------------------
    def _num(self, v):
        return isinstance(v, (int, float)) and not isinstance(v, bool)

    def _expr(self, v) -> Expr:
        if isinstance(v, Expr):
            return v
        if self._num(v):
            return const(v)
        if isinstance(v, _TensorRef):
            raise IRSyntaxError(f'Tensor `{v.name}` must be indexed before it is used in arithmetic')
        raise IRSyntaxError(f'Cannot use {v!r} as an expression')

    def ev(self, n):
        m = getattr(self, 'ev_' + type(n).__name__, None)
        if m is None:
            raise IRSyntaxError(f'Unsupported syntax in expression: {type(n).__name__}')
        return m(n)

    def ev_Expression(self, n):
        return self.ev(n.body)

    def ev_Constant(self, n):
        return n.value

    def ev_Name(self, n):
        name = n.id
        if name in self.ranges:
            return Expr('axis', 'int32', name=name)
        if name in self.tensors:
            return _TensorRef(name, self.tensors[name])
        if name == 'strs':
            return _Strs()
        if name in ('const', 'f_op', 'alter'):
            return _Bound(None, name)
        if name and name[0].isupper():
            raise IRSyntaxError(f'Unknown axis `{name}`')
        raise IRSyntaxError(f'Unknown tensor or function `{name}`')

    def ev_List(self, n):
        return [self.ev(e) for e in n.elts]

    ev_Tuple = ev_List

    def ev_UnaryOp(self, n):
        v = self.ev(n.operand)
        if isinstance(n.op, pyast.USub):
            return -v if self._num(v) else self.t.neg(self._expr(v))
        if isinstance(n.op, pyast.UAdd):
            return v
        if isinstance(n.op, pyast.Invert):
            return ~v if isinstance(v, int) else self.t.invert(self._expr(v))
        raise IRSyntaxError('Unsupported unary operator')

    def ev_BinOp(self, n):
        a, b = self.ev(n.left), self.ev(n.right)
        op = type(n.op)
        if self._num(a) and self._num(b):
            return {pyast.Add: lambda: a + b, pyast.Sub: lambda: a - b, pyast.Mult: lambda: a * b,
                    pyast.Div: lambda: a / b, pyast.FloorDiv: lambda: a // b, pyast.Mod: lambda: a % b,
                    pyast.Pow: lambda: a ** b, pyast.LShift: lambda: a << b, pyast.RShift: lambda: a >> b,
                    pyast.BitAnd: lambda: a & b, pyast.BitOr: lambda: a | b}[op]()
        a, b = self._expr(a), self._expr(b)
        t = self.t
        if op is pyast.Add:
            return t.add(a, b)
        if op is pyast.Sub:
            return t.sub(a, b)
        if op is pyast.Mult:
            return t.mul(a, b)
        if op in (pyast.Div, pyast.FloorDiv):
            return t.div(a, b)
        if op is pyast.Mod:
            return t.mod(a, b)
        if op is pyast.RShift:
            return t.shift('>>', a, b)
        if op is pyast.LShift:
            return t.shift('<<', a, b)
        if op is pyast.BitAnd:
            return t.logic('&', a, b)
        if op is pyast.BitOr:
            return t.logic('|', a, b)
        raise IRSyntaxError(f'Unsupported binary operator: {op.__name__}')

    def ev_Compare(self, n):
        if len(n.ops) != 1:
            raise IRSyntaxError('Chained comparisons are not supported')
        a, b = self.ev(n.left), self.ev(n.comparators[0])
        sym = {pyast.Lt: '<', pyast.LtE: '<=', pyast.Gt: '>', pyast.GtE: '>=', pyast.Eq: '==', pyast.NotEq: '!='}.get(type(n.ops[0]))
        if sym is None:
            raise IRSyntaxError('Unsupported comparison operator')
        return self.t.compare(sym, self._expr(a), self._expr(b))

    def ev_Subscript(self, n):
        base = self.ev(n.value)
        if not isinstance(base, _TensorRef):
            raise IRSyntaxError('The instance to access its dim values must be a tensor array.')
        idx = self.ev(n.slice)
        idx = idx if isinstance(idx, list) else [idx]
        shape = base.info.shape
        if len(idx) != len(shape):
            raise IRSyntaxError(f'Tensor `{base.name}` has {len(shape)} dimension(s) but is indexed with {len(idx)}')
        out = []
        for i, it in enumerate(idx):
            it = self._expr(it)
            if it.kind == 'axis' and self.ranges.get(it.name) is None:
                self.ranges[it.name] = shape[i]
            out.append(it)
        if base.name not in self.reads:
            self.reads.append(base.name)
        return Expr('load', base.info.dtype, name=base.name, args=tuple(out))

    def ev_Attribute(self, n):
        obj = self.ev(n.value)
        if isinstance(obj, _Strs):
            return n.attr
        return _Bound(obj, n.attr)

    def ev_Call(self, n):
        fn = self.ev(n.func)
        if not isinstance(fn, _Bound):
            raise IRSyntaxError('Only method calls and const()/f_op() are callable in an expression')
        args = [self.ev(a) for a in n.args]
        kwargs = {k.arg: self.ev(k.value) for k in n.keywords}
        return self._invoke(fn.obj, fn.attr, args, kwargs)

    # -- methods ------------------------------------------------------------
    def _dim_expr(self, d: Dim) -> Expr:
        return const(d) if isinstance(d, int) else Expr('dim', 'int32', value=d)

    def _invoke(self, obj, name, args, kw):
        t = self.t
        if obj is None:
            if name == 'const':
                dtype = kw.get('dtype', args[1] if len(args) > 1 else None)
                v = args[0]
                return cast(v, dtype) if isinstance(v, Expr) else const(v, dtype)
            if name == 'f_op':
                return t.call(self._expr(args[1]), args[0], args[2:])
            raise IRSyntaxError(f'`{name}` is not supported')
        if isinstance(obj, _TensorRef):
            if name == 'dtype':
                return obj.info.dtype
            if name in ('size', 'val'):
                return self._dim_expr(obj.info.shape[int(args[0])])
            raise IRSyntaxError(f'Unsupported tensor method `{name}`')
        if self._num(obj):
            obj = const(obj)
        if not isinstance(obj, Expr):
            raise IRSyntaxError(f'Cannot call `{name}` on {obj!r}')
        if name == 'call':
            others = args[1] if len(args) > 1 else kw.get('others', [])
            if not isinstance(others, (list, tuple)):
                others = [others]
            return t.call(obj, args[0], [self._expr(o) for o in others], kw.get('output_dtype', kw.get('dtype')))
        if name in ('cast', 'to'):
            return cast(obj, args[0])
        if name == 'like':
            return const(args[0], obj.dtype)
        if name == 'dtype':
            return obj.dtype
        if name == 'up_cast':
            return up_cast(obj)
        if name == 'val':
            if obj.kind != 'axis':
                raise IRSyntaxError('Only tensor/axis objects have val property')
            return Expr('axis_range', 'int32', name=obj.name)
        if name == 'when':
            conds = args[0]
            other = args[1] if len(args) > 1 else kw.get('other')
            other = None if other is None else self._expr(other)
            return t.when(obj, conds, other, kw.get('merge_op', 'all'))
        raise IRSyntaxError(f'Unsupported method `{name}`')


def parse_statement(text: str, tensors: Dict[str, TensorInfo], dim_defaults: Dict[str, Optional[int]]) -> Statement:
    text = text.strip().replace('`', '"').replace("'", '"').replace('=!', '=')
    text, ranges_in, defaults = split_where(text)
    for k, v in defaults.items():
        dim_defaults.setdefault(k, v)

    # axes of the where clause come first, in clause order, then the others in order of
    # appearance (the reference keeps the where clause's dict order and adds the rest)
    ranges: Dict[str, Optional[Dim]] = dict(ranges_in)
    for ax in find_axis_names(text):
        ranges.setdefault(ax, None)

    # legacy scatter spelling  ``out[idx..] =. value``  (reference: lang/einstein_v2.py:309-329)
    set_op = None
    m = re.search(r'(\+|<|>)?=\.', text)
    if m:
        set_op = _SET_OPS.get(m.group(0))
        if set_op is None:
            raise IRSyntaxError(f'Unimplemented set_op: `{m.group(0)}`')
        lval, rval, reduce = text[:m.start()].strip(), text[m.end():].strip(), None
    else:
        at = _top_level_assign(text)
        reduce = None
        if at > 0 and text[at - 1] != ' ':
            if text[at - 1] in _REDUCE_CHARS:
                reduce = text[at - 1]
                lval = text[:at - 1].strip()
            else:
                raise IRSyntaxError(f'Illegal reduce naming in equation near: `{text[:at + 1]}`')
        else:
            lval = text[:at].strip()
        rval = text[at + 1:].strip()

    # scalar tensors: ``name[]`` means ``name[0]`` (reference: lang/einstein_v2.py:331-339)
    lval = re.sub(r'\[ *\]', '[0]', lval)
    rval = re.sub(r'\[ *\]', '[0]', rval)

    if '[' not in lval or not lval.endswith(']'):
        raise IRSyntaxError(f'L-value must be an indexed tensor: `{lval}`')
    output = lval[:lval.index('[')].strip()
    if not re.match(r'^[a-z_][A-Za-z0-9_]*$', output):
        raise IRSyntaxError(f'Tensor variable name must start with lower case letter: {output}')

    interp = _Interp(tensors, ranges)

    def parse_py(src, what):
        try:
            return pyast.parse(src, mode='eval')
        except SyntaxError as e:
            raise IRSyntaxError(f'Cannot parse {what} `{src}`: {e.msg}') from None

    # l-value indices are evaluated first: they may fix axis extents
    # (``space[data[N] % 2, N] = 1`` takes N from data).
    lidx_src = lval[lval.index('[') + 1:-1]
    lidx_nodes = parse_py('[' + lidx_src + ']', 'l-value index')
    out_index: List[Expr] = []
    scalar_axis = None
    for el in lidx_nodes.body.elts:
        v = interp.ev(el)
        if isinstance(v, int) and v == 0 and not set_op:
            if scalar_axis is None:
                i = 0
                while f'I{i}' in ranges:
                    i += 1
                scalar_axis = f'I{i}'
                ranges[scalar_axis] = 1
            v = Expr('axis', 'int32', name=scalar_axis)
        out_index.append(interp._expr(v))

    plain = all(e.kind == 'axis' for e in out_index) and len({e.name for e in out_index}) == len(out_index)
    scatter = bool(set_op) or not plain
    lval_reads = list(interp.reads)

    root = interp.ev(parse_py(rval, 'expression'))
    root = interp._expr(root) if not isinstance(root, Expr) else root

    for ax, r in ranges.items():
        if r is None:
            raise IRSyntaxError(f'The range of axis `{ax}` is undetermined, please use `where` clause '
                                'to set the range explicitly.')

    if scatter:
        if output not in tensors:
            raise IRSyntaxError(f'Scatter target `{output}` must be a declared tensor')
        if reduce:
            raise IRSyntaxError('A scatter statement cannot carry a reduce operator; use `+=.`')
        info = tensors[output]
        if len(out_index) != len(info.shape):
            raise IRSyntaxError(f'Tensor `{output}` has {len(info.shape)} dimension(s) but is indexed with {len(out_index)}')
        data_axes = [(ax, ranges[ax]) for ax in ranges]
        reduce_axes: List[Tuple[str, Dim]] = []
        out_dtype, out_shape = info.dtype, list(info.shape)
        if root.kind == 'when' and len(root.args) == 1:
            root = Expr('when', out_dtype, args=(cast(root.args[0], out_dtype),), conds=root.conds, merge=root.merge)
        else:
            root = cast(root, out_dtype)
        set_op = set_op or 'set'
    else:
        names = [e.name for e in out_index]
        data_axes = [(ax, ranges[ax]) for ax in names]
        reduce_axes = [(ax, ranges[ax]) for ax in ranges if ax not in names]
        out_dtype = root.dtype
        out_shape = [r for _, r in data_axes]
        if reduce_axes and not reduce:
            raise IRSyntaxError(f'Axes {[a for a, _ in reduce_axes]} do not index the output of `{output}` '
                                'and no reduce operator is given')

    reads = lval_reads + [r for r in interp.reads if r not in lval_reads]
    return Statement(output=output, out_index=tuple(out_index), root=root, reduce=reduce, set_op=set_op,
                     data_axes=data_axes, reduce_axes=reduce_axes, out_dtype=out_dtype, out_shape=out_shape,
                     scatter=scatter, reads=reads)


def parse_tensor_spec(spec) -> Tuple[TensorInfo, Dict[str, Optional[int]]]:
    """``"float32[N:4096, 8, M]"`` or ``{"dtype":…, "shape":[…]}`` -> TensorInfo
    plus the named dimensions it introduces with their default extents
    (reference: lang/generic.py:16-33, lang/einstein_v2.py:524-535)."""
    dims: Dict[str, Optional[int]] = {}
    if isinstance(spec, str):
        s = spec.strip()
        if '[' not in s or not s.endswith(']'):
            raise IRSyntaxError(f'Bad tensor spec: `{spec}`')
        dtype, body = s[:-1].split('[', 1)
        items = [x.strip() for x in body.split(',') if x.strip()]
    else:
        dtype, items = spec['dtype'], list(spec['shape'])
    dtype = dtype.strip()
    if dtype not in ITEMSIZE:
        raise IRSyntaxError(f'Unknown dtype `{dtype}`')
    shape: List[Dim] = []
    for it in items:
        if isinstance(it, int):
            shape.append(it)
        elif re.match(r'^-?[0-9]+$', str(it)):
            shape.append(int(it))
        elif ':' in str(it):
            n, v = str(it).split(':')
            n = n.strip()
            if not re.match(r'^[A-Za-z_][A-Za-z0-9_]*$', n):
                raise IRSyntaxError(f'Invalid arg name setting: "{n}"')
            shape.append(n)
            dims[n] = int(v)
        else:
            n = str(it).strip()
            if not re.match(r'^[A-Za-z_][A-Za-z0-9_]*$', n):
                raise IRSyntaxError(f'Invalid dimension: "{n}"')
            shape.append(n)
            dims.setdefault(n, None)
    if not shape:
        shape = [1]
    return TensorInfo(dtype, shape), dims
