"""Expression nodes of the einstein_v2 tensor IR and its typing rules.

The node vocabulary (const, axis, axis_range, load, op, call, cast, when) and
the dtype promotion / algebraic simplification rules restate the behaviour of
the reference front-end's operator-overloading class
(reference: lang/einstein_v2.py:12-257).  The representation is our own: nodes
are immutable records built by an explicit interpreter over the Python grammar
(see parser.py) instead of objects mutated through ``eval``.
"""
from __future__ import annotations

import re
from dataclasses import dataclass, field
from typing import List, Optional, Tuple, Union

# Promotion order when two operand dtypes meet (reference:
# lang/einstein_v2.py:26-32).  ``uint8`` is an extension of this build used for
# packed 4-bit weights; it sits below every reference dtype so it never wins.
PROMOTION_ORDER = ['float64', 'float32', 'float16', 'int64', 'int32', 'int16', 'int8', 'uint8']

C_TYPES = {
    'float64': 'double', 'float32': 'float', 'float16': 'half',
    'int64': 'long long', 'int32': 'int', 'int16': 'short', 'int8': 'signed char',
    'uint8': 'unsigned char',
}

ITEMSIZE = {'float64': 8, 'float32': 4, 'float16': 2, 'int64': 8, 'int32': 4, 'int16': 2, 'int8': 1, 'uint8': 1}

Dim = Union[int, str]   # a static extent or the name of a run-time dimension


def is_int_dtype(dtype: str) -> bool:
    return re.match(r'^u?int[0-9]+$', dtype) is not None


def is_float_dtype(dtype: str) -> bool:
    return dtype.startswith('float')


def merge_dtype(a: str, b: str) -> str:
    for d in PROMOTION_ORDER:
        if d == a or d == b:
            return d
    return a


@dataclass(frozen=True)
class Expr:
    """One IR node.  ``kind`` selects which of the remaining fields are used.

    kind        fields
    ----------  ------------------------------------------------------------
    const       value (python int/float), dtype
    axis        name
    axis_range  name              (extent of an axis, ``AXIS.val()``)
    dim         value (Dim)       (extent of a tensor dimension, ``t.size(i)``)
    load        name (tensor), args (index expressions)
    op          name (operator symbol), args
    call        name (function), args
    cast        args[0]
    when        conds, args=(true, false) or (true,), merge ('all' | 'any')
    """
    kind: str
    dtype: str
    name: Optional[str] = None
    value: object = None
    args: Tuple['Expr', ...] = ()
    conds: Tuple['Expr', ...] = ()
    merge: str = 'all'

    def __repr__(self):
        from .printer import to_ir
        return f'<{self.dtype} {to_ir(self)}>'


def const(value, dtype: Optional[str] = None) -> Expr:
    if dtype is None:
        if isinstance(value, bool):
            value = int(value)
        if isinstance(value, int):
            dtype = 'int32'
        elif isinstance(value, float):
            dtype = 'float32'
        else:
            raise TypeError(f'Unrecognized const node type: {type(value)}')
    return Expr('const', dtype, value=value)


def as_expr(x, dtype: Optional[str] = None) -> Expr:
    """Python number or node -> node, optionally cast/typed to ``dtype``."""
    if isinstance(x, Expr):
        return cast(x, dtype)
    return const(x, dtype)


def cast(x: Expr, dtype: Optional[str]) -> Expr:
    if dtype is None or x.dtype == dtype:
        return x
    return Expr('cast', dtype, args=(x,))


def up_cast(x: Expr) -> Expr:
    if x.dtype in ('int8', 'int16', 'uint8'):
        return cast(x, 'int32')
    if x.dtype == 'float16':
        return cast(x, 'float32')
    return x


def _is_const(x: Expr, v) -> bool:
    return x.kind == 'const' and x.value == v


class Typing:
    """Typed constructors for binary/unary operators.

    ``axis_extent(name)`` must return the static extent of an axis if it is an
    integer known at this point of the statement, else None; it feeds the two
    axis simplifications (reference: lang/einstein_v2.py:95-100,120-127).
    """

    def __init__(self, axis_extent):
        self.axis_extent = axis_extent

    # arithmetic -----------------------------------------------------------
    def mul(self, a: Expr, b: Expr) -> Expr:
        out = merge_dtype(a.dtype, b.dtype)
        if _is_const(b, 1):
            return cast(a, out)
        if _is_const(a, 1):
            return cast(b, out)
        return Expr('op', out, name='*', args=(cast(a, out), cast(b, out)))

    def div(self, a: Expr, b: Expr) -> Expr:
        name = '//' if is_int_dtype(a.dtype) and is_int_dtype(b.dtype) else '/'
        out = merge_dtype(a.dtype, b.dtype)
        if _is_const(b, 1):
            return cast(a, out)
        if b.kind == 'const' and a.kind == 'axis' and name == '//':
            ext = self.axis_extent(a.name)
            if isinstance(ext, int) and ext <= b.value:
                return const(0, out)
        res = Expr('op', out, name=name, args=(a, b))
        if is_float_dtype(a.dtype) and is_int_dtype(b.dtype):
            res = cast(res, a.dtype)
        return res

    def mod(self, a: Expr, b: Expr) -> Expr:
        if b.kind == 'const':
            if b.dtype != 'int32':
                raise TypeError('The right operand of % must be an int32 constant')
            if b.value == 1:
                return const(0, a.dtype)
            if a.kind == 'axis':
                ext = self.axis_extent(a.name)
                if isinstance(ext, int) and ext <= b.value:
                    return a
        return Expr('op', a.dtype, name='%', args=(a, b))

    def add(self, a: Expr, b: Expr) -> Expr:
        out = merge_dtype(a.dtype, b.dtype)
        if _is_const(b, 0):
            return cast(a, out)
        if _is_const(a, 0):
            return cast(b, out)
        return Expr('op', out, name='+', args=(cast(a, out), cast(b, out)))

    def sub(self, a: Expr, b: Expr) -> Expr:
        out = merge_dtype(a.dtype, b.dtype)
        if _is_const(b, 0):
            return cast(a, out)
        return Expr('op', out, name='-', args=(cast(a, out), cast(b, out)))

    def shift(self, name: str, a: Expr, b: Expr) -> Expr:
        return Expr('op', a.dtype, name=name, args=(a, b))

    def neg(self, a: Expr) -> Expr:
        return self.sub(const(0, a.dtype), a)

    # relations / logic: always int8 (reference: lang/einstein_v2.py:166-200)
    def compare(self, name: str, a: Expr, b: Expr) -> Expr:
        if name == '>':
            name, a, b = '<', b, a
        elif name == '>=':
            name, a, b = '<=', b, a
        return Expr('op', 'int8', name=name, args=(a, b))

    def logic(self, name: str, a: Expr, b: Expr) -> Expr:
        return Expr('op', 'int8', name=name, args=(a, b))

    def invert(self, a: Expr) -> Expr:
        return Expr('op', 'int8', name='~', args=(a,))

    # calls ------------------------------------------------------------------
    def call(self, x: Expr, func: str, others=(), dtype: Optional[str] = None) -> Expr:
        """``x.call(func, others)`` with the reference's rewrites
        (reference: lang/einstein_v2.py:225-249)."""
        others = tuple(as_expr(o) for o in others)
        if func == 'sigmoid' and not others:
            # The reference spells this 1 / (exp(x) + 1); kept as is.
            return self.div(const(1), self.add(self.call(x, 'exp'), const(1)))
        if func == 'remainder' and not others:
            return self.sub(x, self.call(x, 'rfloor'))
        if func in ('floor', 'ceil') and not others:
            inner = Expr('call', x.dtype, name=func, args=(up_cast(x),))
            return cast(inner, 'int64' if x.dtype == 'float64' else 'int32')
        if func in ('rfloor', 'rceil') and not others:
            func = func[1:]
        if func in ('exp', 'sqrt', 'rsqrt', 'max', 'min', 'log', 'sin', 'cos', 'floor', 'ceil') \
                and x.dtype == 'float16':
            func = 'fp16_' + func
        if func in ('pow', 'abs', 'tan', 'tanh', 'normcdf', 'erf'):
            ups = tuple(up_cast(a) for a in (x,) + others)
            return cast(Expr('call', up_cast(x).dtype, name=func, args=ups), x.dtype)
        return Expr('call', dtype or x.dtype, name=func, args=(x,) + others)

    def when(self, x: Expr, conds, other=None, merge='all') -> Expr:
        conds = tuple(conds) if isinstance(conds, (list, tuple)) else (conds,)
        for c in conds:
            if not isinstance(c, Expr) or not is_int_dtype(c.dtype):
                raise TypeError('Each condition in a when() must be of integer type')
        if other is None:
            # one-argument form: a store that only happens when the condition
            # holds (reference: samples/01_sort_even_first.py:13)
            return Expr('when', x.dtype, args=(x,), conds=conds, merge=merge)
        other = as_expr(other)
        if x.dtype != other.dtype and '@' not in x.dtype and '@' not in other.dtype:
            raise TypeError('Conditional true and false values must have same datatype '
                            f'({x.dtype} v.s. {other.dtype})')
        return Expr('when', x.dtype, args=(x, other), conds=conds, merge=merge)


def walk(e: Expr):
    """Pre-order traversal over every node of an expression tree."""
    yield e
    for c in e.conds:
        yield from walk(c)
    for a in e.args:
        yield from walk(a)


def rewrite(e: Expr, fn) -> Expr:
    """Bottom-up rebuild; ``fn(node)`` returns a replacement or None."""
    args = tuple(rewrite(a, fn) for a in e.args)
    conds = tuple(rewrite(c, fn) for c in e.conds)
    if args != e.args or conds != e.conds:
        e = Expr(e.kind, e.dtype, name=e.name, value=e.value, args=args, conds=conds, merge=e.merge)
    r = fn(e)
    return e if r is None else r
