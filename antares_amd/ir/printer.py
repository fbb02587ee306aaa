"""Text forms of IR nodes.

``to_ir`` prints an expression back in einstein_v2 syntax (the job of the
reference's reverse emitter, lang/einstein_v2.py:419-485).  ``canonical`` prints
a whole statement list with tensors and axes renamed by first appearance, which
gives a spelling-independent key for recognising known operator patterns.
"""
from __future__ import annotations

from .nodes import Expr


def to_ir(e: Expr, tensor_name=lambda n: n, axis_name=lambda n: n) -> str:
    def go(n: Expr) -> str:
        k = n.kind
        if k == 'const':
            return f'const({n.value!r})' if n.dtype in ('int32', 'float32') else f'const({n.value!r}, `{n.dtype}`)'
        if k == 'axis':
            return axis_name(n.name)
        if k == 'axis_range':
            return f'{axis_name(n.name)}.val()'
        if k == 'dim':
            return f'dim({n.value})'
        if k == 'load':
            return f'{tensor_name(n.name)}[{", ".join(go(a) for a in n.args)}]'
        if k == 'op':
            if len(n.args) == 1:
                return f'({n.name}{go(n.args[0])})'
            return f'({go(n.args[0])} {n.name} {go(n.args[1])})'
        if k == 'call':
            if len(n.args) == 1:
                return f'({go(n.args[0])}).call(`{n.name}`, dtype=`{n.dtype}`)'
            rest = ', '.join(go(a) for a in n.args[1:])
            return f'({go(n.args[0])}).call(`{n.name}`, [{rest}], dtype=`{n.dtype}`)'
        if k == 'cast':
            return f'({go(n.args[0])}).cast(`{n.dtype}`)'
        if k == 'when':
            conds = ', '.join(go(c) for c in n.conds)
            if len(n.args) == 1:
                return f'({go(n.args[0])}).when([{conds}], merge_op="{n.merge}")'
            return f'({go(n.args[0])}).when([{conds}], {go(n.args[1])}, merge_op="{n.merge}")'
        raise ValueError(f'unhandled node kind: {k}')
    return go(e)


def statement_to_ir(st, tensor_name=lambda n: n, axis_name=lambda n: n) -> str:
    lhs = ', '.join(to_ir(i, tensor_name, axis_name) for i in st.out_index)
    op = (st.reduce or '') + '='
    if st.set_op:
        op = {'set': '=.', 'add': '+=.', 'min': '<=.', 'max': '>=.'}[st.set_op]
    return f'{tensor_name(st.output)}[{lhs}] {op} {to_ir(st.root, tensor_name, axis_name)}'


def canonical(statements, dtypes, tensor_order=None) -> str:
    """Spelling-independent key: tensors become $t0,$t1.. (with dtype), axes
    $X0,$X1.. in order of first appearance; extents are left out so one key
    covers every shape.  ``tensor_order`` (a list) receives the tensors' own names
    in that order: $tN of one program and $tN of another with the same key play
    the same part."""
    tmap, amap = {}, {}

    def tname(n):
        if n not in tmap:
            tmap[n] = f'$t{len(tmap)}:{dtypes.get(n, "?")}'
        return tmap[n]

    def aname(n):
        if n not in amap:
            amap[n] = f'$X{len(amap)}'
        return amap[n]

    key = ' ; '.join(statement_to_ir(st, tname, aname) for st in statements)
    if tensor_order is not None:
        tensor_order.extend(tmap)              # dicts keep insertion order
    return key
