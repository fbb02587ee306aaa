"""A parsed program: statements + tensor table + argument order.

Follows the reference's graph parser and argument-property registry
(lang/einstein_v2.py:519-578, lang/generic.py:35-57):

* outputs are ``extra_outputs`` plus the output of the last statement;
* a declared tensor that a statement writes is an in-out tensor and counts as
  an output of the kernel ABI;
* kernel ABI order is inputs sorted by name, then outputs sorted by name,
  then the named run-time dimensions as trailing integer arguments.

Elementwise intermediates are substituted into their consumers before lowering,
the counterpart of the reference's compute_inline pass
(antares/default_codegen.py:239-258), so a multi-statement program such as the
int4 dequant + GEMV of samples/05_llama2_7b_int4.py:135-139 becomes one kernel.
"""
from __future__ import annotations

from dataclasses import dataclass, field, replace
from functools import cached_property
from typing import Dict, List, Optional, Sequence, Tuple

from .nodes import Dim, Expr, rewrite, walk
from .parser import (IRSyntaxError, Statement, TensorInfo, parse_statement, parse_tensor_spec,
                     split_statements)
from .printer import canonical, statement_to_ir


@dataclass
class Graph:
    statements: List[Statement]
    tensors: Dict[str, TensorInfo]              # every tensor: declared + produced
    declared: List[str]                          # declared tensors in declaration order
    outputs: List[str]                           # graph outputs (not sorted)
    dims: Dict[str, Optional[int]]               # named run-time dims -> default extent
    source: str = ''

    # -- argument order (computed once: a Graph is not changed after it is built) --------
    @cached_property
    def inout(self) -> List[str]:
        written = {s.output for s in self.statements}
        return [n for n in self.declared if n in written]

    @cached_property
    def used_inputs(self) -> List[str]:
        used = set()
        for s in self.statements:
            used.update(s.reads)
        produced = {s.output for s in self.statements}
        return [n for n in self.declared if n in used and n not in produced]

    @cached_property
    def abi_inputs(self) -> List[str]:
        return sorted(self.used_inputs)

    @cached_property
    def abi_outputs(self) -> List[str]:
        outs = set(self.outputs) | set(self.inout)
        return sorted(outs)

    @cached_property
    def dim_names(self) -> List[str]:
        return sorted(self.dims)

    def canonical_key(self) -> str:
        return canonical(self.statements, {k: v.dtype for k, v in self.tensors.items()})

    def to_ir(self) -> str:
        return '; '.join(statement_to_ir(s) for s in self.statements)

    # -- shape binding --------------------------------------------------------
    def bind_dims(self, shapes: Dict[str, Sequence[int]]) -> Dict[str, int]:
        """Match actual tensor shapes against declared ones and return the value
        of every named dimension.  Static dimensions must match exactly."""
        env: Dict[str, int] = {}
        for name, shape in shapes.items():
            decl = self.tensors[name].shape
            shape = list(shape) if len(shape) else [1]
            if len(shape) != len(decl):
                raise ValueError(f'Tensor `{name}` expects {len(decl)} dimension(s), got shape {list(shape)}')
            for d, v in zip(decl, shape):
                if isinstance(d, int):
                    if d != v:
                        raise ValueError(f'Tensor `{name}` expects static extent {d}, got {v}')
                elif d in env and env[d] != v:
                    raise ValueError(f'Dimension `{d}` is bound to both {env[d]} and {v}')
                else:
                    env[d] = int(v)
        for d, default in self.dims.items():
            if d not in env:
                if default is None:
                    raise ValueError(f'Dimension `{d}` cannot be inferred from the given tensors')
                env[d] = default
        return env

    def shape_of(self, name: str, env: Dict[str, int]) -> List[int]:
        return [d if isinstance(d, int) else env[d] for d in self.tensors[name].shape]


def parse_program(ir: str, inputs, extra_outputs: Sequence[str] = ()) -> Graph:
    """``inputs`` is either the AutoRT list form ``["x=float32[N:1024]", …]`` or
    the legacy dict form ``{"x": {"dtype":…, "shape":[…]}}`` / ``{"x": "float32[…]"}``."""
    tensors: Dict[str, TensorInfo] = {}
    dims: Dict[str, Optional[int]] = {}
    declared: List[str] = []
    if isinstance(inputs, dict):
        items = list(inputs.items())
    else:
        items = []
        for spec in inputs or []:
            if '=' not in spec:
                raise IRSyntaxError(f'Input spec must look like name=dtype[dims]: `{spec}`')
            n, s = spec.split('=', 1)
            items.append((n.strip(), s.strip()))
    for name, spec in items:
        if not name or not (name[0].islower() or name[0] == '_'):
            raise IRSyntaxError(f'Tensor variable name must start with lower case letter: {name}')
        info, d = parse_tensor_spec(spec)
        tensors[name] = info
        declared.append(name)
        for k, v in d.items():
            if dims.get(k) is None:
                dims[k] = v

    statements: List[Statement] = []
    for text in split_statements(ir):
        st = parse_statement(text, tensors, dims)
        if not st.scatter:
            if st.output in tensors and st.output in declared:
                decl = tensors[st.output]
                if decl.dtype != st.out_dtype:
                    st = replace(st, root=_cast_root(st.root, decl.dtype), out_dtype=decl.dtype)
            else:
                tensors[st.output] = TensorInfo(st.out_dtype, list(st.out_shape))
        statements.append(st)
    if not statements:
        raise IRSyntaxError('Empty program')

    outputs = [o for o in extra_outputs]
    last = statements[-1].output
    if last not in outputs:
        outputs.append(last)
    for o in outputs:
        if o not in tensors:
            raise IRSyntaxError(f'Unknown output tensor `{o}`')
    return Graph(statements=statements, tensors=tensors, declared=declared, outputs=outputs, dims=dims, source=ir)


def _cast_root(root: Expr, dtype: str) -> Expr:
    from .nodes import cast
    if root.kind == 'when' and len(root.args) == 1:
        return Expr('when', dtype, args=(cast(root.args[0], dtype),), conds=root.conds, merge=root.merge)
    return cast(root, dtype)


# ---------------------------------------------------------------------------
# Inlining of elementwise producers into consumers
# ---------------------------------------------------------------------------

def _substitute_axes(e: Expr, mapping: Dict[str, Expr], extents: Dict[str, Dim]) -> Expr:
    def fn(n: Expr):
        if n.kind == 'axis' and n.name in mapping:
            return mapping[n.name]
        if n.kind == 'axis_range' and n.name in extents:
            d = extents[n.name]
            return Expr('const', 'int32', value=d) if isinstance(d, int) else Expr('dim', 'int32', value=d)
        return None
    return rewrite(e, fn)


def _is_inlinable(st: Statement, graph: Graph) -> bool:
    if st.scatter or st.reduce or st.reduce_axes:
        return False
    if st.output in graph.outputs or st.output in graph.declared:
        return False
    if st.root.kind == 'when' and len(st.root.args) == 1:
        return False
    return True


def fuse_elementwise(graph: Graph) -> Graph:
    """Substitute every elementwise intermediate into the statements that read
    it.  The result has one statement per materialised tensor (reduce results,
    scatter targets and graph outputs)."""
    producers: Dict[str, Statement] = {}
    out: List[Statement] = []
    for st in graph.statements:
        def fn(n: Expr):
            if n.kind == 'load' and n.name in producers:
                p = producers[n.name]
                mapping = {ax: idx for (ax, _), idx in zip(p.data_axes, n.args)}
                return _substitute_axes(p.root, mapping, p.axes)
            return None
        root = rewrite(st.root, fn)
        out_index = tuple(rewrite(i, fn) for i in st.out_index)
        reads: List[str] = []
        for e in list(out_index) + [root]:
            for n in walk(e):
                if n.kind == 'load' and n.name not in reads:
                    reads.append(n.name)
        st2 = replace(st, root=root, out_index=out_index, reads=reads)
        if _is_inlinable(st2, graph):
            producers[st2.output] = st2
        else:
            out.append(st2)
    tensors = {k: v for k, v in graph.tensors.items() if k not in producers}
    return Graph(statements=out, tensors=tensors, declared=graph.declared, outputs=graph.outputs,
                 dims=graph.dims, source=graph.source)
