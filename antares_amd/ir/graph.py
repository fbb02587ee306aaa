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

    def canonical_tensor_order(self) -> List[str]:
        """Tensor names in the order in which canonical_key numbers them."""
        order: List[str] = []
        canonical(self.statements, {k: v.dtype for k, v in self.tensors.items()}, order)
        return order

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


# ---------------------------------------------------------------------------
# Wide reductions with few outputs: two statements instead of one
# ---------------------------------------------------------------------------

def _divisor_near(extent: int, target: int) -> int:
    """The divisor of `extent` closest to `target` within a factor of two of it, or 0."""
    best, d = 0, 1
    while d * d <= extent:
        if extent % d == 0:
            for c in (d, extent // d):
                if max(2, target // 2) <= c <= target * 2 and (best == 0 or abs(c - target) < abs(best - target)):
                    best = c
        d += 1
    return best


def bake_small_reduce_extents(graph: Graph, env: Dict[str, int], limit: int = 8) -> Graph:
    """Named dimensions that are the extent of a reduce axis and at most `limit` in this call (the window of a
    pooling, the filter of a convolution given as `input1[F, C, KH:3, KW:3]`) become constants of the graph: the
    lowering then writes loops the compiler unrolls, divides by constants and keeps one copy of the loads that the
    terms of neighbouring outputs share.  The kernels keep all dimensions as arguments; the result is valid for these
    values only and the caller keeps it per shape.  The same graph object comes back when nothing is small."""
    small = {d: env[d] for st in graph.statements for _, d in st.reduce_axes
             if isinstance(d, str) and env.get(d) is not None and 0 < env[d] <= limit}
    if not small:
        return graph

    def fix(dims):
        return [small.get(d, d) if isinstance(d, str) else d for d in dims]
    tensors = {n: replace(t, shape=fix(t.shape)) for n, t in graph.tensors.items()}
    statements = [replace(st, data_axes=[(a, small.get(d, d) if isinstance(d, str) else d) for a, d in st.data_axes],
                          reduce_axes=[(a, small.get(d, d) if isinstance(d, str) else d) for a, d in st.reduce_axes],
                          out_shape=fix(st.out_shape)) for st in graph.statements]
    return Graph(statements=statements, tensors=tensors, declared=graph.declared, outputs=graph.outputs, dims=graph.dims,
                 source=graph.source)


def _interval(e: Expr, extent) -> Optional[Tuple[int, int]]:
    """[lowest, highest] value of an index expression made of axes, their extents, integer constants, + - * and the
    division of something non-negative by a positive constant; None for anything else.  extent(axis name) -> int or None."""
    if e.kind == 'const' and isinstance(e.value, int) and not isinstance(e.value, bool):
        return e.value, e.value
    if e.kind == 'axis':
        n = extent(e.name)
        return (0, n - 1) if n else None
    if e.kind == 'axis_range':                      # `KH.val()`: the extent itself
        n = extent(e.name)
        return (n, n) if n else None
    if e.kind == 'op' and e.name == '//' and len(e.args) == 2:     # a non-negative value divided by a positive constant
        a, b = _interval(e.args[0], extent), _interval(e.args[1], extent)
        if a is None or b is None or a[0] < 0 or b[0] != b[1] or b[0] <= 0:
            return None
        return a[0] // b[0], a[1] // b[0]
    if e.kind == 'cast' and e.dtype in ('int32', 'int64'):
        return _interval(e.args[0], extent)
    if e.kind == 'op' and e.name in ('+', '-', '*') and len(e.args) == 2:
        a, b = _interval(e.args[0], extent), _interval(e.args[1], extent)
        if a is None or b is None:
            return None
        if e.name == '+':
            return a[0] + b[0], a[1] + b[1]
        if e.name == '-':
            return a[0] - b[1], a[1] - b[0]
        c = [x * y for x in a for y in b]
        return min(c), max(c)
    return None


def pad_guarded_factors(graph: Graph, env: Optional[Dict[str, int]] = None) -> Graph:
    """A sum of products in which one factor is a guarded load, `x[..., HO + KH - 1, ...].when([HO + KH - 1 >= 0,
    HO + KH - 1 < 32, ...], 0)` (the zero padding of a convolution, AntaresIR.md:166), is rewritten as

        x__pad[P0, P1, ...] = x[P0 + lo0, P1 + lo1, ...].when([the same conditions on P + lo], 0)
        out[...] +=! x__pad[..., HO + KH - 1 - lo, ...] * w[...]

    where [lo, hi] is the interval each index takes: the guards are evaluated once per element of the padded copy
    instead of once per term of the sum (nine times per element for a 3 x 3 filter, and in the inner loop of the
    contraction).  Only when the guarded value is the load itself (or casts of it: g(0) must be 0 for what stays
    around the padded load), every condition compares one of the load's own index expressions with a constant, the
    unguarded indices provably stay inside the tensor, the copy is at most four times the tensor, and the sum has at
    least 64 terms.  `env`: values of named dimensions for one call (the result is then valid for those only)."""
    from .nodes import Expr as E
    from .printer import to_ir
    env = env or {}

    def value(d):
        return d if isinstance(d, int) else env.get(d)
    out: List[Statement] = []
    tensors = dict(graph.tensors)
    changed = False
    for st in graph.statements:
        done = False
        root = st.root
        terms = 1
        for _, d in st.reduce_axes:
            terms *= value(d) or 0
        if st.reduce == '+' and not st.scatter and root.kind == 'op' and root.name == '*' and len(root.args) == 2 and terms >= 64 and \
                all(value(d) for _, d in st.data_axes):
            ext = {a: value(d) for a, d in st.data_axes + st.reduce_axes}
            for which in (0, 1):
                f = root.args[which]
                if f.kind != 'when' or len(f.args) != 2 or f.merge != 'all' or not (f.args[1].kind == 'const' and f.args[1].value == 0):
                    continue
                # The guarded value must be the load itself or casts of it: the contraction then reads the padded copy
                # through the same casts, and a cast maps the copy's zeros to zeros.  Anything else around the load
                # (`(x[..] + 1).when(..)`, `x[..].call(exp)`) would turn the border's 0 into g(0).
                bare = f.args[0]
                while bare.kind == 'cast' and len(bare.args) == 1:
                    bare = bare.args[0]
                if bare.kind != 'load' or not bare.args or bare.name == st.output or bare.name + '__pad' in tensors:
                    continue
                ld = bare
                if any(n.kind in ('load', 'when') for c in f.conds for n in walk(c)):
                    continue
                shape = [value(d) for d in tensors[ld.name].shape]
                spans = [_interval(ix, ext.get) for ix in ld.args]
                if any(sp is None for sp in spans) or any(n is None for n in shape):
                    continue
                texts = [to_ir(ix) for ix in ld.args]
                # every condition: (index expression of the load) compared with an integer constant
                guarded, ok = set(), True
                for c in f.conds:
                    sides = [to_ir(a) for a in c.args] if c.kind == 'op' and len(c.args) == 2 and c.name in ('<', '<=', '>', '>=', '==', '!=') else []
                    hit = [k for k, t in enumerate(sides) if t in texts]
                    other = c.args[1 - hit[0]] if len(hit) == 1 else None
                    if other is None or not (other.kind == 'const' and isinstance(other.value, int)):
                        ok = False
                        break
                    guarded.add(texts.index(sides[hit[0]]))
                if not ok or not guarded:
                    continue
                if any(d not in guarded and not (0 <= sp[0] and sp[1] < n) for d, (sp, n) in enumerate(zip(spans, shape))):
                    continue
                size, numel = 1, 1
                for sp, n in zip(spans, shape):
                    size *= sp[1] - sp[0] + 1
                    numel *= n
                if size > 4 * numel:
                    continue
                # the padded copy
                pad = ld.name + '__pad'
                axes = []
                for d in range(len(spans)):
                    ax = f'P{d}'
                    while ax in ext or any(ax == a for a, _ in axes):
                        ax += 'p'
                    axes.append((ax, spans[d][1] - spans[d][0] + 1))
                moved = [E('op', 'int32', name='+', args=(E('axis', 'int32', name=ax), E('const', 'int32', value=sp[0]))) if sp[0] else E('axis', 'int32', name=ax)
                         for (ax, _), sp in zip(axes, spans)]
                by_text = dict(zip(texts, moved))
                conds = tuple(E(c.kind, c.dtype, name=c.name, args=tuple(by_text.get(to_ir(a), a) for a in c.args)) for c in f.conds)
                dt = tensors[ld.name].dtype
                fill = E('when', dt, args=(E('load', dt, name=ld.name, args=tuple(moved)), E('const', dt, value=0 if dt.startswith('int') else 0.0)),
                         conds=conds, merge='all')
                tensors[pad] = TensorInfo(dtype=dt, shape=[n for _, n in axes])
                s0 = Statement(output=pad, out_index=tuple(E('axis', 'int32', name=ax) for ax, _ in axes), root=fill, reduce=None, set_op=None,
                               data_axes=list(axes), reduce_axes=[], out_dtype=dt, out_shape=[n for _, n in axes], scatter=False, reads=[ld.name])
                shifted = tuple(E('op', 'int32', name='-', args=(ix, E('const', 'int32', value=sp[0]))) if sp[0] else ix for ix, sp in zip(ld.args, spans))
                inner = rewrite(f.args[0], lambda n: E('load', dt, name=pad, args=shifted) if n is ld else None)
                new_root = E(root.kind, root.dtype, name=root.name, args=(inner, root.args[1]) if which == 0 else (root.args[0], inner))
                reads = [r for r in st.reads if r != ld.name or any(n.kind == 'load' and n.name == ld.name for n in walk(new_root))] + [pad]
                out += [s0, replace(st, root=new_root, reads=reads)]
                done = changed = True
                break
        if not done:
            out.append(st)
    if not changed:
        return graph
    return Graph(statements=out, tensors=tensors, declared=graph.declared, outputs=graph.outputs, dims=graph.dims,
                 source=graph.source)


def split_wide_reductions(graph: Graph, env: Optional[Dict[str, int]] = None, wanted=None) -> Graph:
    """A reduction whose outputs are too few to fill the chip is rewritten as

        out[D] op= f(D, R)      ->      out__part[S, D] op= f(D, S * chunk + Rc)   (S * chunk = extent of R)
                                        out[D]          op= out__part[S, D]

    so that the generic lowering sees S times as many independent outputs (a sum over 16.7 M elements ran on one
    block at 2.5 GB/s before this).  The slice count S aims at about 16384 outputs when the reduced axis is the
    contiguous one (a wavefront per output) and about 262144 when an output axis is (a thread per output).  Only
    divisible axes of known size are split; everything else is left alone.  The accumulation order changes from
    sequential to two-level, as it already does inside a wavefront.

    `env` gives the values of named dimensions for one call; the result is then valid for those values only (the
    slices must tile the axis exactly) and the caller keeps it per shape.

    `wanted(statement, value)` may name a slice count for a statement that the rule above would leave alone (value(d)
    is the extent of dimension d in this call): the lowering asks for one when a contraction has too few output tiles
    to fill the chip.  Such a statement keeps its outputs' order in memory - the slices become the leading dimension
    of `out__part` - so that it is still a contraction with a batch axis in front."""
    from .nodes import Expr as E
    env = env or {}

    def value(d):
        return d if isinstance(d, int) else env.get(d)

    out: List[Statement] = []
    tensors = dict(graph.tensors)
    changed = False
    for st in graph.statements:
        axes = st.reduce_axes
        if not st.reduce or not axes or st.scatter or st.set_op or (st.root.kind == 'when' and len(st.root.args) == 1):
            out.append(st)
            continue
        if any(value(d) is None for _, d in st.data_axes + axes):
            out.append(st)
            continue
        outputs = 1
        for _, d in st.data_axes:
            outputs *= value(d)
        rax, extent = axes[0][0], value(axes[0][1])   # the outermost reduced axis is the one that is sliced
        inner = 1
        for _, d in axes[1:]:
            inner *= value(d)
        asked = wanted(st, value) if wanted is not None else None
        # which axis walks memory in the biggest operand decides how the lowering maps outputs to lanes
        raxes, daxes, score = {a for a, _ in axes}, {a for a, _ in st.data_axes}, 0
        for n in walk(st.root):
            if n.kind == 'load' and n.args:
                names = {m.name for m in walk(n.args[-1]) if m.kind == 'axis'}
                score += len(n.args) if names & raxes else (-len(n.args) if names & daxes else 0)
        want_outputs, min_chunk = (16384, 256) if score >= 0 else (262144, 16)
        if asked is None and (outputs * 2 > want_outputs or extent * inner < 4 * min_chunk):
            out.append(st)
            continue
        target = asked if asked is not None else max(2, min(want_outputs // max(outputs, 1), extent * inner // min_chunk, extent))
        S = _divisor_near(extent, target)
        if S < 2 or S > extent or (S == extent and inner == 1):     # a slice per value of the axis: only when other reduce axes remain
            out.append(st)
            continue
        chunk = extent // S
        s_ax, c_ax = f'{rax}S', f'{rax}C'
        while any(s_ax == a or c_ax == a for a, _ in st.data_axes + axes):
            s_ax, c_ax = s_ax + 'x', c_ax + 'x'
        index = E('op', 'int32', name='+', args=(E('op', 'int32', name='*', args=(E('axis', 'int32', name=s_ax), E('const', 'int32', value=chunk))),
                                                E('axis', 'int32', name=c_ax)))
        root1 = rewrite(st.root, lambda n: index if (n.kind == 'axis' and n.name == rax) else
                        (E('const', 'int32', value=extent) if (n.kind == 'axis_range' and n.name == rax) else None))
        part = st.output + '__part'
        while part in tensors:
            part += '_'
        s_idx = E('axis', 'int32', name=s_ax)
        if asked is not None:       # slices in front: statement 1 stays a contraction, statement 2 sums whole planes
            p_index, p_shape = (s_idx,) + tuple(st.out_index), [S] + list(st.out_shape)
        else:                       # the slices of one output lie next to each other: statement 2 reduces along memory
            p_index, p_shape = tuple(st.out_index) + (s_idx,), list(st.out_shape) + [S]
        tensors[part] = TensorInfo(dtype=st.root.dtype, shape=p_shape)
        s1 = replace(st, output=part, out_index=p_index, root=root1,
                     data_axes=[(s_ax, S)] + list(st.data_axes), reduce_axes=[(c_ax, chunk)] + list(axes[1:]),
                     out_dtype=st.root.dtype, out_shape=p_shape)
        load = E('load', st.root.dtype, name=part, args=p_index)
        s2 = replace(st, root=load, reduce_axes=[(s_ax, S)], reads=[part])
        out += [s1, s2]
        changed = True
    if not changed:
        return graph
    return Graph(statements=out, tensors=tensors, declared=graph.declared, outputs=graph.outputs, dims=graph.dims,
                 source=graph.source)
