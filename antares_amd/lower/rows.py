"""Row kernels: a run of statements that reduces over the last axis of a row and then maps over the row with the
results (softmax, layer normalisation: AntaresIR.md:226-232) lowered to one kernel that does the whole run row by
row, the row kept in registers.  The reference fuses only a tail map into a reduction
(backends/c-rocm/schedule/standard/default.py:42-52)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

from ..ir.nodes import Expr, ITEMSIZE, walk
from .emit_common import BLOCK, ExprEmitter, HIP_TYPE, _REDUCE_OP, _axes_of_all, _decompose, _extents, _multiple_of, _signature, reduce_identity
from .plans import RowGroup



def _row_group_at(graph, i: int) -> int:
    """Number of statements, starting at statement i, that form a row group (0: none): one or more reductions over
    the same single axis R with the same data axes D, each result indexed by the axes of D, and then - if the next
    statement is one - the map over D + [R] that uses the results.  Later statements of the group may read earlier
    results only at the row's own position."""
    sts, tensors = graph.statements, graph.tensors
    first = sts[i]
    if first.scatter or len(first.reduce_axes) != 1 or not first.data_axes:
        return 0
    D, R = list(first.data_axes), first.reduce_axes[0]
    d_names = [a for a, _ in D]
    j, temps = i, {}
    while j < len(sts):
        st = sts[j]
        if st.scatter or not st.reduce or list(st.reduce_axes) != [R] or list(st.data_axes) != D:
            break
        where = [ix.name if ix.kind == 'axis' else None for ix in st.out_index]
        if sorted(map(str, where)) != sorted(d_names) or st.output in temps:
            break
        if st.root.kind == 'when' and len(st.root.args) == 1:
            break
        temps[st.output] = where
        j += 1
    if not temps:
        return 0
    order = list(temps)

    def loads_fit(st, k, forbidden):
        for n in walk(st.root):
            if n.kind != 'load':
                continue
            if n.name in forbidden or n.name == st.output:
                return False
            # a load that involves R must walk memory along it (lanes of a team read neighbouring addresses)
            if any(a.kind == 'axis' and a.name == R[0] for ix in n.args for a in walk(ix)) and _row_run(n, R[0]) is None:
                return False
            if n.name in temps:
                if order.index(n.name) >= k or [a.name if a.kind == 'axis' else None for a in n.args] != temps[n.name]:
                    return False
        return True
    m = sts[j] if j < len(sts) else None
    with_map = (m is not None and not m.scatter and not m.reduce_axes and list(m.data_axes) == D + [R] and m.output not in temps
                and [ix.name if ix.kind == 'axis' else None for ix in m.out_index] == d_names + [R[0]]
                and not (m.root.kind == 'when' and len(m.root.args) == 1)
                and list(tensors[m.output].shape) == [e for _, e in D + [R]]
                and loads_fit(m, len(order), ()))
    forbidden = (m.output,) if with_map else ()
    # a row is a run of memory of its own: some load of every reduction is indexed by all the data axes (in a
    # contraction no load is - its operands are shared between outputs, which the other reduce variants exploit)
    for k in range(len(order)):
        if not any(n.kind == 'load' and set(d_names) <= _axes_of_all(n) for n in walk(sts[i + k].root)):
            return 0
    # a reduction that does not fit ends the run before it
    for k in range(len(order)):
        if not loads_fit(sts[i + k], k, forbidden):
            if with_map or k == 0:
                return 0
            return k
    return len(order) + (1 if with_map else 0)


def _row_run(n: Expr, r_ax: str):
    """For a load whose last index is R or `e + R` / `R + e` (e free of R) and whose other indices are free of R:
    the index list with the last one split as (e or None); else None.  Such a load walks memory along R."""
    if n.kind != 'load' or not n.args:
        return None
    if any(m.kind == 'axis' and m.name == r_ax for a in n.args[:-1] for m in walk(a)):
        return None
    last = n.args[-1]
    if last.kind == 'axis' and last.name == r_ax:
        return (None,)
    if last.kind == 'op' and last.name == '+' and len(last.args) == 2:
        for e, r in (last.args, last.args[::-1]):
            if r.kind == 'axis' and r.name == r_ax and not any(m.kind == 'axis' and m.name == r_ax for m in walk(e)):
                return (e,)
    return None


def _lower_row_group(graph, i: int, count: int, sym: str) -> Tuple[str, RowGroup]:
    """Kernels that compute the whole run row by row.  Every reduction meets in the row's team of lanes (a block of
    256 or one wavefront) and its result stays in a register for the statements that follow; reduce results are
    also stored, as the per-statement kernels would.  Where a row fits, it is read once, all loads in flight
    together, and kept in registers (4 or 16 vectors of 1 or 16 bytes per lane); longer rows are walked once per
    statement by a block (the first walk brings the row from memory, the later ones find it in cache)."""
    sts, tensors, dims = graph.statements[i:i + count], graph.tensors, graph.dim_names
    m = sts[-1] if not sts[-1].reduce_axes else None
    reduces = sts[:-1] if m is not None else sts
    D, (r_ax, r_ext) = list(sts[0].data_axes), sts[0].reduce_axes[0]
    temps = [st.output for st in reduces]
    written = temps + ([m.output] if m is not None else [])
    inputs = sorted({r for st in sts for r in st.reads} - set(written))
    args = inputs + written
    d_idx = [a for a, _ in D]
    oct_m = HIP_TYPE[m.out_dtype] if m is not None else None
    plain = ExprEmitter(tensors)

    # loads that walk memory along R are held in registers, one slot per distinct address expression
    slots: Dict[str, Tuple[Expr, object]] = {}

    def slot_of(n):
        run = _row_run(n, r_ax) if n.kind == 'load' and n.name not in written else None
        if run is None:
            return None
        key = n.name + '[' + ', '.join(plain.expr(a) for a in n.args) + ']'
        if key not in slots:
            slots[key] = (n, run[0], f'__c{len(slots)}')
        return slots[key]
    for st in sts:
        for n in walk(st.root):
            slot_of(n)
    row_tensors = sorted({n.name for n, _, _ in slots.values()})
    widest = max([ITEMSIZE[tensors[t].dtype] for t in row_tensors] + ([ITEMSIZE[tensors[m.output].dtype]] if m is not None else [1]))
    vmax = max(1, 16 // widest)
    # 16-byte vectors need every row to start at a multiple of the vector: indices in front of the last one are
    # multiplied by the last extent (a multiple, the launcher checks it); an offset added to R must be one provably
    vector_ok = vmax > 1 and all(e is None or _multiple_of(e, vmax, r_ax) for _, e, _ in slots.values()) and \
        all(tensors[n.name].shape[-1] == r_ext or len(n.args) == 1 for n, _, _ in slots.values())

    def emit(symbol: str, team: int, V: int, E: int) -> str:
        """team lanes per row, E vectors of V elements per lane held in registers (E == 0: the row is walked)."""
        def override(n):
            if n.name in temps:
                return f'__t_{n.name}'
            sl = slot_of(n) if E else None
            if sl is not None:
                return f'{sl[2]}[__e]' + ('[__k]' if V > 1 else '')
            return None
        em = ExprEmitter(tensors, load_override=override)
        lane = 'threadIdx.x' if team == BLOCK else '(threadIdx.x & 63)'

        def over_row(per_chunk_before, per_element, per_chunk_after):
            """Loop over this lane's share of the row: chunk-level lines, then element-level lines inside."""
            out = []
            if E:
                out += ['    #pragma unroll', f'    for (int __e = 0; __e < {E}; ++__e) {{',
                        f'      const int __r0 = ({lane} + {team} * __e) * {V};', f'      if (__r0 < __ext_{r_ax}) {{']
            else:
                out += ['    #pragma unroll 4', f'    for (int __r0 = {lane}; __r0 < __ext_{r_ax}; __r0 += {team}) {{', '      {']
            ind = '        '
            out += [ind + l for l in per_chunk_before]
            if per_element:
                if V > 1:
                    out += [ind + '#pragma unroll', ind + f'for (int __k = 0; __k < {V}; ++__k) {{',
                            ind + f'  const int {r_ax} = __r0 + __k; (void){r_ax};'] + [ind + '  ' + l for l in per_element] + [ind + '}']
                else:
                    out += [ind + f'const int {r_ax} = __r0; (void){r_ax};'] + [ind + l for l in per_element]
            out += [ind + l for l in per_chunk_after]
            out += ['      }', '    }']
            return out

        body = [_signature(symbol, args, tensors, dims, written) + ' {'] + _extents(sts[0])
        body.append('  const long long __rows = ' + (' * '.join(f'(long long)__ext_{ax}' for ax, _ in D) or '1LL') + ';')
        if V > 1:
            for n, _, reg in slots.values():
                body.append(f'  typedef {HIP_TYPE[tensors[n.name].dtype]} __vec{reg} __attribute__((ext_vector_type({V})));')
            if m is not None:
                body.append(f'  typedef {oct_m} __vec_out __attribute__((ext_vector_type({V})));')
        if team == BLOCK:
            for st in reduces:
                body.append(f'  __shared__ {HIP_TYPE[st.root.dtype]} __smem_{st.output}[4];')
            body.append('  for (long long __o = blockIdx.x; __o < __rows; __o += gridDim.x) {')
        else:
            per_block = BLOCK // team
            body.append(f'  for (long long __o = (long long)blockIdx.x * {per_block} + (threadIdx.x >> 6); __o < __rows; '
                        f'__o += (long long)gridDim.x * {per_block}) {{')
        body += _decompose('__o', D, '    ')
        if E and slots:
            loads = []
            for n, e, reg in slots.values():
                ct = f'__vec{reg}' if V > 1 else HIP_TYPE[tensors[n.name].dtype]
                body.append(f'    {ct} {reg}[{E}];')
                last = '__r0' if e is None else f'({plain.expr(e)}) + __r0'
                off = plain.offset(n.name, [plain.expr(a) for a in n.args[:-1]] + [last])
                loads.append(f'{reg}[__e] = ' + (f'*(const __vec{reg}*)&{n.name}[{off}];' if V > 1 else f'{n.name}[{off}];'))
            body += over_row(loads, [], [])
        for st in reduces:
            act, oct_ = HIP_TYPE[st.root.dtype], HIP_TYPE[st.out_dtype]
            op = _REDUCE_OP[st.reduce] + '()'
            body.append(f'    {act} __acc_{st.output} = {reduce_identity(st.reduce, st.root.dtype)};')
            body += over_row([], [f'__acc_{st.output} = {op}(__acc_{st.output}, ({act})({em.expr(st.root)}));'], [])
            meet = (f'art_block_reduce(__acc_{st.output}, {op}, __smem_{st.output})' if team == BLOCK
                    else f'art_wave_reduce(__acc_{st.output}, {op})')
            body += [f'    const {oct_} __t_{st.output} = ({oct_}){meet};',
                     f'    if ({lane} == 0) {st.output}[{plain.offset(st.output, [plain.expr(ix) for ix in st.out_index])}] = __t_{st.output};']
        if m is not None and V > 1:
            body += over_row(['__vec_out __out;'], [f'__out[__k] = ({oct_m})({em.expr(m.root)});'],
                             [f'*(__vec_out*)&{m.output}[{plain.offset(m.output, d_idx + ["__r0"])}] = __out;'])
        elif m is not None:
            body += over_row([], [f'{m.output}[{plain.offset(m.output, d_idx + [r_ax])}] = ({oct_m})({em.expr(m.root)});'], [])
        body += ['  }', '}']
        return '\n'.join(body)

    group = RowGroup(symbol=sym, args=args, count=count, row_axes=D, red_axis=(r_ax, r_ext), pure=m is None)
    code = [emit(sym, BLOCK, 1, 0)]
    if slots:
        group.vec_tensors = sorted(set(row_tensors) | ({m.output} if m is not None else set()))
        for V in sorted({1, vmax if vector_ok else 1}):
            for team, E in ((64, 4), (BLOCK, 4), (BLOCK, 16)):
                name = f'{sym}_{"w" if team == 64 else "b"}{E}' + (f'v{V}' if V > 1 else '')
                group.cached.append((team, V, E, name))
                code.append(emit(name, team, V, E))
    return '\n\n'.join(code), group
