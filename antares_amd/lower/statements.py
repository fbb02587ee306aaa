"""One statement -> its kernels: elementwise / gather maps (flat, vectorised, tiled permutation copies), reductions
(wavefront, block, thread per output, register-tiled patches, and the matrix kernel of `matrix.py` where it applies)
and scatters.  Replaces the reference's elementwise and reduce schedules
(backends/c-rocm/schedule/standard/algo_format.py:6-51, algo_reduce.py:6-59)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

from ..ir.nodes import Expr, ITEMSIZE, walk
from .emit_common import BLOCK, ExprEmitter, HIP_TYPE, _REDUCE_OP, _decompose, _extents, _root_and_cond, _signature, reduce_identity
from .matrix import _matrix_contraction, _matrix_kernel, _matrix_tail
from .plans import KernelPlan



def _transpose_axes(st, tensors):
    """(A, B) when the statement is a permutation copy (possibly with elementwise work on top): one load, indexed
    by all data axes, each once and bare, whose last axis A differs from the last axis B of the store.  Reading
    walks memory along A, writing along B; a tile in LDS turns one into the other."""
    axes = [a for a, _ in st.data_axes]
    if st.scatter or st.reduce_axes or len(axes) < 2 or [i.name for i in st.out_index if i.kind == 'axis'] != axes:
        return None
    if st.root.kind == 'when' and len(st.root.args) == 1:
        return None
    loads = [n for n in walk(st.root) if n.kind == 'load']
    if len(loads) != 1 or loads[0].name == st.output:
        return None
    idx = loads[0].args
    if any(a.kind != 'axis' for a in idx) or sorted(a.name for a in idx) != sorted(axes):
        return None
    if sum(1 for n in walk(st.root) if n.kind == 'axis') != len(idx):       # a bare axis used as a value
        return None
    a_ax, b_ax = idx[-1].name, axes[-1]
    return None if a_ax == b_ax else (a_ax, b_ax)


def _row_vector_loads(st, tensors):
    """Loads that walk memory along the statement's last data axis L, for a statement that stores densely along L:
    every load either does not mention L at all (one value for the whole vector) or has the bare axis L as its last
    index and L nowhere else (a contiguous run: bias rows, gathered rows, `table[ids[N], C]`).  Returns (L, those
    loads) or None when the statement is not of that shape."""
    axes = [a for a, _ in st.data_axes]
    exts = [e for _, e in st.data_axes]
    if not axes or st.scatter or st.reduce_axes or [i.name for i in st.out_index if i.kind == 'axis'] != axes:
        return None
    if len(st.out_index) != len(axes) or list(tensors[st.output].shape) != exts:
        return None
    if st.root.kind == 'when' and len(st.root.args) == 1:
        return None
    L = axes[-1]
    runs = []
    for n in walk(st.root):
        if n.kind != 'load':
            continue
        if n.name == st.output:
            return None
        uses = [any(m.kind == 'axis' and m.name == L for m in walk(a)) for a in n.args]
        if not any(uses):
            continue
        if any(uses[:-1]) or n.args[-1].kind != 'axis':
            return None
        runs.append(n)
    return (L, runs) if runs else None


def _is_flat_map(st, tensors) -> bool:
    """True when every load (and the store) addresses element ``flat`` of a
    tensor whose extents equal the statement's data extents."""
    axes = [a for a, _ in st.data_axes]
    exts = [e for _, e in st.data_axes]
    if st.scatter or st.reduce_axes or [i.name for i in st.out_index if i.kind == 'axis'] != axes:
        return False
    if list(tensors[st.output].shape) != exts:
        return False
    for e in [st.root]:
        for n in walk(e):
            if n.kind == 'load':
                if [a.name if a.kind == 'axis' else None for a in n.args] != axes:
                    return False
                if list(tensors[n.name].shape) != exts:
                    return False
    # bare axes outside of loads need the decomposed index; allow them only in 1-D
    loads_axes = 0
    all_axes = 0
    for n in walk(st.root):
        if n.kind == 'axis':
            all_axes += 1
        if n.kind == 'load':
            loads_axes += sum(1 for a in n.args if a.kind == 'axis')
    return all_axes == loads_axes or len(axes) == 1


def lower_statement(st, graph, name: str, tail=None) -> Tuple[str, KernelPlan]:
    """Kernels of one statement.  `tail`: the map statement behind a reduction that is applied to each result where it
    is stored (the reference's tail fusion, AntaresIR.md:248-250: `conv_out +=! ...; output0 = f(conv_out, bias)` is
    one kernel); the reduction's own output is then never written."""
    tensors, dims = graph.tensors, graph.dim_names
    reads = [r for r in st.reads]
    args = sorted(set(reads) - {st.output}) + [st.output]
    written = [st.output]
    if tail is not None:
        args = sorted((set(reads) | set(tail.reads)) - {st.output, tail.output}) + [tail.output]
        written = [tail.output]

    def one_touch(n: Expr) -> Optional[str]:
        """A load that reads every element of its tensor exactly once in the whole program - indexed by all axes of
        the statement, each once, and no other statement or load touches the tensor - carries the non-temporal
        hint (an evict-first stream: measured +10 % on the 4 096 000-element sigmoid)."""
        axes = [ax for ax, _ in st.data_axes + st.reduce_axes]
        if n.name == st.output or any(a.kind != 'axis' for a in n.args):
            return None
        if sorted(a.name for a in n.args) != sorted(axes):
            return None
        if sum(1 for s_ in graph.statements if n.name in s_.reads or n.name == s_.output) != 1:
            return None
        if sum(1 for m in walk(st.root) if m.kind == 'load' and m.name == n.name) != 1:
            return None
        return f'__builtin_nontemporal_load(&{n.name}[{plain.offset(n.name, [plain.expr(a) for a in n.args])}])'

    plain = ExprEmitter(tensors)
    em = ExprEmitter(tensors, load_override=one_touch)
    total = ' * '.join(f'(long long)__ext_{ax}' for ax, _ in st.data_axes) or '1LL'
    oct_ = HIP_TYPE[st.out_dtype]
    src: List[str] = []
    variants: Dict[str, str] = {}
    plan = KernelPlan(name=name, args=args, dims=dims, variants=variants,
                      kind='scatter' if st.scatter else ('reduce' if st.reduce_axes else 'map'),
                      output=written[0], data_axes=list(st.data_axes), reduce_axes=list(st.reduce_axes), covers=2 if tail is not None else 1)

    def header(sym):
        return [_signature(sym, args, tensors, dims, written) + ' {'] + _extents(st) + \
               [f'  const long long __total = {total};',
                f'  const long long __tid = (long long)blockIdx.x * {BLOCK} + threadIdx.x;',
                f'  const long long __nthr = (long long)gridDim.x * {BLOCK};']

    root, cond = _root_and_cond(st, em)
    dst = f'{st.output}[{em.offset(st.output, [em.expr(i) for i in st.out_index])}]'

    if plan.kind == 'map':
        sym = name
        body = header(sym)
        body.append('  for (long long __i = __tid; __i < __total; __i += __nthr) {')
        body += _decompose('__i', st.data_axes, '    ', '__total')
        store = f'{dst} = ({oct_})({em.expr(root)});'
        body.append(f'    if ({cond}) {{ {store} }}' if cond else f'    {store}')
        body += ['  }', '}']
        src.append('\n'.join(body))
        variants['scalar'] = sym
        if _is_flat_map(st, tensors) and cond is None:
            names = sorted({n.name for n in walk(root) if n.kind == 'load'} | {st.output})
            width = max(ITEMSIZE[tensors[n].dtype] for n in names)
            V = max(1, 16 // width)
            if V > 1:
                sym = name + '_v'
                body = header(sym)
                for n in names:
                    body.append(f'  typedef {HIP_TYPE[tensors[n].dtype]} __vec_{n} __attribute__((ext_vector_type({V})));')
                body.append(f'  const long long __nvec = __total / {V};')
                body.append('  for (long long __v = __tid; __v < __nvec; __v += __nthr) {')
                # a tensor no other statement of the program touches is streamed: non-temporal accesses measured
                # 4520 against 4110 GB/s on the 4 096 000-element sigmoid
                def streamed(n):
                    return sum(1 for s_ in graph.statements if n in s_.reads or n == s_.output) == 1
                for n in names:
                    if n != st.output or n in reads:
                        src_ = f'((const __vec_{n}*){n})[__v]'
                        body.append(f'    const __vec_{n} __in_{n} = ' + (f'__builtin_nontemporal_load(&{src_});' if streamed(n) else f'{src_};'))
                body.append(f'    __vec_{st.output} __out;')
                vem = ExprEmitter(tensors, load_override=lambda n: f'__in_{n.name}[__e]')
                body.append('    #pragma unroll')
                body.append(f'    for (int __e = 0; __e < {V}; ++__e) {{')
                if len(st.data_axes) == 1:
                    body.append(f'      const int {st.data_axes[0][0]} = (int)(__v * {V} + __e); (void){st.data_axes[0][0]};')
                body.append(f'      __out[__e] = ({oct_})({vem.expr(root)});')
                body.append('    }')
                dst_ = f'((__vec_{st.output}*){st.output})[__v]'
                body.append(f'    __builtin_nontemporal_store(__out, &{dst_});' if streamed(st.output) else f'    {dst_} = __out;')
                body.append('  }')
                body.append(f'  for (long long __i = __nvec * {V} + __tid; __i < __total; __i += __nthr) {{')
                body += _decompose('__i', st.data_axes, '    ', '__total')
                body.append(f'    {dst} = ({oct_})({em.expr(root)});')
                body += ['  }', '}']
                src.append('\n'.join(body))
                variants['vec'] = sym
                plan.vec, plan.vec_tensors = V, names
        rv = _row_vector_loads(st, tensors) if 'vec' not in variants and cond is None else None
        if rv is not None:
            L, runs = rv
            names = sorted({n.name for n in runs} | {st.output})
            V = max(1, 16 // max(ITEMSIZE[tensors[n].dtype] for n in names))
            if V > 1:
                sym = name + '_r'
                body = header(sym)
                for n in names:
                    body.append(f'  typedef {HIP_TYPE[tensors[n].dtype]} __vec_{n} __attribute__((ext_vector_type({V})));')
                body.append(f'  const long long __lv = __ext_{L} / {V};')
                body.append(f'  const long long __nvec = __total / {V};')
                body.append('  for (long long __v = __tid; __v < __nvec; __v += __nthr) {')
                body.append('    long long __r = __v;')
                body.append(f'    const int __l0 = (int)(__r % __lv) * {V}; __r /= __lv;')
                for ax, _ in reversed(st.data_axes[:-1]):
                    body.append(f'    const int {ax} = (int)(__r % __ext_{ax}); __r /= __ext_{ax};')
                def streamed(n):
                    return sum(1 for s_ in graph.statements if n in s_.reads or n == s_.output) == 1
                for k, n in enumerate(runs):
                    off = plain.offset(n.name, [plain.expr(a) for a in n.args[:-1]] + ['__l0'])
                    ref = f'*(const __vec_{n.name}*)&{n.name}[{off}]'
                    once = one_touch(n) is not None
                    body.append(f'    const __vec_{n.name} __run_{k} = ' + (f'__builtin_nontemporal_load(&({ref}));' if once else f'{ref};'))
                def run_lane(n):
                    for k, m in enumerate(runs):
                        if m is n:
                            return f'__run_{k}[__e]'
                    return None
                rem = ExprEmitter(tensors, load_override=run_lane)
                body.append(f'    __vec_{st.output} __out;')
                body.append('    #pragma unroll')
                body.append(f'    for (int __e = 0; __e < {V}; ++__e) {{')
                body.append(f'      const int {L} = __l0 + __e; (void){L};')
                body.append(f'      __out[__e] = ({oct_})({rem.expr(root)});')
                body.append('    }')
                dst_ = f'((__vec_{st.output}*){st.output})[__v]'
                body.append(f'    __builtin_nontemporal_store(__out, &{dst_});' if streamed(st.output) else f'    {dst_} = __out;')
                body += ['  }', '}']
                src.append('\n'.join(body))
                variants['rowvec'] = sym
                plan.row_vec = V
                plan.row_tensors = names
                plan.row_dims = [st.data_axes[-1][1]] + [tensors[n.name].shape[-1] for n in runs]
        tr = _transpose_axes(st, tensors)
        if tr is not None:
            a_ax, b_ax = tr
            others = [(ax, e) for ax, e in st.data_axes if ax not in (a_ax, b_ax)]
            sym = name + '_x'
            body = [_signature(sym, args, tensors, dims, written) + ' {'] + _extents(st)
            body += [f'  __shared__ {oct_} __tile[64][65];',
                     '  const int __tx = threadIdx.x & 63, __ty = threadIdx.x >> 6;',
                     f'  const long long __ta = ((long long)__ext_{a_ax} + 63) / 64, __tb = ((long long)__ext_{b_ax} + 63) / 64;',
                     '  const long long __batch = ' + (' * '.join(f'(long long)__ext_{ax}' for ax, _ in others) or '1LL') + ';',
                     '  for (long long __t = blockIdx.x; __t < __ta * __tb * __batch; __t += gridDim.x) {',
                     '    const long long __ia = __t % __ta, __ib = (__t / __ta) % __tb;',
                     '    long long __r = __t / (__ta * __tb); (void)__r;']
            for ax, _ in reversed(others):
                body.append(f'    const int {ax} = (int)(__r % __ext_{ax}); __r /= __ext_{ax};')
            body += ['    for (int __row = __ty; __row < 64; __row += 4) {       // read along the input\'s last axis',
                     f'      const int {a_ax} = (int)(__ia * 64 + __tx), {b_ax} = (int)(__ib * 64 + __row);',
                     f'      if ({a_ax} < __ext_{a_ax} && {b_ax} < __ext_{b_ax}) __tile[__row][__tx] = ({oct_})({plain.expr(root)});',
                     '    }',
                     '    __syncthreads();',
                     '    for (int __row = __ty; __row < 64; __row += 4) {       // write along the output\'s last axis',
                     f'      const int {a_ax} = (int)(__ia * 64 + __row), {b_ax} = (int)(__ib * 64 + __tx);',
                     f'      if ({a_ax} < __ext_{a_ax} && {b_ax} < __ext_{b_ax}) {dst} = __tile[__tx][__row];',
                     '    }',
                     '    __syncthreads();',
                     '  }', '}']
            src.append('\n'.join(body))
            variants['tile'] = sym
            plan.tile_axes = (a_ax, b_ax)
            # The same with 16-byte vectors on both sides (whole tiles, aligned pointers): a lane reads V neighbours
            # along the input's last axis and writes V neighbours along the output's; in between the tile lies in
            # LDS with a row pitch that spreads both the scalar writes and the transposed scalar reads over the
            # banks.  4096 x 4096 fp32: 28 us against 39 (a plain copy of the same bytes: 25).
            ld = [n for n in walk(st.root) if n.kind == 'load'][0]
            size = ITEMSIZE[tensors[ld.name].dtype]
            if size == ITEMSIZE[tensors[st.output].dtype] and size in (2, 4):
                V = 16 // size
                VR, RP, P = 64 // V, BLOCK // (64 // V), 64 + 4 // size
                PASSES = 64 // RP
                ict = HIP_TYPE[tensors[ld.name].dtype]
                sym = name + '_xv'
                def streamed(n):
                    return sum(1 for s_ in graph.statements if n in s_.reads or n == s_.output) == 1
                in_off = plain.offset(ld.name, ['__a0' if a.name == a_ax else a.name for a in ld.args])
                out_off = plain.offset(st.output, ['__b0' if ax == b_ax else ax for ax, _ in st.data_axes])
                vem = ExprEmitter(tensors, load_override=lambda n: '__v[__p][__e]')
                body = [_signature(sym, args, tensors, dims, written) + ' {'] + _extents(st)
                body += [f'  __shared__ {oct_} __tile[64 * {P}];',
                         f'  typedef {ict} __vin __attribute__((ext_vector_type({V})));',
                         f'  typedef {oct_} __vout __attribute__((ext_vector_type({V})));',
                         f'  const int __lv = threadIdx.x % {VR}, __grp = threadIdx.x / {VR};',
                         f'  const long long __ta = (long long)__ext_{a_ax} / 64, __tb = (long long)__ext_{b_ax} / 64;',
                         '  const long long __batch = ' + (' * '.join(f'(long long)__ext_{ax}' for ax, _ in others) or '1LL') + ';',
                         '  for (long long __t = blockIdx.x; __t < __ta * __tb * __batch; __t += gridDim.x) {',
                         '    const long long __ia = __t % __ta, __ib = (__t / __ta) % __tb;',
                         '    long long __r = __t / (__ta * __tb); (void)__r;']
                for ax, _ in reversed(others):
                    body.append(f'    const int {ax} = (int)(__r % __ext_{ax}); __r /= __ext_{ax};')
                ref = f'(const __vin*)&{ld.name}[{in_off}]'
                body += [f'    __vin __v[{PASSES}];',
                         '    #pragma unroll',
                         f'    for (int __p = 0; __p < {PASSES}; ++__p) {{       // read along the input\'s last axis',
                         f'      const int __a0 = (int)(__ia * 64 + __lv * {V}), {b_ax} = (int)(__ib * 64 + __grp + {RP} * __p);',
                         f'      __v[__p] = ' + (f'__builtin_nontemporal_load({ref});' if streamed(ld.name) else f'*{ref};'),
                         '    }',
                         '    #pragma unroll',
                         f'    for (int __p = 0; __p < {PASSES}; ++__p) {{',
                         '      #pragma unroll',
                         f'      for (int __e = 0; __e < {V}; ++__e)',
                         f'        __tile[(__grp + {RP} * __p) * {P} + __lv * {V} + __e] = ({oct_})({vem.expr(root)});',
                         '    }',
                         '    __syncthreads();',
                         '    #pragma unroll',
                         f'    for (int __p = 0; __p < {PASSES}; ++__p) {{       // write along the output\'s last axis',
                         f'      const int {a_ax} = (int)(__ia * 64 + __grp + {RP} * __p), __b0 = (int)(__ib * 64 + __lv * {V});',
                         '      __vout __o;',
                         '      #pragma unroll',
                         f'      for (int __e = 0; __e < {V}; ++__e) __o[__e] = __tile[(__lv * {V} + __e) * {P} + __grp + {RP} * __p];',
                         f'      __vout* __d = (__vout*)&{st.output}[{out_off}];',
                         '      ' + ('__builtin_nontemporal_store(__o, __d);' if streamed(st.output) else '*__d = __o;'),
                         '    }',
                         '    __syncthreads();',
                         '  }', '}']
                src.append('\n'.join(body))
                variants['tilevec'] = sym
                plan.tile_tensors = sorted({ld.name, st.output})

    elif plan.kind == 'scatter':
        sym = name
        body = header(sym)
        body.append('  for (long long __i = __tid; __i < __total; __i += __nthr) {')
        body += _decompose('__i', st.data_axes, '    ', '__total')
        val = f'({oct_})({em.expr(root)})'
        store = {'set': f'{dst} = {val};', 'add': f'atomicAdd(&{dst}, {val});',
                 'min': f'atomicMin(&{dst}, {val});', 'max': f'atomicMax(&{dst}, {val});'}[st.set_op]
        body.append(f'    if ({cond}) {{ {store} }}' if cond else f'    {store}')
        body += ['  }', '}']
        src.append('\n'.join(body))
        variants['scalar'] = sym

    else:
        act = HIP_TYPE[root.dtype]
        ident = reduce_identity(st.reduce, root.dtype)
        op = _REDUCE_OP[st.reduce] + '()'
        red_total = ' * '.join(f'(long long)__ext_{ax}' for ax, _ in st.reduce_axes)
        def result_store(acc):         # C text that stores one result held in `acc`
            if tail is None:
                text = f'{dst} = ({oct_}){acc};'
                return f'if ({cond}) {{ {text} }}' if cond else text
            # the tail sees the result as the reduction's output would hold it (rounded to its type)
            tem = ExprEmitter(tensors, load_override=lambda n: '__t' if n.name == st.output else None)
            troot, tcond = _root_and_cond(tail, tem)
            tdst = f'{tail.output}[{plain.offset(tail.output, [plain.expr(i) for i in tail.out_index])}]'
            text = f'{tdst} = ({HIP_TYPE[tail.out_dtype]})({tem.expr(troot)});'
            text = f'if ({tcond}) {{ {text} }}' if tcond else text
            return f'{{ const {oct_} __t = ({oct_}){acc}; (void)__t; {text} }}'
        store = result_store('__acc')

        def reduce_body(sym, out_var, out_step, lane, nlanes, finish):
            b = header(sym)
            b.append(f'  const long long __red = {red_total};')
            if sym.endswith('_b'):
                b.append(f'  __shared__ {act} __smem[4];')
            b.append(f'  for (long long __o = {out_var}; __o < __total; __o += {out_step}) {{')
            b += _decompose('__o', st.data_axes, '    ', '__total')
            b.append(f'    {act} __acc = {ident};')
            if nlanes == '1':
                # a thread walks all of the reduce space: one loop per reduce axis, in the same order as the flat walk,
                # no divisions - a pooling window or a depthwise filter is then a handful of adds per term
                for d, (ax, _) in enumerate(st.reduce_axes):
                    if d == len(st.reduce_axes) - 1:
                        b.append('    ' + '  ' * d + '#pragma unroll 4')
                    b.append('    ' + '  ' * d + f'for (int {ax} = 0; {ax} < __ext_{ax}; ++{ax})' + (' {' if d == len(st.reduce_axes) - 1 else ''))
                b.append('    ' + '  ' * len(st.reduce_axes) + f'__acc = {op}(__acc, ({act})({em.expr(root)}));')
                b.append('    ' + '  ' * (len(st.reduce_axes) - 1) + '}')
            else:
                b.append('    #pragma unroll 4')
                b.append(f'    for (long long __k = {lane}; __k < __red; __k += {nlanes}) {{')
                b += _decompose('__k', st.reduce_axes, '      ', '__red', tmp='__q')
                b.append(f'      __acc = {op}(__acc, ({act})({em.expr(root)}));')
                b.append('    }')
            b += finish
            b += ['  }', '}']
            return '\n'.join(b)

        src.append(reduce_body(name + '_t', '__tid', '__nthr', '0', '1', [f'    {store}']))
        src.append(reduce_body(name + '_w', '(__tid >> 6)', '(__nthr >> 6)', '(threadIdx.x & 63)', '64',
                               [f'    __acc = art_wave_reduce(__acc, {op});', f'    if ((threadIdx.x & 63) == 0) {{ {store} }}']))
        src.append(reduce_body(name + '_b', '(long long)blockIdx.x', '(long long)gridDim.x', 'threadIdx.x', str(BLOCK),
                               [f'    __acc = art_block_reduce(__acc, {op}, __smem);', f'    if (threadIdx.x == 0) {{ {store} }}']))
        variants.update({'thread': name + '_t', 'wave': name + '_w', 'block': name + '_b'})
        plan.reduce_contiguous = _reduce_axis_contiguous(st, tensors)
        pa = _patch_axes(st)
        if pa is not None:
            # Register tiling for contractions (the reference's tiled schedule, backends/c-rocm/schedule/standard/
            # algo_tiling.py:35-98): a thread owns TX x TY neighbouring outputs along two data axes chosen so that every
            # operand is constant along one of them; the statement's expression is written out for each of the 16
            # outputs and the compiler keeps one copy of every load they share.  Each output still accumulates its terms
            # in the reference's order.
            xa, ya = pa
            ext = dict(st.data_axes)

            def tile(e):                 # 4 outputs along an axis, 2 where a static extent only divides by 2
                return 4 if not isinstance(e, int) or e % 4 == 0 else (2 if e % 2 == 0 else 0)
            TX, TY = tile(ext[xa]), tile(ext[ya])
        if pa is not None and TX and TY:
            sym = name + '_p'
            b = header(sym)
            b.append(f'  const long long __red = {red_total};')
            b.append(f'  const long long __px = __ext_{xa} / {TX}, __py = __ext_{ya} / {TY};')
            b.append(f'  const long long __patches = __total / {TX * TY};')
            b.append('  for (long long __o = __tid; __o < __patches; __o += __nthr) {')
            others = [ax for ax, _ in st.data_axes if ax not in (xa, ya)]
            b.append('    int __x0, __y0' + ''.join(f', {ax}' for ax in others) + ';')
            for small in (True, False):         # 32-bit divisions whenever the patch count fits them
                b.append('    if (__patches <= 0x7fffffffLL) {' if small else '    } else {')
                b.append('      unsigned int __r = (unsigned int)__o;' if small else '      long long __r = __o;')
                cast = '(unsigned int)' if small else ''
                for ax, _ in reversed(st.data_axes):
                    if ax == ya:
                        b.append(f'      __y0 = (int)(__r % {cast}__py) * {TY}; __r /= {cast}__py;')
                    elif ax == xa:
                        b.append(f'      __x0 = (int)(__r % {cast}__px) * {TX}; __r /= {cast}__px;')
                    else:
                        b.append(f'      {ax} = (int)(__r % {cast}__ext_{ax}); __r /= {cast}__ext_{ax};')
            b.append('    }')
            b.append('    ' + ' '.join(f'(void){ax};' for ax in others))
            b.append(f'    {act} __acc[{TX}][{TY}];')
            b.append('    #pragma unroll')
            b.append(f'    for (int __i = 0; __i < {TX}; ++__i)')
            b.append('      #pragma unroll')
            b.append(f'      for (int __j = 0; __j < {TY}; ++__j) __acc[__i][__j] = {ident};')
            for d, (ax, _) in enumerate(st.reduce_axes):       # one loop per reduce axis, in the order of the flat walk
                b.append('    ' + ' ' * d + f'for (int {ax} = 0; {ax} < __ext_{ax}; ++{ax})' + (' {' if d == len(st.reduce_axes) - 1 else ''))
            b.append('      #pragma unroll')
            b.append(f'      for (int __i = 0; __i < {TX}; ++__i) {{')
            b.append('        #pragma unroll')
            b.append(f'        for (int __j = 0; __j < {TY}; ++__j) {{')
            b.append(f'          const int {xa} = __x0 + __i, {ya} = __y0 + __j; (void){xa}; (void){ya};')
            b.append(f'          __acc[__i][__j] = {op}(__acc[__i][__j], ({act})({plain.expr(root)}));')
            b += ['        }', '      }', '    }']
            b.append('    #pragma unroll')
            b.append(f'    for (int __i = 0; __i < {TX}; ++__i) {{')
            b.append('      #pragma unroll')
            b.append(f'      for (int __j = 0; __j < {TY}; ++__j) {{')
            b.append(f'        const int {xa} = __x0 + __i, {ya} = __y0 + __j; (void){xa}; (void){ya};')
            b.append(f'        const {act} __acc_ = __acc[__i][__j];')
            b.append('        ' + result_store('__acc_'))
            b += ['      }', '    }', '  }', '}']
            src.append('\n'.join(b))
            variants['patch'] = sym
            plan.patch, plan.patch_dims = (TX, TY), [ext[xa], ext[ya]]
        mc = _matrix_contraction(st, tensors)
        if mc is not None and tail is not None:
            mc['tail'] = (tail, _matrix_tail(st, tail, mc, tensors))      # lower_graph fuses only what these kernels can take
        if mc is not None:
            src.append(_matrix_kernel(st, tensors, dims, args, written, name + '_m', mc))
            src.append(_matrix_kernel(st, tensors, dims, args, written, name + '_m64', mc, TS=64))
            variants['matrix'], variants['matrix64'] = name + '_m', name + '_m64'
            ext = dict(st.data_axes + st.reduce_axes)
            plan.matrix = {key: [ext[a] for a in mc[key]] for key in ('m', 'n', 'batch', 'k')}
            plan.matrix['half_tiles'] = bool(mc['half'])      # fp16 or int8 tiles: two of the big blocks fit a compute unit
            wide_ok = {t: mc['vec'][t] or mc['rowrun'][t] for t in ('a', 'b')}
            if wide_ok['a'] or wide_ok['b']:
                src.append(_matrix_kernel(st, tensors, dims, args, written, name + '_mv', mc, vectors=True))
                src.append(_matrix_kernel(st, tensors, dims, args, written, name + '_m64v', mc, TS=64, vectors=True))
                variants['matrixv'], variants['matrix64v'] = name + '_mv', name + '_m64v'
                wide = [ITEMSIZE[tensors[mc['l' + t].name].dtype] for t in ('a', 'b') if wide_ok[t]]
                plan.matrix['vec_tensors'] = [mc['l' + t].name for t in ('a', 'b') if wide_ok[t]]
                plan.matrix['vec_width'] = [16 // min(wide)]
                plan.matrix['vec_pitch'] = [mc['pitch'][t] for t in ('a', 'b') if wide_ok[t]] + \
                    [mc['pitch'][t + '_run'] for t in ('a', 'b') if wide_ok[t] and t + '_run' in mc['pitch']]     # row and run lengths, as dimensions to multiply

    return '\n\n'.join(src), plan


def _patch_axes(st):
    """(X, Y) for the register-tiled reduce variant: Y is the last data axis (lanes of a wavefront stay neighbours in
    memory), X the data axis that leaves the most loads constant along X or Y - all of them in a matrix product or a
    convolution.  None when the store is not indexed by the bare data axes, or no load is constant along either."""
    axes = [a for a, _ in st.data_axes]
    if len(axes) < 2 or st.scatter or [i.name for i in st.out_index if i.kind == 'axis'] != axes or len(st.out_index) != len(axes):
        return None
    loads = [n for n in walk(st.root) if n.kind == 'load']
    if not loads or any(n.name == st.output for n in loads):
        return None
    def mentions(n, ax):
        return any(m.kind == 'axis' and m.name == ax for a in n.args for m in walk(a))
    ya = axes[-1]
    best, best_score = None, 0
    for xa in axes[:-1]:
        score = sum(1 for n in loads if not mentions(n, xa) or not mentions(n, ya))
        shared_x = sum(1 for n in loads if not mentions(n, xa))
        if shared_x and score >= best_score:          # later axes win ties: their neighbours are closer in memory
            best, best_score = xa, score
    if best is None or not any(not mentions(n, ya) for n in loads):
        return None
    return best, ya


def _reduce_axis_contiguous(st, tensors) -> Optional[bool]:
    """Looks at the last index of every load: votes, weighted by rank, whether a
    reduce axis or a data axis walks memory contiguously."""
    raxes = {a for a, _ in st.reduce_axes}
    daxes = {a for a, _ in st.data_axes}
    score = 0
    for n in walk(st.root):
        if n.kind == 'load' and n.args:
            names = {m.name for m in walk(n.args[-1]) if m.kind == 'axis'}     # `S * chunk + C` walks memory along C
            w = len(n.args)
            if names & raxes:
                score += w
            elif names & daxes:
                score -= w
    if score == 0:
        return None
    return score > 0


def _tail_of(graph, i: int):
    """The statement behind statement i when it is a map that can be applied where the reduction i stores its results
    (AntaresIR.md:248-250, tail fusion), else None: same data axes, both outputs indexed by them bare and in order, the
    reduction's output read at that very position, by this map only, and not wanted by the caller."""
    if i + 1 >= len(graph.statements):
        return None
    st, nx = graph.statements[i], graph.statements[i + 1]
    if not st.reduce_axes or st.scatter or nx.reduce_axes or nx.scatter or nx.set_op:
        return None
    if (st.root.kind == 'when' and len(st.root.args) == 1) or list(st.data_axes) != list(nx.data_axes) or not st.data_axes:
        return None
    axes = [a for a, _ in st.data_axes]

    def bare(index):
        return [x.name if x.kind == 'axis' else None for x in index] == axes
    t = st.output
    if not bare(st.out_index) or not bare(nx.out_index) or t in graph.outputs or t in graph.declared or nx.output == t:
        return None
    if any(t in s_.reads or s_.output in (t, nx.output) for k, s_ in enumerate(graph.statements) if k not in (i, i + 1)):
        return None
    if nx.output in nx.reads or nx.output in st.reads or t in st.reads:
        return None
    loads = [n for n in walk(nx.root) if n.kind == 'load' and n.name == t]
    if not loads or any(not bare(n.args) for n in loads):
        return None
    mc = _matrix_contraction(st, graph.tensors)
    if mc is not None and _matrix_tail(st, nx, mc, graph.tensors) is None:
        return None                 # the matrix kernels could not take it: two launches beat losing them
    return nx
