"""Contractions on the matrix instructions: recognising a sum of products of two loads whose indices split into a
row / column part and a k part (`_matrix_contraction`), the kernel template with its address tables in LDS
(`_matrix_kernel`), a map fused behind the contraction (`_matrix_tail`) and the k-slicing request
(`contraction_slices`).  Replaces the reference's tiled schedule, backends/c-rocm/schedule/standard/algo_tiling.py:35-98."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

from ..ir.nodes import Expr, ITEMSIZE, walk
from .emit_common import BLOCK, ExprEmitter, HIP_TYPE, _axes_of, _decompose, _extents, _signature



def _matrix_kernel(st, tensors, dims, args, written, sym: str, mc, TS: int = 128, vectors: bool = False) -> str:
    """A sum of products of two loads on v_mfma_f32_32x32x2_f32 (the reference's counterpart: its tiled schedule for
    contractions, backends/c-rocm/schedule/standard/algo_tiling.py:35-98, on the vector units).  A block of 256
    threads = 2 x 2 wavefronts owns 128 rows x 128 columns of one batch, where a row is a point of the axes only
    the first load uses and a column a point of those only the second uses; k runs over the reduce axes in tiles of
    16.  An element's address is (row or column offset) + (k offset): the row, column and output offsets of the tile
    are worked out once into LDS tables, the k offsets once per tile, so the inner loads are a table look-up and an
    add - whatever the index expressions are (a convolution's `HO + KH`, a gathered row, a transposed operand).
    Both operands are staged in LDS as [row or column][k] and fed to the matrix instruction exactly as the fp32
    GEMM kernel of the library feeds it; rows, columns and batches past the extents are clamped on the way in and
    cut on the way out; the k a last partial tile lacks are staged as zeros (their addresses wrap into the
    tensors).  TS = 64 gives blocks of 64 x 64 outputs (a wavefront then owns one 32 x 32 tile): four times the
    blocks for products too small to fill the chip with the big ones.  A guarded operand (AntaresIR.md:166, a padded
    convolution) has the row part and the k part of every compared value tabled the same way and is fetched from
    its own address only where its conditions hold."""
    la, lb = mc['la'], mc['lb']

    def half_cast(f, ld):
        return f.kind == 'cast' and f.dtype == 'float32' and f.args[0] is ld and tensors[ld.name].dtype == 'float16'
    # fp16 operands that are only cast up: the tiles stay fp16 in LDS and go to v_mfma_f32_32x32x16_f16 - the
    # products of two fp16 values are exact in float32 either way, and the matrix time is a sixteenth
    IM = st.root.dtype == 'int32'                     # int8 operands cast to int32: int8 tiles, v_mfma_i32_32x32x32_i8, int32 accumulators
    HM = (half_cast(mc['fa'], la) and half_cast(mc['fb'], lb)) or st.root.dtype == 'float16' or IM      # operands staged as loaded
    BK = 64 if IM else (32 if (TS == 64 or HM) else 16)   # k per tile: the small blocks take twice the k per barrier
    LD, RS = BK + (16 if IM else (8 if HM else 4)), BLOCK // BK       # elements per row of a staged tile (16-byte aligned, rows on distinct banks); rows between a lane's elements when lanes walk k
    ET = 'signed char' if IM else ('half_t' if HM else 'float')      # element type of the staged tiles
    VW = 16 if IM else (8 if HM else 4)               # elements per 16-byte vector of them
    KG = 32 if IM else (16 if HM else 8)              # k one round of matrix instructions multiplies
    ZERO = '0' if IM else '0.f'
    # how an operand travels: 'rows' (lanes along rows, PER k each), 'k' (lanes along k, PER rows each), or 'kvec' (a
    # lane fetches 16 bytes of k of PER / VL rows: rows of k in memory, whole vectors, aligned - the launcher checks)
    def vector_ok(x, ld):       # the staged value must be the loaded one, in the tile's element type
        return vectors and mc['vec'][x] and (HM or (tensors[ld.name].dtype == 'float32' and mc['f' + x] is ld))
    mode = {x: ('kvec' if vector_ok(x, ld) else ('tr' if (vectors and mc['rowrun'][x]) else ('k' if mc['parts'][x][2] else 'rows')))
            for x, ld in (('a', la), ('b', lb))}
    PT = TS + (32 if HM else 8)                       # elements per k row of a tile staged as it lies, [k][row]: the k rows a wavefront reads together start on different banks
    VR = 16 if IM else (8 if HM else 4)               # rows per 16-byte vector of it
    CG = TS // VR                                     # 16-byte groups of rows in such a tile
    KP = BLOCK // CG                                  # k rows of it that one pass of the 256 threads covers
    VL = 16 // ITEMSIZE[tensors[la.name].dtype] if mode['a'] == 'kvec' else (16 // ITEMSIZE[tensors[lb.name].dtype] if mode['b'] == 'kvec' else VW)
    VPR = BK // VL                                    # vectors per row of a tile
    RV = BLOCK // VPR                                 # rows a pass of the 256 threads covers
    NT, PER, HALF = TS // 64, TS * BK // BLOCK, TS // 2   # accumulator tiles per wavefront and direction, elements a thread stages per operand and tile, rows of a wavefront
    DEPTH = 2 if TS == 64 else 1                      # tiles on their way in registers: small blocks have nothing else to hide a load behind
    ta, tb, oct_ = HIP_TYPE[tensors[la.name].dtype], HIP_TYPE[tensors[lb.name].dtype], HIP_TYPE[st.out_dtype]
    plain = ExprEmitter(tensors)
    ext = dict(st.data_axes + st.reduce_axes)
    # A guarded operand (`x[...].when([conditions], 0)`, the padding of a convolution): every compared value is (row
    # part) + (k part) like an address, both parts are tabled beside the offsets, an element is fetched only where all
    # its conditions hold - rows and k are points of the statement's own axes, clamped or wrapped, so a fetch that
    # happens is one the statement makes - and staged as zero where they do not.
    G = mc.get('guards') or {'a': [], 'b': []}
    # the two bounds of a padded index compare the same value: one pair of tables per distinct value
    GV = {x: list(dict.fromkeys((g[0], g[1]) for g in G[x])) for x in 'ab'}

    def holds(x, row, k):       # C text: the compared values of (row slot, k slot), then the conjunction over them
        vals = [f'const int __v{c} = __gm{x}[{c}][{row}] + __gk{x}[__buf][{k}][{c}];' for c in range(len(GV[x]))]
        terms = []
        for qm, qk, op, other, left in G[x]:
            v = f'__v{GV[x].index((qm, qk))}'
            terms.append(f'({v} {op} {other})' if left else f'({other} {op} {v})')
        return ' '.join(vals), ' && '.join(terms)

    def prod(names):
        return ' * '.join(f'(long long)__ext_{a}' for a in names) or '1LL'

    def decompose(var, names, indent, wide=True):
        # 64-bit division costs some hundred instructions; k (walked once per tile by one wavefront, on every
        # other wavefront's way to the barrier) always fits 32 bits
        out = [f'{indent}long long __q = {var};' if wide else f'{indent}unsigned int __q = (unsigned int)({var});']
        for a in reversed(names):
            if wide:
                out.append(f'{indent}const int {a} = (int)(__q % __ext_{a}); __q /= __ext_{a}; (void){a};')
            else:
                out.append(f'{indent}const int {a} = (int)(__q % (unsigned int)__ext_{a}); __q /= (unsigned int)__ext_{a}; (void){a};')
        return out
    out_axes = [a for a, _ in st.data_axes]
    # With a tail (the map statement behind the reduction, applied where a result is stored) the stores go to the tail's
    # output, which is indexed by the same axes in the same order; every other tensor the tail reads is addressed as
    # (row part) + (column part) through two more tables per load.
    tail, extra = mc.get('tail') or (None, [])
    out_name = st.output if tail is None else tail.output
    rows_of_out = plain.offset(out_name, [a if (a in mc['m'] or a in mc['batch']) else '0' for a in out_axes])
    cols_of_out = plain.offset(out_name, [a if a in mc['n'] else '0' for a in out_axes])
    val_a = [ExprEmitter(tensors, load_override=lambda n, j=j: f'__ra[__S][{j}]').expr(mc['fa']) for j in range(PER)]
    val_b = [ExprEmitter(tensors, load_override=lambda n, j=j: f'__rb[__S][{j}]').expr(mc['fb']) for j in range(PER)]
    if HM:
        val_a, val_b = [f'__ra[__S][{j}]' for j in range(PER)], [f'__rb[__S][{j}]' for j in range(PER)]
    def stored(acc):                # C text that stores the result held in `acc` at (row __r, column __c) of the tile
        # results leave as a stream (non-temporal stores: a 1 GiB result of 8 x 32 products of 1024 x 1024 x 128 takes 278 us
        # instead of 342), except the slices of a sliced contraction, which the next kernel reads back at once
        if tail is None and '__part' in st.output:
            return f'{st.output}[__cm[__r] + __cn[__c]] = ({oct_}){acc};'
        if tail is None:
            return f'__builtin_nontemporal_store(({oct_}){acc}, &{st.output}[__cm[__r] + __cn[__c]]);'
        where = {i: f'{ld.name}[__xm{q}[__r] + __xn{q}[__c]]' for q, (ld, _, _, ids) in enumerate(extra) for i in ids}
        tem = ExprEmitter(tensors, load_override=lambda n: '__t' if n.name == st.output else where[id(n)])
        return (f'{{ const {oct_} __t = ({oct_}){acc}; (void)__t; '
                f'__builtin_nontemporal_store(({HIP_TYPE[tail.out_dtype]})({tem.expr(tail.root)}), &{tail.output}[__cm[__r] + __cn[__c]]); }}')
    b = [_signature(sym, args, tensors, dims, written) + ' {'] + _extents(st)
    b += [f'  typedef {"int" if IM else "float"} __f16v __attribute__((ext_vector_type(16)));',
          '  typedef int __i4 __attribute__((ext_vector_type(4)));',
          f'  typedef {ET} __f4 __attribute__((ext_vector_type({VW})));      // 16 bytes of a staged tile',
          f'  __shared__ __attribute__((aligned(16))) {ET} __As[2][{BK * PT if mode["a"] == "tr" else TS * LD}];     // [row][k], {BK} k and 16 bytes of padding per row ([k][row] when staged as it lies)',
          f'  __shared__ __attribute__((aligned(16))) {ET} __Bs[2][{BK * PT if mode["b"] == "tr" else TS * LD}];     // [column][k]',
          '  typedef short __s4 __attribute__((ext_vector_type(4)));',
          '  typedef __attribute__((address_space(3))) __s4 __lds_s4;',
          '  typedef int __i2 __attribute__((ext_vector_type(2)));',
          '  typedef __attribute__((address_space(3))) __i2 __lds_i2;',
          f'  __shared__ long long __am[{TS}], __bn[{TS}], __cm[{TS}], __cn[{TS}], __ak[2][{BK}], __bk[2][{BK}];'] + \
         [f'  __shared__ long long __xm{q}[{TS}], __xn{q}[{TS}];      // row and column part of the offsets into {ld.name} (read by the tail)'
          for q, (ld, _, _, _) in enumerate(extra)] + \
         [f'  __shared__ int __gm{x}[{len(GV[x])}][{TS}], __gk{x}[2][{BK}][{len(GV[x])}];      // the guards of operand {x}: row part and k part of each compared value'
          for x in 'ab' if G[x]] + [
          f'  const long long __M = {prod(mc["m"])}, __N = {prod(mc["n"])}, __B = {prod(mc["batch"])};',
          f'  const long long __K = {prod(mc["k"])};',
          f'  const int __T = (int)((__K + {BK - 1}) / {BK});      // the last tile may be partial: its missing k are staged as zeros',
          f'  const long long __tn_n = (__N + {TS - 1}) / {TS}, __tiles = ((__M + {TS - 1}) / {TS}) * __tn_n;',
          '  const int __tid = threadIdx.x, __lane = __tid & 63, __wave = __tid >> 6, __wm = __wave >> 1, __wn = __wave & 1;',
          '  for (long long __blk = blockIdx.x; __blk < __tiles * __B; __blk += gridDim.x) {',
          '    const long long __t0 = __blk % __tiles, __tm = __t0 / __tn_n, __tn = __t0 % __tn_n;']
    b += _decompose('__blk / __tiles', [(a, None) for a in mc['batch']], '    ', '__B', tmp='__q') if mc['batch'] else []
    b += [f'    if (__tid < {TS}) {{                            // row offsets of the first operand and of the output',
          f'      long long __row = __tm * {TS} + __tid;',
          '      if (__row >= __M) __row = __M - 1;']
    b += _decompose('__row', [(a, None) for a in mc['m']], '      ', '__M', tmp='__q')       # 32-bit divisions whenever the count fits
    b += [f'      __xm{q}[__tid] = {rowpart};' for q, (_, rowpart, _, _) in enumerate(extra)]
    b += [f'      __gma[{c}][__tid] = {g[0]};' for c, g in enumerate(GV['a'])]
    b += [f'      __am[__tid] = {mc["parts"]["a"][0]};', f'      __cm[__tid] = {rows_of_out};',
          f'    }} else if (__tid < {2 * TS}) {{                  // column offsets of the second operand and of the output',
          f'      long long __colq = __tn * {TS} + (__tid - {TS});',
          '      if (__colq >= __N) __colq = __N - 1;']
    b += _decompose('__colq', [(a, None) for a in mc['n']], '      ', '__N', tmp='__q')
    b += [f'      __xn{q}[__tid - {TS}] = {colpart};' for q, (_, _, colpart, _) in enumerate(extra)]
    b += [f'      __gmb[{c}][__tid - {TS}] = {g[0]};' for c, g in enumerate(GV['b'])]
    b += [f'      __bn[__tid - {TS}] = {mc["parts"]["b"][0]};', f'      __cn[__tid - {TS}] = {cols_of_out};',
          '    }',
          f'    auto __ktab = [&](int __kt, int __buf) {{       // k offsets of tile __kt: {BK} for each operand',
          f'      if (__tid < {2 * BK}) {{',
          f'        const long long __kk = (long long)__kt * {BK} + (__tid & {BK - 1});']
    b += decompose('__kk', mc['k'], '        ', wide=False)
    b += [f'        if (__tid < {BK}) {{ __ak[__buf][__tid] = {mc["parts"]["a"][1]}; ' +
          ' '.join(f'__gka[__buf][__tid][{c}] = {g[1]};' for c, g in enumerate(GV['a'])) + ' }',
          f'        else {{ __bk[__buf][__tid - {BK}] = {mc["parts"]["b"][1]}; ' +
          ' '.join(f'__gkb[__buf][__tid - {BK}][{c}] = {g[1]};' for c, g in enumerate(GV['b'])) + ' }',
          '      }',
          '    };',
          '    __ktab(0, 0);',
          '    if (__T > 1) __ktab(1, 1);',
          '    __syncthreads();',
          f'    const int __ml = __tid & {TS - 1}, __kh = (__tid / {TS}) * {PER};     // lanes along rows: {PER} k of one row (column) per thread',
          f'    const int __kl = __tid & {BK - 1}, __rw = __tid / {BK};             // lanes along k: one k of {PER} rows (columns) per thread',
          '    (void)__ml; (void)__kh; (void)__kl; (void)__rw;']
    for x, ld, ct, tab, ktab_, lds, vals in (('a', la, ta, '__am', '__ak', '__As', val_a), ('b', lb, tb, '__bn', '__bk', '__Bs', val_b)):
        if mode[x] == 'kvec':
            b += [f'    typedef {ct} __v{x} __attribute__((ext_vector_type({VL})));',
                  f'    const {ct}* __p{x}[{TS // RV}];', '    #pragma unroll',
                  f'    for (int __j = 0; __j < {TS // RV}; ++__j) __p{x}[__j] = {ld.name} + {tab}[__tid / {VPR} + {RV} * __j];',
                  f'    __v{x} __r{x}[{DEPTH}][{TS // RV}];']
            continue
        if mode[x] == 'tr':
            # a lane owns 8 neighbouring rows (a whole vector: all inside the extents or all past them) and every KP-th k;
            # the last of them names the address, so that a group past the end re-reads the last whole vector
            b += [f'    typedef {ct} __w{x} __attribute__((ext_vector_type({VR})));',
                  f'    const {ct}* __p{x} = {ld.name} + ({tab}[(__tid % {CG}) * {VR} + {VR - 1}] - {VR - 1});',
                  f'    __w{x} __r{x}[{DEPTH}][{BK // KP}];']
            continue
        if mode[x] == 'k':
            b += [f'    const {ct}* __p{x}[{PER}];', '    #pragma unroll',
                  f'    for (int __j = 0; __j < {PER}; ++__j) __p{x}[__j] = {ld.name} + {tab}[__rw + {RS} * __j];']
        else:
            b.append(f'    const {ct}* __p{x} = {ld.name} + {tab}[__ml];')
        b.append(f'    {ct} __r{x}[{DEPTH}][{PER}];')
        if G[x]:
            b.append(f'    unsigned int __g{x}[{DEPTH}];              // bit j: element j of the set is inside its guards')
    b += ['    auto __load = [&](auto __set, int __buf, int __ktile) {', '      constexpr int __S = decltype(__set)::value; (void)__ktile;']
    for x, ktab_ in (('a', '__ak'), ('b', '__bk')):
        if mode[x] == 'kvec':       # a vector starts where its first k does (the table; k past the end wraps to valid ones, staged as zeros)
            b += [f'      {{ const long long __ko = {ktab_}[__buf][(__tid % {VPR}) * {VL}];', '        #pragma unroll',
                  f'        for (int __j = 0; __j < {TS // RV}; ++__j) __r{x}[__S][__j] = *(const __v{x}*)(__p{x}[__j] + __ko); }}']
            continue
        if mode[x] == 'tr':
            b += ['      #pragma unroll',
                  f'      for (int __j = 0; __j < {BK // KP}; ++__j) __r{x}[__S][__j] = *(const __w{x}*)(__p{x} + {ktab_}[__buf][__tid / {CG} + {KP} * __j]);']
            continue
        if G[x]:
            row, k = (f'__rw + {RS} * __j', '__kl') if mode[x] == 'k' else ('__ml', '__kh + __j')
            at = f'__p{x}[__j] + {ktab_}[__buf][__kl]' if mode[x] == 'k' else f'__p{x} + {ktab_}[__buf][__kh + __j]'
            b += [f'      {{ unsigned int __in = 0u;', '        #pragma unroll',
                  f'        for (int __j = 0; __j < {PER}; ++__j) {{',
                  f'          {holds(x, row, k)[0]}',
                  f'          const bool __h = {holds(x, row, k)[1]};',
                  f'          __r{x}[__S][__j] = *(__h ? {at} : {(la if x == "a" else lb).name});       // outside: the tensor\'s first element, not used',
                  '          __in |= (unsigned int)__h << __j;', '        }', f'        __g{x}[__S] = __in; }}']
        elif mode[x] == 'k':
            b += [f'      {{ const long long __ko = {ktab_}[__buf][__kl];', '        #pragma unroll',
                  f'        for (int __j = 0; __j < {PER}; ++__j) __r{x}[__S][__j] = __p{x}[__j][__ko]; }}']
        else:
            b += ['      #pragma unroll', f'      for (int __j = 0; __j < {PER}; ++__j) __r{x}[__S][__j] = __p{x}[{ktab_}[__buf][__kh + __j]];']
    b += ['    };', '    auto __stage = [&](auto __set, int __buf, int __kt) {', '      constexpr int __S = decltype(__set)::value; (void)__S;']
    for x, lds, vals in (('a', '__As', val_a), ('b', '__Bs', val_b)):
        if mode[x] == 'kvec':
            b += [f'      {{ const bool __in = (long long)__kt * {BK} + (__tid % {VPR}) * {VL} + {VL} <= __K;']
            for j in range(TS // RV):
                dst = f'&{lds}[__buf][(__tid / {VPR} + {RV * j}) * {LD} + (__tid % {VPR}) * {VL}]'
                b += [f'        *(__v{x}*){dst} = __in ? __r{x}[__S][{j}] : (__v{x})(0);']
            b += ['      }']
            continue
        if mode[x] == 'tr':
            for j in range(BK // KP):
                b += [f'      {{ const int __ks = __tid / {CG} + {KP * j};',
                      f'        *(__w{x}*)&{lds}[__buf][__ks * {PT} + (__tid % {CG}) * {VR}] = (long long)__kt * {BK} + __ks < __K ? __r{x}[__S][{j}] : (__w{x})(0); }}']
            continue
        def inside(j, x=x):
            return f' && ((__g{x}[__S] >> {j}) & 1u)' if G[x] else ''
        if mode[x] == 'k':
            b += [f'      {{ const bool __in = (long long)__kt * {BK} + __kl < __K;']
            b += [f'        {lds}[__buf][(__rw + {RS * j}) * {LD} + __kl] = __in{inside(j)} ? ({ET})({vals[j]}) : ({ET})0.f;' for j in range(PER)]
            b += ['      }']
        else:
            def guarded(j):
                return f'(__k0 + {j} < __K{inside(j)} ? ({ET})({vals[j]}) : ({ET})0.f)'
            b += [f'      {{ const long long __k0 = (long long)__kt * {BK} + __kh;']
            for q in range(PER // VW):
                b += [f'        *(__f4*)&{lds}[__buf][__ml * {LD} + __kh + {VW * q}] = __f4{{' + ', '.join(guarded(VW * q + e) for e in range(VW)) + '};']
            b += ['      }']
    def feed(x, lds, w):            # C text that fetches operand x of accumulator tile __i for round __g
        if mode[x] != 'tr':
            base = '__row0' if x == 'a' else '__col0'
            return f'          __{x}[__i] = *(const __f4*)&{lds}[__buf][({base} + 32 * __i) * {LD} + __g * {KG} + __kq];'
        # 16 lanes read a patch of 4 k x 16 rows and each receives the four k of one row; two patches, 4 k apart, make
        # the 8 consecutive k a lane supplies: k = (lane / 32) * 8 .. + 7, row = lane % 32 of the tile - as above
        if not HM:  # float32 needs no transposing read: four 4-byte reads, k = g * 8 + (lane / 32) * 4 + m for instruction m
            at = f'{lds}[__buf][(__g * 8 + __kq + %d) * {PT} + {w} * {HALF} + 32 * __i + (__lane & 31)]'
            return f'          __{x}[__i] = __f4{{' + ', '.join(at % m for m in range(4)) + '};'
        if IM:      # 16 lanes read a patch of 8 k x 16 rows (a lane supplies 8 bytes of one k) and each receives the 8 k of one row
            at = f'&{lds}[__buf][(__g * 32 + __tq) * {PT} + {w} * {HALF} + 32 * __i + __tc]'
            return (f'          {{ const __i2 __lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__lds_i2*)({at})), '
                    f'__hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__lds_i2*)({at} + 8 * {PT}));\n'
                    f'            __{x}[__i] = __builtin_bit_cast(__f4, __i4{{__lo[0], __lo[1], __hi[0], __hi[1]}}); }}')
        at = f'&{lds}[__buf][(__g * 16 + __tq) * {PT} + {w} * {HALF} + 32 * __i + __tc]'
        return (f'          {{ const __s4 __lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__lds_s4*)({at})), '
                f'__hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__lds_s4*)({at} + 4 * {PT}));\n'
                f'            typedef half_t __h4 __attribute__((ext_vector_type(4)));\n'
                f'            const __h4 __l = __builtin_bit_cast(__h4, __lo), __h = __builtin_bit_cast(__h4, __hi);\n'
                f'            __{x}[__i] = __f4{{__l[0], __l[1], __l[2], __l[3], __h[0], __h[1], __h[2], __h[3]}}; }}')
    b += ['    };',
          f'    __f16v __acc[{NT}][{NT}];',
          '    #pragma unroll',
          f'    for (int __i = 0; __i < {NT}; ++__i)',
          '      #pragma unroll',
          f'      for (int __j = 0; __j < {NT}; ++__j)',
          '        #pragma unroll',
          f'        for (int __e = 0; __e < 16; ++__e) __acc[__i][__j][__e] = {ZERO};',
          f'    const int __row0 = __wm * {HALF} + (__lane & 31), __col0 = __wn * {HALF} + (__lane & 31), __kq = (__lane >> 5) * {VW};',
          ('    const int __tq = (__lane >> 5) * 16 + ((__lane & 15) >> 1), __tc = ((__lane & 31) >> 4) * 16 + (__lane & 1) * 8; (void)__tq; (void)__tc;' if IM else
           '    const int __tq = (__lane >> 5) * 8 + ((__lane & 15) >> 2), __tc = ((__lane & 31) >> 4) * 16 + (__lane & 3) * 4; (void)__tq; (void)__tc;'),
          '    auto __multiply = [&](int __buf) {',
          '      #pragma unroll',
          f'      for (int __g = 0; __g < {BK // KG}; ++__g) {{',
          f'        __f4 __a[{NT}], __b[{NT}];',
          '        #pragma unroll',
          f'        for (int __i = 0; __i < {NT}; ++__i) {{',
          feed('a', '__As', '__wm'),
          feed('b', '__Bs', '__wn'),
          '        }']
    if IM:      # a lane supplies 16 consecutive k of its row (column), the same ones for both operands
        b += ['        #pragma unroll',
              f'        for (int __i = 0; __i < {NT}; ++__i)',
              '          #pragma unroll',
              f'          for (int __j = 0; __j < {NT}; ++__j)',
              '            __acc[__i][__j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(__i4, __a[__i]), __builtin_bit_cast(__i4, __b[__j]), __acc[__i][__j], 0, 0, 0);']
    elif HM:    # a lane supplies 8 consecutive k of its row (column): k = (lane / 32) * 8 .. + 7 of the 16
        b += ['        #pragma unroll',
              f'        for (int __i = 0; __i < {NT}; ++__i)',
              '          #pragma unroll',
              f'          for (int __j = 0; __j < {NT}; ++__j)',
              '            __acc[__i][__j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__a[__i], __b[__j], __acc[__i][__j], 0, 0, 0);']
    else:       # instruction m multiplies k = m (lanes 0-31) and k = 4 + m (lanes 32-63) of the 8
        b += ['        #pragma unroll',
              '        for (int __m = 0; __m < 4; ++__m)',
              '          #pragma unroll',
              f'          for (int __i = 0; __i < {NT}; ++__i)',
              '            #pragma unroll',
              f'            for (int __j = 0; __j < {NT}; ++__j)',
              '              __acc[__i][__j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__a[__i][__m], __b[__j][__m], __acc[__i][__j], 0, 0, 0);']
    b += ['      }',
          '    };']
    if DEPTH == 1:
        b += ['    __load(art_ic<0>{}, 0, 0);',
              '    __stage(art_ic<0>{}, 0, 0);',
              '    __syncthreads();',
              '    for (int __t = 0; __t < __T; ++__t) {',
              '      const int __buf = __t & 1;',
              '      if (__t + 1 < __T) __load(art_ic<0>{}, __buf ^ 1, __t + 1);    // tile t + 1 travels while tile t is multiplied',
              '      if (__t + 2 < __T) __ktab(__t + 2, __buf);            // its k offsets were read a tile ago',
              '      __multiply(__buf);',
              '      if (__t + 1 < __T) __stage(art_ic<0>{}, __buf ^ 1, __t + 1);   // the other buffer: everybody left it at the last barrier',
              '      __syncthreads();',
              '    }']
    else:
        b += ['    // Tile t is multiplied out of LDS buffer t % 2 and came through register set t % 2.  While it is multiplied,',
              '    // tile t + 1 waits in the other register set and tile t + 2 is asked for into the set tile t has left; the k',
              '    // offsets of tile t + 3 go into the table that the loads of tile t + 1 read one barrier ago.',
              '    __load(art_ic<0>{}, 0, 0);',
              '    if (__T > 1) __load(art_ic<1>{}, 1, 1);',
              '    __syncthreads();                               // everybody has read the k offsets of tile 0',
              '    if (__T > 2) __ktab(2, 0);',
              '    __stage(art_ic<0>{}, 0, 0);',
              '    __syncthreads();',
              '    for (int __t = 0; __t < __T; __t += 2) {',
              '      if (__t + 2 < __T) __load(art_ic<0>{}, 0, __t + 2);',
              '      if (__t + 3 < __T) __ktab(__t + 3, 1);',
              '      __multiply(0);',
              '      if (__t + 1 < __T) __stage(art_ic<1>{}, 1, __t + 1);    // the other buffer: everybody left it at the last barrier',
              '      __syncthreads();',
              '      if (__t + 1 < __T) {',
              '        if (__t + 3 < __T) __load(art_ic<1>{}, 1, __t + 3);',
              '        if (__t + 4 < __T) __ktab(__t + 4, 0);',
              '        __multiply(1);',
              '        if (__t + 2 < __T) __stage(art_ic<0>{}, 0, __t + 2);',
              '        __syncthreads();',
              '      }',
              '    }']
    b += [
          '    // accumulator element e of tile (i, j): row i*32 + (e/4)*8 + (lane/32)*4 + e%4, column j*32 + lane%32',
          '    #pragma unroll',
          f'    for (int __i = 0; __i < {NT}; ++__i)',
          '      #pragma unroll',
          f'      for (int __j = 0; __j < {NT}; ++__j) {{',
          f'        const int __c = __wn * {HALF} + __j * 32 + (__lane & 31);',
          '        #pragma unroll',
          '        for (int __e = 0; __e < 16; ++__e) {',
          f'          const int __r = __wm * {HALF} + __i * 32 + (__e >> 2) * 8 + (__lane >> 5) * 4 + (__e & 3);',
          f'          if (__tm * {TS} + __r < __M && __tn * {TS} + __c < __N) {stored("__acc[__i][__j][__e]")}',
          '        }',
          '      }',
          '    __syncthreads();                               // the tables and buffers are rewritten by the next tile',
          '  }', '}']
    return '\n'.join(b)


def _split_index(e: Expr, em: ExprEmitter, outer: set, inner: set):
    """An index expression as (part that depends on `outer` axes only, part that depends on `inner` axes only), each
    as C text or None, when it is one of the two or a sum of such parts; else None."""
    used = _axes_of(e)
    if used <= outer:
        return em.expr(e), None
    if used <= inner:
        return None, em.expr(e)
    if e.kind == 'op' and e.name == '+' and len(e.args) == 2:
        l, r = _split_index(e.args[0], em, outer, inner), _split_index(e.args[1], em, outer, inner)
        if l is None or r is None:
            return None

        def add(x, y):
            return y if x is None else (x if y is None else f'({x}) + ({y})')
        return add(l[0], r[0]), add(l[1], r[1])
    if e.kind == 'op' and e.name == '-' and len(e.args) == 2:
        l, r = _split_index(e.args[0], em, outer, inner), _split_index(e.args[1], em, outer, inner)
        if l is None or r is None:
            return None

        def sub(x, y):
            return x if y is None else (f'-({y})' if x is None else f'({x}) - ({y})')
        return sub(l[0], r[0]), sub(l[1], r[1])
    return None


def _matrix_contraction(st, tensors):
    """Reads a sum of products of two factors, one load each, as a matrix product on the fp32 matrix instructions:
    data axes that only the first load uses are rows (M), those only the second uses are columns (N), those both use
    are a batch, the reduce axes are k.  Every index of a load must split into a part that depends on k axes and a
    part that does not, so that an element's address is a row (column) offset plus a k offset.  -> dict or None."""
    if st.scatter or st.reduce != '+' or st.root.dtype not in ('float32', 'float16', 'int32') or not st.reduce_axes or not st.data_axes:
        return None
    root = st.root
    if root.kind == 'when' or root.kind != 'op' or root.name != '*' or len(root.args) != 2:
        return None
    axes = [a for a, _ in st.data_axes]
    if [i.name if i.kind == 'axis' else None for i in st.out_index] != axes:
        return None
    fa, fb = root.args
    # a factor may be guarded: `x[...].when([conditions], 0)` - the padding of a convolution
    guards = {'a': [], 'b': []}
    for tag in ('a', 'b'):
        f = fa if tag == 'a' else fb
        if f.kind == 'when':
            zero = len(f.args) == 2 and f.args[1].kind == 'const' and f.args[1].value == 0
            if not zero or f.merge != 'all':
                return None
            guards[tag] = list(f.conds)
            if tag == 'a':
                fa = f.args[0]
            else:
                fb = f.args[0]
    la, lb = [n for n in walk(fa) if n.kind == 'load'], [n for n in walk(fb) if n.kind == 'load']
    if len(la) != 1 or len(lb) != 1 or st.output in (la[0].name, lb[0].name):
        return None
    la, lb = la[0], lb[0]
    if any(n.kind in ('load', 'when') for tag in guards for c in guards[tag] for n in walk(c)):
        return None
    # A float16 statement (AntaresIR.md:115 with float16 tensors; the reference rounds every product and every partial
    # sum to float16) is taken only as the product of two float16 loads: the matrix instruction multiplies them
    # exactly and sums in float32, the result is rounded once - closer to the exact sum than the running float16 sum.
    if st.root.dtype == 'float16' and not (fa is la and fb is lb and tensors[la.name].dtype == tensors[lb.name].dtype == 'float16'):
        return None
    # An int32 statement is taken as the product of two int8 loads cast to int32: v_mfma_i32_32x32x32_i8 multiplies and
    # sums them exactly, and integer sums do not depend on their order - the result is the reference's, bit for bit.
    if st.root.dtype == 'int32' and not all(f.kind == 'cast' and f.dtype == 'int32' and f.args[0] is ld and tensors[ld.name].dtype == 'int8'
                                            for f, ld in ((fa, la), (fb, lb))):
        return None
    # axes may be used inside the indices of the two loads and inside the guards only
    inside = sum(1 for n in (la, lb) for a in n.args for m in walk(a) if m.kind == 'axis') + \
        sum(1 for tag in guards for c in guards[tag] for m in walk(c) if m.kind == 'axis')
    if sum(1 for m in walk(root) if m.kind == 'axis') != inside:
        return None
    ua, ub = set().union(*[_axes_of(a) for a in la.args]), set().union(*[_axes_of(a) for a in lb.args])
    # The lanes of a wavefront hold neighbouring COLUMNS of the result: the factor that uses the output's last axis
    # is made the second one (the product commutes exactly), so that stores run along memory - a convolution's
    # `output0[N, F, HO, WO]` is then written along WO, not in pieces a feature map apart.
    if axes[-1] in ua and axes[-1] not in ub:
        fa, fb, la, lb, ua, ub = fb, fa, lb, la, ub, ua
        guards = {'a': guards['b'], 'b': guards['a']}
    k_axes = [a for a, _ in st.reduce_axes]
    if not set(k_axes) <= ua or not set(k_axes) <= ub:
        return None
    m_axes = [a for a in axes if a in ua and a not in ub]
    n_axes = [a for a in axes if a in ub and a not in ua]
    batch = [a for a in axes if a in ua and a in ub]
    if not m_axes or not n_axes or len(m_axes) + len(n_axes) + len(batch) != len(axes):
        return None
    if any(ITEMSIZE[tensors[ld.name].dtype] not in ((1,) if st.root.dtype == 'int32' else (2, 4)) for ld in (la, lb)):
        return None
    plain = ExprEmitter(tensors)
    parts = {}
    for tag, ld, own in (('a', la, m_axes), ('b', lb, n_axes)):
        outer, inner = set(own) | set(batch), set(k_axes)
        sp = [_split_index(ix, plain, outer, inner) for ix in ld.args]
        if any(x is None for x in sp):
            return None
        # lanes walk k when the operand's last index is made of k axes alone (k is then the contiguous axis), else rows
        parts[tag] = (plain.offset(ld.name, [x[0] or '0' for x in sp]), plain.offset(ld.name, [x[1] or '0' for x in sp]),
                      sp[-1][0] is None)
        # a guard compares an expression that splits the same way with something free of axes
        conds = []
        for c in guards[tag]:
            if c.kind != 'op' or c.name not in ('<', '<=', '>', '>=', '==', '!=') or len(c.args) != 2:
                return None
            left = bool(_axes_of(c.args[0]))
            if left == bool(_axes_of(c.args[1])):
                return None
            sp_c = _split_index(c.args[0 if left else 1], plain, outer, inner)
            if sp_c is None:
                return None
            conds.append((sp_c[0] or '0', sp_c[1] or '0', c.name, plain.expr(c.args[1 if left else 0]), left))
        guards[tag] = conds
    # an operand whose last indices are THE reduce axes, bare and in their order, over dimensions of exactly their
    # extents (`input1[F, C, KH, KW]` of a convolution; the `[N, K]` of a product), lies in memory as rows of k:
    # 16-byte vectors of k can be fetched when k is a multiple of the vector and the tensor is aligned
    # The first of them may be one slice of a longer axis, `S * chunk + Kc` with the slice S a batch axis and chunk the
    # extent of Kc (what slicing a contraction leaves): a row of the slice is still a run of k, starting a whole number
    # of slices into a row of the tensor.  `pitch` is the row length of the tensor, which must be whole vectors too.
    vec, pitch = {}, {}
    red = dict(st.reduce_axes)

    def bare_or_slice(ix, k):
        if ix.kind == 'axis':
            return ix.name == k
        if ix.kind == 'op' and ix.name == '+' and len(ix.args) == 2:
            sl, ax = ix.args
            return (ax.kind == 'axis' and ax.name == k and sl.kind == 'op' and sl.name == '*' and len(sl.args) == 2 and
                    sl.args[0].kind == 'axis' and sl.args[0].name in batch and sl.args[1].kind == 'const' and sl.args[1].value == red[k])
        return False
    for tag, ld in (('a', la), ('b', lb)):
        nk = len(k_axes)
        tail = ld.args[-nk:] if len(ld.args) >= nk else []
        vec[tag] = (len(tail) == nk and bare_or_slice(tail[0], k_axes[0]) and
                    all(ix.kind == 'axis' and ix.name == k for ix, k in zip(tail[1:], k_axes[1:])) and
                    not any(set(k_axes) & _axes_of(a) for a in ld.args[:-nk]) and
                    all(d == red[k] for d, k in zip(tensors[ld.name].shape[-nk + 1:] if nk > 1 else [], k_axes[1:])) and
                    (tail[0].kind != 'axis' or tensors[ld.name].shape[-nk] == red[k_axes[0]]) and not guards[tag])
        pitch[tag] = list(tensors[ld.name].shape[-nk:])
        # ... or at least its last index is the fastest reduce axis, bare (the channels of an image stored
        # `[N, H, W, C]`): a vector is then a run of that axis, which the launcher wants in whole vectors, like the rows
        if not vec[tag] and not guards[tag] and ld.args[-1].kind == 'axis' and ld.args[-1].name == k_axes[-1] and \
                not any(k_axes[-1] in _axes_of(a) for a in ld.args[:-1]):
            vec[tag] = True
            pitch[tag] = [tensors[ld.name].shape[-1]]
            runs = [red[k_axes[-1]]]
            if runs != pitch[tag]:
                pitch[tag + '_run'] = runs
    # The other way round, for fp16 tiles: an operand whose last index is its fastest row (column) axis, bare, over a
    # dimension of exactly that extent (`input1[K, M]` of a product, V of an attention) has neighbouring rows next to
    # each other in memory.  It is fetched in 16-byte vectors of rows, staged as it lies ([k][row]) and transposed on
    # its way out of LDS (ds_read_b64_tr_b16), when that extent is whole vectors.
    half = st.root.dtype == 'float16' or all(f.kind == 'cast' and f.dtype == 'float32' and f.args[0] is ld and tensors[ld.name].dtype == 'float16'
                                             for f, ld in ((fa, la), (fb, lb)))
    rowrun = {}
    for tag, ld, own in (('a', la, m_axes), ('b', lb, n_axes)):
        last = ld.args[-1]
        ext_own = dict(st.data_axes)[own[-1]]
        plain32 = (fa if tag == 'a' else fb) is ld and tensors[ld.name].dtype == 'float32' and not half
        rowrun[tag] = ((half or st.root.dtype == 'int32' or plain32) and not vec[tag] and not guards[tag] and not parts[tag][2] and last.kind == 'axis' and last.name == own[-1] and
                       not any(own[-1] in _axes_of(a) for a in ld.args[:-1]) and tensors[ld.name].shape[-1] == ext_own)
        if rowrun[tag]:
            pitch[tag] = [ext_own]
    return {'fa': fa, 'fb': fb, 'la': la, 'lb': lb, 'm': m_axes, 'n': n_axes, 'batch': batch, 'k': k_axes, 'parts': parts, 'vec': vec,
            'guards': guards, 'pitch': pitch, 'rowrun': rowrun, 'half': half or st.root.dtype == 'int32'}


def _matrix_tail(st, tail, mc, tensors):
    """What the matrix kernels need to apply `tail` at their stores: [(load, row part, column part)] for every load of
    another tensor than the reduction's output - its offset must be a sum of a part made of row (and batch) axes and a
    part made of column axes, like the output's own - or None when the tail cannot be applied there (a conditional
    store, an axis used as a value, an index that mixes rows and columns, more than four such loads)."""
    if tail.root.kind == 'when' and len(tail.root.args) == 1:
        return None
    plain = ExprEmitter(tensors)
    loads = [n for n in walk(tail.root) if n.kind == 'load' and n.name != st.output]
    inside = sum(1 for n in walk(tail.root) if n.kind == 'load' for a in n.args for m in walk(a) if m.kind == 'axis')
    if sum(1 for m in walk(tail.root) if m.kind == 'axis') != inside:
        return None
    if any(m.kind == 'load' for n in loads for a in n.args for m in walk(a)):
        return None                 # a gathered index would be counted as a load of its own
    rows, cols = set(mc['m']) | set(mc['batch']), set(mc['n'])
    out, seen = [], {}
    for ld in loads:
        sp = [_split_index(ix, plain, rows, cols) for ix in ld.args]
        if any(x is None for x in sp):
            return None
        entry = (ld, plain.offset(ld.name, [x[0] or '0' for x in sp]), plain.offset(ld.name, [x[1] or '0' for x in sp]))
        key = (ld.name,) + entry[1:]
        if key in seen:             # the same element read twice (`x.when(x > 0, 0)`): one pair of tables
            seen[key].append(id(ld))
            continue
        seen[key] = [id(ld)]
        out.append(entry + (seen[key],))
    if len(out) > 4:
        return None
    return out


def contraction_slices(tensors):
    """-> wanted(statement, value) for split_wide_reductions: how many slices of k a contraction on the matrix
    instructions should be cut into, or None.  Blocks of 64 x 64 outputs that number fewer than two per compute unit
    leave a wavefront alone on its SIMD with nothing to hide its loads behind; with at least 1024 values of k the
    product is cut into up to 8 slices (each at least 256 long) that run as a batch and are summed by a second
    statement - 16 bytes more traffic per output and slice, against a main loop that fills the chip."""
    def wanted(st, value):
        if '__part' in st.output:
            return None
        mc = _matrix_contraction(st, tensors)
        if mc is None:
            return None
        ext = dict(st.data_axes + st.reduce_axes)

        def prod(names):
            n = 1
            for a in names:
                n *= value(ext[a])
            return n
        M, N, B, K = prod(mc['m']), prod(mc['n']), prod(mc['batch']), prod(mc['k'])
        blocks = ((M + 63) // 64) * ((N + 63) // 64) * B
        if M < 32 or N < 32 or blocks < 16 or blocks >= 512 or K < 1024:
            return None
        slices = min(8, K // 256, (1024 + blocks - 1) // blocks)
        return slices if slices >= 2 else None
    return wanted
