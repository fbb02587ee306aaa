"""Generic lowering of einstein_v2 statements to HIP kernels for gfx950.

Replaces the reference's TVM-driven code generation for the c-rocm backend
(antares/default_codegen.py:13-358 with the three schedules under
backends/c-rocm/schedule/standard/) by direct emission from hand-written
templates:

* elementwise / gather statements: one flat grid-stride loop; when every tensor
  is read and written at the same flat position the kernel moves 16-byte
  vectors per lane, and so it does when every load is a run along the last
  axis or constant along it (bias rows, gathered rows: `table[ids[N], C]`)
  (the reference's untuned default is one scalar element per block,
  antares/common.py:81-100); a copy whose store walks memory along another
  axis than its load goes through 64 x 64 tiles in LDS, with 16-byte vectors
  on both sides when the tiles are whole and the tensors aligned;
* reduce statements: variants compiled together — one wavefront per
  output (DPP / readlane reduction), one 256-thread block per output, one
  thread per output, and for contractions one thread per 4 x 4 patch of
  outputs (register tiling: operands that are constant along one of the two
  tiled axes are loaded once per patch), and for float32 sums of products of
  two loads whose indices split into a row / column part and a k part (matrix
  products in any layout, batched, convolutions) a kernel on the fp32 matrix
  instructions with its address arithmetic in LDS tables — and the launcher picks by extents
  and by which axis is contiguous in memory (the reference reduces through LDS because its TVM patch
  disables wavefront shuffles off CUDA, engine/device-stub/tvm_v0.8.0.patch:186-191);
* scatter statements: one thread per point of the iteration space, atomics for
  ``+=.  <=.  >=.``;
* runs of statements that reduce over the last axis of a row and then map over
  the row with the results (softmax, layer normalisation) get, besides their
  own kernels, one kernel that does the whole run with a block per row.

Kernel signatures follow the reference's HIP kernel ABI
(backends/c-rocm/config.py:25-85): tensor pointers first, in the order given by
the caller, then the named run-time dimensions as ``int`` arguments.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

from ..ir.nodes import Expr, ITEMSIZE, walk
from .hip_prelude import PRELUDE

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


@dataclass
class RowGroup:
    """A run of statements that one kernel computes row by row: reductions over the last axis of a row followed by
    the map that uses their results (softmax, layer normalisation, AntaresIR.md:226-232)."""
    symbol: str                    # the kernel for rows of any length: a block per row, the row walked per statement
    args: List[str]                # inputs (sorted), then the reduce results in statement order, then the map's output
    count: int                     # statements covered, starting with the one that carries the group
    row_axes: List[Tuple[str, object]]
    red_axis: Tuple[str, object]
    # kernels that keep the row in registers: (lanes per row: 64 or 256, elements per vector, vectors per lane, symbol)
    cached: List[Tuple[int, int, int, str]] = field(default_factory=list)
    vec_tensors: List[str] = field(default_factory=list)   # tensors that must be 16-byte aligned for the vector kernels
    pure: bool = False             # reductions only, no map behind them

    def _extents(self, env: Dict[str, int]) -> Tuple[int, int]:
        e = self.red_axis[1]
        n = e if isinstance(e, int) else env[e]
        rows = 1
        for _, e in self.row_axes:
            rows *= e if isinstance(e, int) else env[e]
        return rows, n

    def choose(self, env: Dict[str, int], pointers: Dict[str, int]) -> Tuple[str, int]:
        """-> (kernel symbol, grid.x) for these extents and addresses; grid 0 when the per-statement kernels do
        better (rows shorter than two wavefronts leave most lanes idle).  Among the kernels that hold a row of this
        length in registers: 16-byte vectors when the row length and the addresses allow, a wavefront per row when
        there are enough rows to fill the chip that way (no barriers), else a block per row."""
        rows, n = self._extents(env)
        if n < 128 or rows == 0:
            return self.symbol, 0
        aligned = all(pointers[t] % 16 == 0 for t in self.vec_tensors)
        fits = [(team, v, e, sym) for team, v, e, sym in self.cached
                if n <= team * v * e and (v == 1 or (aligned and n % v == 0))]
        if not self.pure and rows < 64 and n > 65536:
            return self.symbol, 0          # a handful of very long rows: too few blocks; the statements run one by one
        if self.pure and rows < 512 and not (fits and rows * n <= 65536):
            # few long rows: slicing them first (split_wide_reductions) fills the chip; what is left of a sliced
            # reduction - a few rows that fit in registers - is one short launch with every load in flight
            return self.symbol, 0
        if not fits:
            return self.symbol, min(rows, MAX_GRID)
        vmax = max(v for _, v, _, _ in fits)
        fits = [f for f in fits if f[1] == vmax]
        waves = [f for f in fits if f[0] == 64]
        if waves and rows >= 8192:
            pick = min(waves, key=lambda f: f[2])
        else:
            blocks = [f for f in fits if f[0] == BLOCK] or fits
            pick = min(blocks, key=lambda f: f[2])
        per_block = BLOCK // pick[0]
        return pick[3], min((rows + per_block - 1) // per_block, MAX_GRID)


@dataclass
class KernelPlan:
    """Everything the runtime needs to launch one statement."""
    name: str                      # base kernel name
    args: List[str]                # tensor argument order
    dims: List[str]                # named dimensions passed after the tensors
    variants: Dict[str, str]       # variant tag -> kernel symbol
    kind: str                      # 'map' | 'reduce' | 'scatter'
    output: str
    data_axes: List[Tuple[str, object]]
    reduce_axes: List[Tuple[str, object]]
    vec: int = 1                   # elements per lane in the vector variant
    vec_tensors: List[str] = field(default_factory=list)   # tensors that must be 16-byte aligned for it
    row_vec: int = 1               # elements per lane in the row-vector variant (vectors along the last data axis)
    row_tensors: List[str] = field(default_factory=list)   # tensors that must be 16-byte aligned for it
    row_dims: List[object] = field(default_factory=list)    # extents (int or dimension name) that must be multiples of row_vec
    reduce_contiguous: Optional[bool] = None   # True: a reduce axis is fastest in the biggest operand
    patch: Optional[Tuple[int, int]] = None    # outputs per thread of the register-tiled reduce variant, along patch_dims
    patch_dims: List[object] = field(default_factory=list)   # the two extents (int or dimension name) it tiles
    tile_axes: Optional[Tuple[str, str]] = None   # permutation copies: last axis of the load, last axis of the store
    tile_tensors: List[str] = field(default_factory=list)   # tensors that must be 16-byte aligned for the vector form of it
    row_group: Optional[RowGroup] = None          # set on the first statement of a run that one row kernel can compute
    matrix: Optional[Dict[str, List[object]]] = None   # matrix-instruction variant: extents of its row, column, batch and k axes (and what its vector form needs)
    covers: int = 1                # statements these kernels compute: 2 when the map behind a reduction is applied at its store

    def _tiles(self, env: Dict[str, int]) -> int:
        """64 x 64 tiles of the transposing variant, 0 when it does not apply or an axis is too short to pay."""
        if self.tile_axes is None or 'tile' not in self.variants:
            return 0
        n = 1
        for ax, e in self.data_axes:
            v = e if isinstance(e, int) else env[e]
            if ax in self.tile_axes:
                if v < 16:
                    return 0
                n *= (v + 63) // 64
            else:
                n *= v
        return n

    def _vector_tiles(self, env: Dict[str, int], pointers: Dict[str, int]) -> int:
        """Tiles of the transposing variant that moves 16-byte vectors on both sides: whole 64 x 64 tiles only."""
        if self.tile_axes is None or 'tilevec' not in self.variants or any(pointers[t] % 16 for t in self.tile_tensors):
            return 0
        n = 1
        for ax, e in self.data_axes:
            v = e if isinstance(e, int) else env[e]
            if ax in self.tile_axes:
                if v % 64:
                    return 0
                n *= v // 64
            else:
                n *= v
        return n

    def _row_vectors(self, env: Dict[str, int], pointers: Dict[str, int], total: int) -> int:
        """Vectors of the row-vector variant for these extents and addresses, 0 when it does not apply."""
        if 'rowvec' not in self.variants or total < self.row_vec:
            return 0
        if any(pointers[t] % 16 for t in self.row_tensors):
            return 0
        if any((d if isinstance(d, int) else env[d]) % self.row_vec for d in self.row_dims):
            return 0
        return total // self.row_vec

    def _matrix_choice(self, env: Dict[str, int], pointers: Optional[Dict[str, int]] = None) -> Tuple[Optional[str], int]:
        """(variant tag, blocks) of the matrix-instruction variants, (None, 0) when they do not apply: there must be
        enough k to pay for staging it, and enough tiles - of 128 x 128 outputs when those fill the chip, else of
        64 x 64 (a block multiplies a quarter as much per k, so small products spread over four times the compute
        units)."""
        if self.matrix is None or 'matrix' not in self.variants:
            return None, 0
        def prod(key):
            n = 1
            for e in self.matrix[key]:
                n *= e if isinstance(e, int) else env[e]
            return n
        M, N, B, K = prod('m'), prod('n'), prod('batch'), prod('k')
        if K < 32 or M < 32 or N < 32:
            return None, 0
        big = ((M + 127) // 128) * ((N + 127) // 128) * B
        small = ((M + 63) // 64) * ((N + 63) // 64) * B
        # the kernels that fetch k-contiguous operands in 16-byte vectors need whole vectors and aligned tensors
        v = ''
        if 'matrixv' in self.variants and pointers is not None and K % self.matrix['vec_width'][0] == 0 and \
                all(pointers[t] % 16 == 0 for t in self.matrix['vec_tensors']):
            def whole(dims_):
                n = 1
                for d in dims_:
                    n *= d if isinstance(d, int) else env[d]
                return n % self.matrix['vec_width'][0] == 0
            if all(whole(p) for p in self.matrix.get('vec_pitch', [])):
                v = 'v'
        # Which block size: the big blocks run in rounds - a compute unit holds one of them with float32 tiles, two with
        # fp16 or int8 tiles, and a round takes as long whether it is full or not - while the small blocks share compute
        # units and take time in proportion to their number, about a 900th of a round each (a 700th with fp16 tiles;
        # measured on squares of 1664 to 4096 with k = 1024 - fp32 2176^2 145 us in big blocks, 104 in small ones, fp16 29
        # against 36 - and on 3 x 3 convolutions of 25088 x 128 outputs).  Tiles
        # that are mostly padding (64 columns in tiles of 128) count as whole blocks on both sides, which settles them.
        half = self.matrix.get('half_tiles')
        rounds = -(-big // (512 if half else 256))
        if 'matrix64' in self.variants and 16 <= small <= MAX_GRID * 64 and small < (700 if half else 900) * rounds:
            return 'matrix64' + v, small
        if big >= 16 and big <= MAX_GRID * 64:
            return 'matrix' + v, big
        if 'matrix64' in self.variants and 16 <= small <= MAX_GRID * 64:
            return 'matrix64' + v, small
        return None, 0

    def _matrix_blocks(self, env: Dict[str, int]) -> int:
        return self._matrix_choice(env)[1]

    def _patches(self, env: Dict[str, int], total: int) -> int:
        """Threads of the register-tiled reduce variant for these extents, 0 when it does not apply."""
        if 'patch' not in self.variants or self.patch is None:
            return 0
        for d, t in zip(self.patch_dims, self.patch):
            if (d if isinstance(d, int) else env[d]) % t:
                return 0
        return total // (self.patch[0] * self.patch[1])

    def choose(self, env: Dict[str, int], pointers: Dict[str, int]) -> Tuple[str, int, int]:
        """-> (kernel symbol, grid.x, block.x) for these extents and addresses."""
        total = 1
        for _, e in self.data_axes:
            total *= e if isinstance(e, int) else env[e]
        red = 1
        for _, e in self.reduce_axes:
            red *= e if isinstance(e, int) else env[e]
        if total == 0:
            return next(iter(self.variants.values())), 0, BLOCK
        if self.kind == 'map':
            if 'vec' in self.variants and all(pointers[t] % 16 == 0 for t in self.vec_tensors) and total >= self.vec:
                work = (total + self.vec - 1) // self.vec
                return self.variants['vec'], min((work + BLOCK - 1) // BLOCK, MAX_GRID), BLOCK
            rows = self._row_vectors(env, pointers, total)
            if rows:
                return self.variants['rowvec'], min((rows + BLOCK - 1) // BLOCK, MAX_GRID), BLOCK
            tiles = self._vector_tiles(env, pointers)
            if tiles:
                return self.variants['tilevec'], min(tiles, MAX_GRID), BLOCK
            tiles = self._tiles(env)
            if tiles:
                return self.variants['tile'], min(tiles, MAX_GRID), BLOCK
            return self.variants['scalar'], min((total + BLOCK - 1) // BLOCK, MAX_GRID), BLOCK
        if self.kind == 'scatter':
            return self.variants['scalar'], min((total + BLOCK - 1) // BLOCK, MAX_GRID), BLOCK
        # reduce
        tag, blocks = self._matrix_choice(env, pointers)
        if tag:
            return self.variants[tag], blocks, BLOCK
        patches = self._patches(env, total)
        if patches >= 131072 and red >= 8:           # two wavefronts per SIMD and more: below that one output per thread hides latency better
            return self.variants['patch'], min((patches + BLOCK - 1) // BLOCK, MAX_GRID), BLOCK
        lanes_ok = self.reduce_contiguous is not False
        if red >= 2048 and total <= 1024 and lanes_ok:
            return self.variants['block'], min(total, MAX_GRID), BLOCK
        if red >= 64 and lanes_ok and (self.reduce_contiguous or total < 64 * 1024):
            waves_per_block = BLOCK // 64
            return self.variants['wave'], min((total + waves_per_block - 1) // waves_per_block, MAX_GRID), BLOCK
        return self.variants['thread'], min((total + BLOCK - 1) // BLOCK, MAX_GRID), BLOCK


    def candidates(self, env: Dict[str, int], pointers: Dict[str, int]) -> List[Tuple[str, str, int]]:
        """Every launch configuration that computes the same result for these extents and addresses:
        (variant tag, kernel symbol, grid.x).  All kernels are grid-stride, so any grid is valid; the
        candidates cover each applicable variant at the heuristic grid and at smaller power-of-two caps."""
        total = 1
        for _, e in self.data_axes:
            total *= e if isinstance(e, int) else env[e]
        if total == 0:
            return []
        tags = []
        if self.kind == 'map':
            if 'vec' in self.variants and all(pointers[t] % 16 == 0 for t in self.vec_tensors) and total >= self.vec:
                tags.append(('vec', (total + self.vec - 1) // self.vec))
            if self._row_vectors(env, pointers, total):
                tags.append(('rowvec', self._row_vectors(env, pointers, total)))
            if self._vector_tiles(env, pointers):
                tags.append(('tilevec', self._vector_tiles(env, pointers) * BLOCK))
            if self._tiles(env):
                tags.append(('tile', self._tiles(env) * BLOCK))
            tags.append(('scalar', total))
        elif self.kind == 'scatter':
            tags.append(('scalar', total))
        else:
            waves_per_block = BLOCK // 64
            tags += [('thread', total), ('wave', (total + waves_per_block - 1) // waves_per_block * BLOCK), ('block', total * BLOCK)]
            if self._patches(env, total):
                tags.append(('patch', self._patches(env, total)))
            if self._matrix_choice(env, pointers)[0]:
                tags.append((self._matrix_choice(env, pointers)[0], self._matrix_blocks(env) * BLOCK))
        out = []
        for tag, work in tags:
            if tag not in self.variants:
                continue
            full = max(1, min((work + BLOCK - 1) // BLOCK, MAX_GRID))
            grids = {full}
            cap = 256
            while cap < full:
                grids.add(cap)
                cap *= 2
            out += [(tag, self.variants[tag], g) for g in sorted(grids, reverse=True)]
        return out


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



def _axes_of(e: Expr) -> set:
    return {m.name for m in walk(e) if m.kind == 'axis'}


def _axes_of_all(load: Expr) -> set:
    return set().union(*[_axes_of(a) for a in load.args]) if load.args else set()


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


def lower_graph(graph, prefix: str = 'autort') -> Tuple[str, List[KernelPlan]]:
    """Fused graph -> (HIP source text with container-format headers, plans).

    The text carries the same ``// GLOBALS`` / ``// LOCAL`` headers as the
    reference's kernel files (antares/antares_compiler.py:183-232) so it can be
    read with the same eyes; the runtime itself works from the plans.
    """
    def disp(n):
        t = graph.tensors[n]
        return f'{n}:{t.dtype}{list(t.shape)}'.replace("'", '')
    head = '// GLOBALS: ' + ', '.join(disp(n) for n in graph.abi_inputs) + ' -> ' + \
        ', '.join(disp(n) for n in graph.abi_outputs) + '\n// BACKEND: c-mi355x (gfx950)\n'
    if graph.dims:
        head += '// VAMAP: ' + ','.join(f'{d}:{v if v is not None else "?"}' for d, v in sorted(graph.dims.items())) + '\n'
    head += '// COMPUTE_V1: - einstein_v2(' + repr(' '.join(graph.source.split())) + ')\n'
    parts, plans = [head + PRELUDE], []
    grouped_until = 0
    for i, st in enumerate(graph.statements):
        count = _row_group_at(graph, i) if i >= grouped_until else 0
        # a map behind a reduction is applied at the reduction's stores (its own kernels stay in the text and are not
        # launched); not where a row kernel may take the reduction
        tail = _tail_of(graph, i) if not count and i >= grouped_until else None
        code, plan = lower_statement(st, graph, f'{prefix}_k{i}', tail=tail)
        if count:
            # the row kernel travels with the first statement's kernels; the per-statement kernels stay for the
            # extents it is not launched at
            row_code, plan.row_group = _lower_row_group(graph, i, count, f'{prefix}_k{i}_rows')
            code += '\n\n' + row_code
            grouped_until = i + count
        ins = ', '.join(disp(n) for n in plan.args[:-1])
        parts.append(f'// LOCAL: {plan.name} -- {ins} -> {disp(plan.output)}\n\n{code}\n')
        plans.append(plan)
    sep = '\n// ---------------------------------------------------------------------------\n'
    return sep.join(parts), plans
