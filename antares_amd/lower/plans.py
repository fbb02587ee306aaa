"""Launch plans of the generic lowering: what the host needs to launch the kernels of one statement (`KernelPlan`:
the compiled variants and the per-call choice among them by extents and alignment) or of a run of statements that one
row kernel computes (`RowGroup`).  The counterpart of the reference's `// [thread_extent]` annotations and its
`get_execution_parallism` (backends/c-rocm/config.py:9-24), decided per call instead of per compile."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

from ..ir.nodes import Expr, ITEMSIZE, walk
from .emit_common import BLOCK, MAX_GRID



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
