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

The families live in modules of their own - `statements.py` (maps, reductions, scatters), `matrix.py` (contractions on
the matrix instructions), `rows.py` (row kernels), `plans.py` (launch plans), `emit_common.py` (types, expression
emitter, signatures); this module keeps `lower_graph` and re-exports their names.

Kernel signatures follow the reference's HIP kernel ABI
(backends/c-rocm/config.py:25-85): tensor pointers first, in the order given by
the caller, then the named run-time dimensions as ``int`` arguments.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

from ..ir.nodes import Expr, ITEMSIZE, walk
from .hip_prelude import PRELUDE

# the kernel families (this module keeps `lower_graph` and re-exports their names)
from .emit_common import (HIP_TYPE, BLOCK, MAX_GRID, _CALLS, _REDUCE_OP, dim_c, reduce_identity, const_c, ExprEmitter, _signature, _extents, _decompose, _root_and_cond, _axes_of, _axes_of_all, _multiple_of)  # noqa: F401
from .plans import (RowGroup, KernelPlan)  # noqa: F401
from .statements import (_transpose_axes, _row_vector_loads, _is_flat_map, lower_statement, _patch_axes, _reduce_axis_contiguous, _tail_of)  # noqa: F401
from .matrix import (_matrix_kernel, _split_index, _matrix_contraction, _matrix_tail, contraction_slices)  # noqa: F401
from .rows import (_row_group_at, _row_run, _lower_row_group)  # noqa: F401


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
