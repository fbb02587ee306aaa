"""Kernel container text that the reference's evaluator can drive.

``ExecutionModule`` (graph_evaluator/execute_module.hpp:274-319) reads a source
file whose header names the global tensors with numeric shapes
(``// GLOBALS: a:float32[4096] -> out:float32[4096]``), the values of run-time
dimensions (``// VAMAP: N:4096,...`` — appended to every launch as trailing
integer arguments, run_graph.cpp:168-178) and, per kernel, a ``// LOCAL:`` line
plus ``// [thread_extent] blockIdx.x = n`` comments for the launch shape.
``lower_graph`` already emits the same kernels behind the same argument
convention; this module fixes the shapes to concrete extents, picks the kernel
variant and grid the runtime would pick for them, and writes the result in that
layout (the writer on the reference side: antares/antares_compiler.py:179-248).
With a ``backend.hpp`` that forwards ``namespace ab`` to the C ABI
(include/c-mi355x/backend.hpp) the evaluator runs these kernels unchanged.
"""
from __future__ import annotations

from typing import Dict, Optional

from .hip_codegen import lower_graph
from .hip_prelude import PRELUDE


def emit_evaluator_module(graph, dims: Optional[Dict[str, int]] = None, prefix: str = 'template_op') -> str:
    """``graph``: a fused Graph.  ``dims`` overrides the declared defaults of named dimensions."""
    env = {d: (v if v is not None else 1) for d, v in graph.dims.items()}
    env.update(dims or {})

    def disp(n):
        t = graph.tensors[n]
        return f'{n}:{t.dtype}{[d if isinstance(d, int) else env[d] for d in t.shape]}'

    text, plans = lower_graph(graph, prefix=prefix)
    pieces = text.split('\n// ---------------------------------------------------------------------------\n')
    head = '// GLOBALS: ' + ', '.join(disp(n) for n in graph.abi_inputs) + ' -> ' + \
        ', '.join(disp(n) for n in graph.abi_outputs) + '\n// BACKEND: c-mi355x (gfx950)\n'
    if graph.dims:
        head += '// VAMAP: ' + ','.join(f'{d}:{env[d]}' for d in graph.dim_names) + '\n'
    head += '// CONFIG: \n// COMPUTE_V1: - einstein_v2(' + repr(' '.join(graph.source.split())) + ')\n'
    out = [head + PRELUDE]
    assert len(pieces) == len(plans) + 1
    skip = 0
    for plan, piece in zip(plans, pieces[1:]):
        if skip:                    # a map that the kernels of the reduction before it apply at their stores
            skip -= 1
            continue
        skip = plan.covers - 1
        symbol, grid, block = plan.choose(env, {n: 0 for n in plan.args})      # evaluator buffers are 256-byte aligned
        code = piece.split('\n', 1)[1]                                          # drop lower_graph's own LOCAL line
        ins = ', '.join(disp(n) for n in plan.args[:-1])
        out.append(f'// LOCAL: {symbol} -- {ins} -> {disp(plan.output)}\n'
                   f'// [thread_extent] blockIdx.x = {max(grid, 1)}\n// [thread_extent] threadIdx.x = {block}\n{code}')
    return '\n// ---------------------------------------------------------------------------\n'.join(out)
