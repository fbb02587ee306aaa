"""Runs a kernel container the way the reference's pybind module does.

The reference hands generated code around as one text file (antares/antares_compiler.py:179-248): a line
``// GLOBALS: a:float32[8, 200] -> out:float32[8]``, then per kernel a ``// LOCAL: <fn> -- inputs -> outputs`` line,
the code, and ``// [thread_extent] blockIdx.x = n`` comments.  `ExecutionModule` (graph_evaluator/
execute_module.hpp:250-394) parses that file, compiles it, and launches the kernels in file order, allocating the
tensors that only live between two kernels; frameworks/pytorch/main_ops.cc:17-54 wraps it for torch as

    key = inject(source)              # remember a container, return its number
    forward(key, inputs + outputs)    # torch tensors in GLOBALS order; outputs are written in place

This module is that pair on the C ABI of this library: containers come from
`antares_amd.lower.evaluator_emit.emit_evaluator_module` (or from a file written by it), kernels are compiled
in-process for gfx950 and launched on torch's current stream.  Launch extents given by `$` keys (grids sized at
launch time from the integer arguments) follow the reference's rule; this build's own emitter does not write them.
"""
from __future__ import annotations

import re
from typing import Dict, List, Tuple

import torch

from ..runtime import capi
from .op import TORCH_DTYPE, compile_cached, current_stream_handle

_PROP_RE = re.compile(r'^\s*([A-Za-z_][A-Za-z0-9_]*):([a-z0-9]+)\[([^\]]*)\]\s*$')


def _between(text: str, begin: str, end: str, start: int = 0) -> str:
    """The text between `begin` and the next `end` (execute_module.hpp:61-71); '' when `begin` is missing."""
    i = text.find(begin, start)
    if i < 0:
        return ''
    i += len(begin)
    j = text.find(end, i)
    return text[i:] if j < 0 else text[i:j]


def _properties(encoded: str) -> List[Tuple[str, str, List[int]]]:
    """``a:float32[8, 200], b:int32[4]`` -> [(name, dtype, shape)] (execute_module.hpp:213-236)."""
    out = []
    for part in re.findall(r'[^,\[\]]+\[[^\]]*\]', encoded):
        m = _PROP_RE.match(part)
        if not m:
            raise ValueError(f'cannot read the tensor description `{part.strip()}`')
        shape = [int(x) for x in m.group(3).split(',') if x.strip()]
        out.append((m.group(1), m.group(2), shape))
    return out


class ExecutionModule:
    def __init__(self, source: str):
        if source.startswith('file://'):
            with open(source[len('file://'):]) as f:
                source = f.read()
        params = _between(source, '// GLOBALS: ', '\n').split(' -> ')
        if len(params) != 2:
            raise ValueError('the container has no `// GLOBALS: inputs -> outputs` line')
        self.global_inputs, self.global_outputs = _properties(params[0]), _properties(params[1])
        self.backend = _between(source, '// BACKEND: ', ' (')
        # `// VAMAP: N:4096,M:64`: values of the named dimensions, handed to every kernel as trailing int arguments
        # in this order (graph_evaluator/run_graph.cpp:164-175)
        self.dim_values = [int(item.split(':')[1]) for item in _between(source, '// VAMAP: ', '\n').split(',') if ':' in item]
        self.local_tensors: Dict[str, Tuple[str, List[int]]] = {}
        self.kernels = []
        for piece in source.split('-------\n')[1:]:
            name = _between(piece, '// LOCAL: ', ' -- ')
            io = _between(piece, ' -- ', '\n').split(' -> ')
            if not name or len(io) != 2:
                continue
            ins, outs = _properties(io[0]), _properties(io[1])
            for n, dt, shape in ins + outs:
                self.local_tensors[n] = (dt, shape)
            threads: Dict[str, int] = {}
            for key, val in re.findall(r'// \[thread_extent\] (\S+) = (-?\d+)', piece):
                if threads.get(key, 0) > 0 and threads[key] != int(val):
                    raise ValueError(f'Multiple `{key}` extents conflict in values: {threads[key]} v.s. {val}')
                threads[key] = int(val)
            # Run-time sized grid (backends/c-rocm/include/backend.hpp:184-194, 204-215): `$` is the position of the
            # first integer argument that sizes it, `$$` a constant factor, `$i` the elements a block takes of the
            # i-th such argument (negative: that argument does not count).
            dynamic = None
            if threads.get('$', 0):
                divisors = []
                while threads.get(f'${len(divisors)}', 0):
                    divisors.append(threads[f'${len(divisors)}'])
                dynamic = (threads['$'], threads.get('$$', 1), divisors)
            self.kernels.append({'name': name, 'in': [p[0] for p in ins], 'out': [p[0] for p in outs], 'threads': threads,
                                 'dynamic': dynamic})
        if not self.kernels:
            raise ValueError('the container holds no kernel')
        self._image = compile_cached(source)
        self._module = None

    def _functions(self):
        if self._module is None:
            self._module = capi.Module(self._image)
        return self._module

    def compute(self, tensors: List[torch.Tensor]):
        """`tensors`: the global inputs, then the global outputs (GLOBALS order)."""
        want = self.global_inputs + self.global_outputs
        if len(tensors) != len(want):
            raise ValueError(f'the container takes {len(self.global_inputs)} input(s) and {len(self.global_outputs)} output(s), '
                             f'got {len(tensors)} tensor(s)')
        memory: Dict[str, torch.Tensor] = {}
        dev = tensors[0].device
        for (name, dtype, shape), t in zip(want, tensors):
            if not t.is_cuda:
                raise RuntimeError(f'tensor `{name}` must live on the GPU; there is no CPU fallback')
            numel = 1
            for d in shape:
                numel *= d
            if t.numel() != numel or t.element_size() != torch.empty(0, dtype=TORCH_DTYPE[dtype]).element_size() or not t.is_contiguous():
                raise ValueError(f'tensor `{name}` must be a dense {dtype}{shape}, got {t.dtype}{list(t.shape)}')
            if t.data_ptr() % 16:
                raise ValueError(f'tensor `{name}` must start on a 16-byte boundary (the kernels of a container use 128-bit accesses)')
            memory[name] = t
        capi.init(dev.index or 0)
        module = self._functions()
        stream = current_stream_handle(dev.index)
        for k in self.kernels:
            for n in k['out']:                      # tensors that only live between two kernels
                if n not in memory:
                    dt, shape = self.local_tensors[n]
                    memory[n] = torch.empty(shape, dtype=TORCH_DTYPE[dt], device=dev)
            th = k['threads']
            args = [memory[n].data_ptr() for n in k['in'] + k['out']] + self.dim_values
            grid_x = th.get('blockIdx.x', 1)
            if k['dynamic'] is not None:
                first, grid_x, divisors = k['dynamic']
                if first + len(divisors) > len(args) or first < len(k['in']) + len(k['out']):
                    raise ValueError(f'kernel `{k["name"]}`: `$ = {first}` does not point at its integer arguments')
                for i, d in enumerate(divisors):
                    if d > 0:
                        grid_x *= (args[first + i] + d - 1) // d
                if grid_x == 0:
                    continue                        # nothing to do at these sizes (backend.hpp:214)
            capi.launch(module.function(k['name']),
                        (grid_x, th.get('blockIdx.y', 1), th.get('blockIdx.z', 1)),
                        (th.get('threadIdx.x', 1), th.get('threadIdx.y', 1), th.get('threadIdx.z', 1)), stream, args)


_sources: List[str] = []
_modules: Dict[int, ExecutionModule] = {}


def inject(source: str) -> int:
    """main_ops.cc:17-22: remembers a container and returns its key."""
    _sources.append(source)
    return len(_sources) - 1


def forward(custom_key: int, tensors: List[torch.Tensor]) -> None:
    """main_ops.cc:24-48: runs container `custom_key` on `tensors` (inputs, then outputs, in GLOBALS order).  The
    parsed module is kept per (key, device), as there."""
    if not tensors:
        raise ValueError('forward() needs the tensors of the container')
    if not 0 <= custom_key < len(_sources):
        raise KeyError(f'no container with key {custom_key}')
    comp_key = custom_key * 32 + (tensors[0].device.index or 0)
    module = _modules.get(comp_key)
    if module is None:
        module = _modules[comp_key] = ExecutionModule(_sources[custom_key])
    module.compute(list(tensors))
