"""The legacy plugin surface of the reference tree, on the same engine.

    from antares_amd.autort.custom_op import CustomOp
    op = CustomOp(ir='out[N, M] = a[N, M] + b[N, M]', input_orders={'a': a, 'b': b}, device=dev).tune(step=0).emit()
    y = op(a, b)

Mirrors ``CustomOp`` of frameworks/pytorch/custom_op.py:39-148: ``input_orders``
maps a tensor name to a tensor or to ``(name, dtype, shape)``; ``emit()`` builds
the kernels and fills ``output_infos`` / ``output_names`` / ``kernel_sources``;
calling the module takes the inputs in ``input_orders`` order, allocates the
outputs and returns one tensor or a tuple.  Where the reference shells out to
the ``antares`` service and a pybind module (main_ops.cc:17-54), this one lowers
in-process and launches through the C ABI.  ``kernel_sources`` is the kernel
container the reference would have received from the service, and ``custom_key``
the number ``inject`` gave it: ``forward(op.custom_key, inputs + outputs)`` of
``antares_amd.autort.execution_module`` runs that container as the pybind module
does; calling the operator itself takes the faster route through ``autort.export``
(hand-written kernels where the program is a known pattern).
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple, Union

import torch

from ..lower.evaluator_emit import emit_evaluator_module
from .execution_module import inject
from .op import ExportedOp

_DTYPE_NAME = {torch.float64: 'float64', torch.float32: 'float32', torch.float16: 'float16', torch.int64: 'int64',
               torch.int32: 'int32', torch.int16: 'int16', torch.int8: 'int8', torch.uint8: 'uint8'}
_DTYPE_TORCH = {v: k for k, v in _DTYPE_NAME.items()}


class CustomOp(torch.nn.Module):
    def __init__(self, ir: str, input_orders: Dict[str, Union[torch.Tensor, Tuple]], extra_outputs: Sequence[str] = (),
                 device=None):
        super().__init__()
        self.ir = ir.replace('"', '`').replace('\n', ' ').strip()       # custom_op.py:43
        self.extra_outputs = list(extra_outputs)
        specs: List[str] = []
        for name, v in input_orders.items():
            if isinstance(v, tuple):                                    # (name, dtype, shape), custom_op.py:46-47
                dtype, shape = v[1], v[2]
            else:
                dtype, shape = v.dtype, v.shape
            dname = dtype if isinstance(dtype, str) else _DTYPE_NAME.get(dtype)
            if dname not in _DTYPE_TORCH:
                raise TypeError(f'CustomOp: tensor `{name}` has unsupported dtype {dtype}')
            specs.append(f'{name}={dname}[{", ".join(str(int(d)) for d in shape)}]')
        self.input_specs = specs
        self.custom_device = 'cpu' if device is None else torch.device(device).type
        if self.custom_device != 'cuda':
            raise RuntimeError('CustomOp: this backend runs on the MI355X only; pass device=autort.device()')
        self._steps = 0
        self._op = None

    def to(self, *args, **kwargs):
        raise Exception('Deprecated Usage: Legacy `CustomOp(..).to(device)` has been simplified to `CustomOp(.., device=device)`')

    def tune(self, step: int = 100, use_cache: bool = False, timeout: int = -1) -> 'CustomOp':
        """Records the number of tuning trials; they run at the first call on the GPU
        (custom_op.py:128-134 runs the search here through the `antares` service)."""
        self._steps = max(0, int(step))
        return self

    def emit(self) -> 'CustomOp':
        config = f'tune:{self._steps}' if self._steps > 0 else None
        op = ExportedOp(self.ir, self.input_specs, config=config, extra_outputs=self.extra_outputs)
        op.compile()
        g = op.graph
        env = g.bind_dims({})
        self.output_infos = [(n, _DTYPE_TORCH[g.tensors[n].dtype], [int(d) for d in g.shape_of(n, env)]) for n in g.outputs]
        self.output_names = [x[0] for x in self.output_infos]
        self.kernel_sources = emit_evaluator_module(op.lowered)
        self.custom_key = inject(self.kernel_sources)
        self._op = op
        return self

    def output(self, index: int = 0):
        return self.output_infos[index]

    def forward(self, *inputs):
        if self._op is None:
            raise RuntimeError('CustomOp: call emit() before using the operator')
        ordered = [t.contiguous().to(self.custom_device) for t in inputs]
        return self._op(*ordered)
