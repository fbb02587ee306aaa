"""The AutoRT operator surface on MI355X.

    import autort                      # or: from antares_amd import autort
    f = autort.export(ir="sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))",
                      inputs=["data=float32[N:4096000]"], config="tune:5")
    y = f(x); y = autort.ops.sigmoid_f32(x)

Same entry points and argument meaning as the reference's wheel, as far as its
call sites show them (README.md:63-87, samples/*.py): ``export``, ``ops``,
``device``, ``download``, ``profile``.
"""
from __future__ import annotations

import contextlib
import os
from typing import Optional, Sequence

import torch

from .op import ExportedOp, parse_config


class _Ops:
    """``autort.ops.<name>``: operators exported in this process, operators
    persisted by an earlier session or by the command line (module files, see
    ``store.py``), and the built-in ones."""

    def __init__(self):
        object.__setattr__(self, '_table', {})

    def _register(self, name: str, op):
        self._table[name] = op

    def __getattr__(self, name: str):
        table = object.__getattribute__(self, '_table')
        if name in table:
            return table[name]
        from . import builtin, store
        record = None if name.startswith('_') else store.load(name)
        if record is not None:
            op = ExportedOp(record['ir'], list(record['inputs']), config=record['config'], name=record['name'],
                            extra_outputs=record['extra_outputs'], tuned=record.get('tuned') or None)
            table[name] = op
            return op
        op = builtin.lookup(name)
        if op is None:
            raise AttributeError(f'autort.ops has no operator `{name}`; create it with autort.export(..., name="{name}")')
        table[name] = op
        return op

    def __dir__(self):
        from . import builtin, store
        return sorted(set(self._table) | set(builtin.names()) | set(store.names()))


ops = _Ops()


def export(ir: str, inputs: Sequence[str] = (), config: Optional[str] = None, name: Optional[str] = None,
           extra_outputs: Sequence[str] = ()) -> ExportedOp:
    """Create an operator from einstein_v2 text.  ``inputs`` lists the tensors in
    calling order as ``"name=dtype[dims]"``; a dimension may be an integer, a
    named run-time dimension with a default (``N:4096``) or a bare name.  The
    operator is also registered as ``autort.ops.<name>`` (default: the name of
    the last output tensor) and written to a module file, so that later sessions
    find it under the same name (README.md:75-86)."""
    op = ExportedOp(ir, list(inputs), config=config, name=name, extra_outputs=extra_outputs)
    ops._register(op.name, op)
    op.persist()
    return op


def device(index: int = 0) -> torch.device:
    """The device operators run on (samples/05_llama2_7b_int4.py:78)."""
    if not torch.cuda.is_available():
        raise RuntimeError('autort.device(): no MI355X / ROCm device is visible')
    return torch.device('cuda', index)


def download(path: str, url: str = None, is_zip: bool = False) -> str:
    """The reference fetches model files here (samples/05_llama2_7b_int4.py:11);
    this build never touches the network: the file must already exist."""
    if not os.path.exists(path):
        raise FileNotFoundError(f'{path} is not present and downloading is disabled in this build ({url})')
    return path


@contextlib.contextmanager
def profile(enabled: bool = True):
    """Times the enclosed region with events on the current stream and prints
    the result (call site: samples/02_mnist.py:86)."""
    if not enabled or not torch.cuda.is_available():
        yield
        return
    from ..runtime import capi
    capi.init(torch.cuda.current_device())
    start, stop = capi.Event(), capi.Event()
    stream = torch.cuda.current_stream().cuda_stream
    start.record(stream)
    try:
        yield
    finally:
        stop.record(stream)
        print(f'[autort.profile] {start.elapsed_ms(stop):.3f} ms')
