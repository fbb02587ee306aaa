"""TEST INFRASTRUCTURE ONLY — CPU oracle driver.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may use this module.

Compiles the kernels written by cpu_emit.py with the reference's CPU-backend
compiler line (backends/c-mcpu/include/backend.hpp:157: ``g++ -std=c++17 -O2
-ffast-math -fPIC -shared``), loads them with ctypes and runs them on the
rank-striding thread pool of libref_runtime.so.  Timing follows the reference
evaluator's protocol (graph_evaluator/run_graph.cpp:214-236): one warm-up run,
one probe run, then n = clamp(1 / t_probe, 1, 10000) timed runs, mean reported.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import subprocess
import tempfile
import time
from typing import Dict, List, Optional

import numpy as np

from . import cpu_emit

_HERE = os.path.dirname(os.path.abspath(__file__))
_BUILD = os.path.join(_HERE, '_build')
NP_DTYPE = {'float64': np.float64, 'float32': np.float32, 'float16': np.float16, 'int64': np.int64,
            'int32': np.int32, 'int16': np.int16, 'int8': np.int8, 'uint8': np.uint8}

_runtime = None


def runtime() -> ctypes.CDLL:
    """libref_runtime.so (thread pool, fill, digest); built by oracle/Makefile."""
    global _runtime
    if _runtime is None:
        path = os.path.join(_HERE, 'libref_runtime.so')
        if not os.path.exists(path):
            subprocess.check_call(['make', '-C', _HERE, 'libref_runtime.so'])
        lib = ctypes.CDLL(path)
        lib.ref_run.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
        lib.ref_run.restype = ctypes.c_int
        lib.ref_threads.restype = ctypes.c_int
        lib.ref_set_threads.argtypes = [ctypes.c_int]
        lib.ref_fill.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_char_p, ctypes.c_int]
        lib.ref_digest.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_char_p, ctypes.POINTER(ctypes.c_double)]
        _runtime = lib
    return _runtime


def threads() -> int:
    return runtime().ref_threads()


def compile_source(source: str, fast_math: bool = True) -> ctypes.CDLL:
    os.makedirs(_BUILD, exist_ok=True)
    flags = ['-std=c++17', '-O2', '-fPIC', '-shared'] + (['-ffast-math'] if fast_math else [])
    key = hashlib.sha256((source + ' '.join(flags)).encode()).hexdigest()[:20]
    so = os.path.join(_BUILD, f'k_{key}.so')
    if not os.path.exists(so):
        src = os.path.join(_BUILD, f'k_{key}.cpp')
        with open(src, 'w') as f:
            f.write(source)
        tmp = so + f'.tmp{os.getpid()}'
        subprocess.check_call(['g++', src] + flags + ['-I', _HERE, '-o', tmp])
        os.replace(tmp, so)
    return ctypes.CDLL(so)


class CpuModule:
    """An einstein_v2 program compiled for the CPU oracle."""

    def __init__(self, graph, nranks: int = 64, fast_math: bool = True):
        from antares_amd.ir import fuse_elementwise
        self.graph = fuse_elementwise(graph)
        self.source, self.kernels = cpu_emit.emit_module(graph, nranks=nranks)
        self.lib = compile_source(self.source, fast_math)
        self.fns = [ctypes.cast(getattr(self.lib, k['name']), ctypes.c_void_p) for k in self.kernels]

    def _bind(self, tensors: Dict[str, np.ndarray]):
        g = self.graph
        shapes = {n: tensors[n].shape for n in g.declared if n in tensors}
        env = g.bind_dims(shapes)
        bufs: Dict[str, np.ndarray] = {}
        for n in g.abi_inputs:
            a = np.ascontiguousarray(tensors[n])
            want = NP_DTYPE[g.tensors[n].dtype]
            if a.dtype != want:
                if a.dtype.itemsize == np.dtype(want).itemsize and a.dtype.kind in 'iu' and np.dtype(want).kind in 'iu':
                    a = a.view(want)
                else:
                    raise TypeError(f'tensor `{n}`: expected {np.dtype(want)}, got {a.dtype}')
            bufs[n] = a
        for k in self.kernels:
            for n in k['args']:
                if n in bufs:
                    continue
                if n in tensors:       # in-out tensor or caller-provided output
                    a = tensors[n]
                    assert a.flags['C_CONTIGUOUS'] and a.dtype == NP_DTYPE[g.tensors[n].dtype], n
                    bufs[n] = a
                else:
                    bufs[n] = np.zeros(g.shape_of(n, env), dtype=NP_DTYPE[g.tensors[n].dtype])
        return env, bufs

    def _launch_plan(self, env, bufs):
        plan = []
        for k, fn in zip(self.kernels, self.fns):
            vals = [bufs[n].ctypes.data for n in k['args']] + [env[d] for d in self.graph.dim_names]
            arr = (ctypes.c_void_p * len(vals))(*vals)
            plan.append((fn, k['nranks'], arr))
        return plan

    def __call__(self, **tensors) -> Dict[str, np.ndarray]:
        env, bufs = self._bind(tensors)
        rt = runtime()
        for fn, nranks, arr in self._launch_plan(env, bufs):
            rc = rt.ref_run(fn, nranks, arr)
            assert rc == 0
        return {n: bufs[n] for n in self.graph.abi_outputs}

    def time(self, max_runs: int = 10000, budget_s: Optional[float] = None, **tensors) -> dict:
        """Seconds per run by the reference evaluator's protocol; ``budget_s``
        caps the timed loop (the number of runs actually timed is reported)."""
        env, bufs = self._bind(tensors)
        plan = self._launch_plan(env, bufs)
        rt = runtime()

        def once():
            for fn, nranks, arr in plan:
                rt.ref_run(fn, nranks, arr)
        once()
        t0 = time.perf_counter(); once(); tpr = max(time.perf_counter() - t0, 1e-9)
        n = int(max(1, min(max_runs, 1.0 / tpr)))
        if budget_s is not None:
            n = int(max(1, min(n, budget_s / tpr)))
        t0 = time.perf_counter()
        for _ in range(n):
            once()
        tpr = (time.perf_counter() - t0) / n
        return {'seconds': tpr, 'runs': n, 'threads': threads()}


def fill(arr: np.ndarray, dtype: str, arg_index: int) -> np.ndarray:
    rc = runtime().ref_fill(arr.ctypes.data, arr.size, dtype.encode(), arg_index)
    assert rc == 0, dtype
    return arr


def digest(arr: np.ndarray, dtype: str) -> float:
    out = ctypes.c_double()
    rc = runtime().ref_digest(np.ascontiguousarray(arr).ctypes.data, arr.size, dtype.encode(), ctypes.byref(out))
    assert rc == 0, dtype
    return out.value
