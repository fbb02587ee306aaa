"""The C-ABI library: it loads, exports every function the header declares, and
its error paths return codes + messages instead of exiting.  No kernel runs here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope='module')
def lib():
    from antares_amd.runtime import capi
    if not os.path.exists(capi.LIB_PATH):
        from antares_amd import build
        build.build(verbose=False)
    return capi


def declared_functions():
    text = open(os.path.join(ROOT, 'include', 'antares_amd.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(art_[a-z0-9_]+)\s*\(', text)))


def test_every_declared_function_is_exported_and_bound(lib):
    names = declared_functions()
    assert 'art_gemv_w4a16' in names and 'art_launch' in names and len(names) >= 20
    handle = ctypes.CDLL(lib.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), f'{n} is declared in the header but not exported'
    assert sorted(lib.exported_symbols()) == names, 'ctypes table and header disagree'


def test_compile_without_gpu_and_error_reporting(lib):
    image = lib.compile_hip('extern "C" __global__ void k(float* a) { a[threadIdx.x] = 1.0f; }')
    assert image[:4] == b'\x7fELF'
    with pytest.raises(lib.ArtError, match='compilation failed'):
        lib.compile_hip('extern "C" __global__ void k(float* a) { this is not C++ }')
    assert 'error' in lib.lib().art_compile_log().decode()


def test_bad_arguments_return_errors(lib):
    l = lib.lib()
    assert l.art_launch(None, 1, 1, 1, 64, 1, 1, 0, None, None, 0) != 0
    assert b'null function' in l.art_last_error()
    assert l.art_gemv_w4a16(None, None, None, None, None, 1, 4096, 4096, None) != 0
    assert b'null pointer' in l.art_last_error()
    assert l.art_module_load(None, 0, None) != 0
    assert l.art_module_load_file(b'/nonexistent/kernel.hsaco', None) != 0
    import ctypes
    h = ctypes.c_void_p()
    assert l.art_module_load_file(b'/nonexistent/kernel.hsaco', ctypes.byref(h)) != 0
    assert b'cannot open' in l.art_last_error()


def test_missing_library_fails_loudly(monkeypatch, lib):
    monkeypatch.setattr(lib, '_lib', None)
    monkeypatch.setattr(lib, 'LIB_PATH', '/nonexistent/libantares_amd.so')
    with pytest.raises(lib.ArtError, match='no CPU fallback'):
        lib.lib()


def test_operator_refuses_cpu_tensors():
    import torch
    import autort
    f = autort.export(ir='o[N] = a[N] + 1', inputs=['a=float32[N:8]'])
    with pytest.raises(RuntimeError, match='no CPU fallback'):
        f(torch.zeros(8))
    with pytest.raises(TypeError, match='must be float32'):
        f(torch.zeros(8, dtype=torch.int32))
