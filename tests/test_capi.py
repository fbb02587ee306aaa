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


@pytest.mark.gpu
def test_device_copies_and_the_read_only_launch():
    """art_memcpy_dtod (ab::memcpyDtoD) copies on the stream it is given; art_read_bytes reads a buffer and writes nothing."""
    import torch
    from ctypes import c_void_p
    from antares_amd.runtime import capi
    capi.init(0)
    l = capi.lib()
    src = torch.arange(1 << 20, dtype=torch.int32, device='cuda')
    dst = torch.zeros_like(src)
    capi.check(l.art_memcpy_dtod(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), src.numel() * 4, None))
    capi.check(l.art_stream_synchronize(None))
    assert torch.equal(dst, src)
    sink = torch.zeros(4096, dtype=torch.int32, device='cuda')
    buf = torch.randint(0, 256, (2048 * 11008,), dtype=torch.uint8, device='cuda')
    before = buf.clone()
    capi.check(l.art_read_bytes(c_void_p(buf.data_ptr()), buf.numel(), c_void_p(sink.data_ptr()), None))
    capi.check(l.art_read_bytes(c_void_p(buf.data_ptr()), 32768 * 3, c_void_p(sink.data_ptr()), None))
    torch.cuda.synchronize()
    assert torch.equal(buf, before) and int(sink.abs().sum()) == 0
    assert l.art_read_bytes(c_void_p(buf.data_ptr()), 1000, c_void_p(sink.data_ptr()), None) != 0


@pytest.mark.gpu
def test_store_only_launch_and_phases_meeting_inside_one_launch():
    """art_fill_bytes writes the constant and nothing else; art_phase_chain_probe runs its phases to the end in every
    mode (no block gives up waiting on a free chip), twice in a row on one workspace, and rejects sizes it cannot take."""
    import torch
    from ctypes import c_void_p
    from antares_amd.runtime import capi
    capi.init(0)
    l = capi.lib()
    buf = torch.zeros(1 << 20, dtype=torch.int32, device='cuda')
    capi.check(l.art_fill_bytes(c_void_p(buf.data_ptr()), (1 << 20) * 4 - 64, 0x01020304, None))
    torch.cuda.synchronize()
    assert bool((buf[:-16] == 0x01020304).all()) and int(buf[-16:].abs().sum()) == 0
    assert l.art_fill_bytes(c_void_p(buf.data_ptr()), 24, 1, None) != 0
    phases, nbytes = 6, 32768 * 40
    src = torch.randint(0, 256, (phases * nbytes,), dtype=torch.uint8, device='cuda')
    before = src.clone()
    sink = torch.zeros(4096, dtype=torch.int32, device='cuda')
    status = torch.zeros(1, dtype=torch.int32, device='cuda')
    for rep in range(2):
        for mode in (0, 1, 2):
            print(f'[case] phase chain mode {mode} rep {rep}', flush=True)
            capi.check(l.art_phase_chain_probe(c_void_p(src.data_ptr()), src.numel(), nbytes, phases, mode, c_void_p(sink.data_ptr()),
                                               c_void_p(status.data_ptr()), None))
            torch.cuda.synchronize()
            assert int(status.item()) == 0
    assert torch.equal(src, before) and int(sink.abs().sum()) == 0
    assert l.art_phase_chain_probe(c_void_p(src.data_ptr()), src.numel(), nbytes, phases + 1, 1, c_void_p(sink.data_ptr()),
                                   c_void_p(status.data_ptr()), None) != 0
    assert l.art_phase_chain_probe(c_void_p(src.data_ptr()), src.numel(), 1000, 1, 1, c_void_p(sink.data_ptr()),
                                   c_void_p(status.data_ptr()), None) != 0


@pytest.mark.gpu
def test_a_released_stream_gives_its_workspace_back():
    """A process that creates and destroys streams: every stream that launches a split-K kernel gets a 64 MiB
    workspace (40 slots per device); `art_release_stream` hands it back, so the 41st, 42nd ... stream still works, and
    a released stream that launches again simply gets a new one."""
    import numpy as np
    import torch
    from ctypes import c_void_p
    from antares_amd import workloads
    from antares_amd.runtime import capi
    capi.init(0)
    lib = capi.lib()
    p = {k: v.cuda() for k, v in workloads.w4_problem(5, 1, 1024, 256).items()}
    want = None
    for i in range(48):
        s = torch.cuda.Stream()
        y = torch.zeros(1, 256, dtype=torch.float16, device='cuda')
        s.wait_stream(torch.cuda.current_stream())
        capi.check(lib.art_gemv_w4a16(c_void_p(p['x'].data_ptr()), c_void_p(p['qweight'].data_ptr()), c_void_p(p['scales'].data_ptr()),
                                      c_void_p(p['qzeros'].data_ptr()), c_void_p(y.data_ptr()), 1, 1024, 256, c_void_p(s.cuda_stream)))
        if i % 7 == 0:            # a stream that is released and used again
            capi.check(lib.art_release_stream(c_void_p(s.cuda_stream)))
            capi.check(lib.art_gemv_w4a16(c_void_p(p['x'].data_ptr()), c_void_p(p['qweight'].data_ptr()), c_void_p(p['scales'].data_ptr()),
                                          c_void_p(p['qzeros'].data_ptr()), c_void_p(y.data_ptr()), 1, 1024, 256, c_void_p(s.cuda_stream)))
        capi.check(lib.art_release_stream(c_void_p(s.cuda_stream)))          # waits for the stream's work
        got = y.cpu().numpy()
        want = got if want is None else want
        assert np.array_equal(got, want), i
    capi.check(lib.art_release_stream(c_void_p(torch.cuda.Stream().cuda_stream)))      # a stream with no workspace: no error
    assert lib.art_release_stream(c_void_p(0)) != 0 and b'default stream' in lib.art_last_error()
