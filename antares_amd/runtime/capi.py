"""ctypes binding of libantares_amd.so (declared in include/antares_amd.h).

The library is built in-tree by ``antares_amd.build`` (hipcc, gfx950).  There
is no fallback: if it is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, byref, c_char, c_char_p, c_float, c_int, c_longlong, c_size_t, c_uint, c_uint64,
                    c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), 'csrc', 'libantares_amd.so')


class ArtError(RuntimeError):
    pass


class ArtProps(ctypes.Structure):
    _fields_ = [('name', c_char * 256), ('arch', c_char * 64), ('compute_units', c_int),
                ('wavefront_size', c_int), ('max_threads_per_block', c_int), ('lds_bytes_per_block', c_int),
                ('clock_khz', c_int), ('memory_clock_khz', c_int), ('memory_bus_width_bits', c_int),
                ('l2_bytes', c_int), ('total_memory_bytes', c_size_t)]


# name -> (restype, argtypes); everything returning c_int is checked.
_SIGNATURES = {
    'art_init': (c_int, [c_int]),
    'art_last_error': (c_char_p, []),
    'art_compile_log': (c_char_p, []),
    'art_device_props': (c_int, [POINTER(ArtProps)]),
    'art_module_compile': (c_int, [c_char_p, c_char_p, POINTER(c_void_p), POINTER(c_size_t)]),
    'art_blob_free': (None, [c_void_p]),
    'art_module_load': (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    'art_module_load_file': (c_int, [c_char_p, POINTER(c_void_p)]),
    'art_module_unload': (c_int, [c_void_p]),
    'art_get_function': (c_int, [c_void_p, c_char_p, POINTER(c_void_p)]),
    'art_launch': (c_int, [c_void_p, c_uint, c_uint, c_uint, c_uint, c_uint, c_uint, c_uint, c_void_p,
                           POINTER(c_uint64), c_int]),
    'art_event_create': (c_int, [POINTER(c_void_p)]),
    'art_event_record': (c_int, [c_void_p, c_void_p]),
    'art_event_elapsed_ms': (c_int, [c_void_p, c_void_p, POINTER(c_float)]),
    'art_event_destroy': (c_int, [c_void_p]),
    'art_stream_synchronize': (c_int, [c_void_p]),
    'art_copy_bytes': (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    'art_workspace_bytes': (c_size_t, []),
    'art_release_stream': (c_int, [c_void_p]),
    'art_alloc': (c_int, [c_size_t, POINTER(c_void_p)]),
    'art_free': (c_int, [c_void_p]),
    'art_memcpy_htod': (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    'art_memcpy_dtoh': (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    'art_memcpy_dtod': (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    'art_read_bytes': (c_int, [c_void_p, c_size_t, c_void_p, c_void_p]),
    'art_fill_bytes': (c_int, [c_void_p, c_size_t, c_uint, c_void_p]),
    'art_phase_chain_probe': (c_int, [c_void_p, c_size_t, c_size_t, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    'art_gemv_w4a16': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    'art_gemv_w4a16_tuned': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    'art_gemv_w4a16_knobs': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    'art_gemm_w4a16_tuned': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    'art_gemm_w4a16_residual': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    'art_partition_even_first_i32_tuned': (c_int, [c_void_p, c_void_p, c_longlong, c_int, c_void_p]),
    'art_gemv_w4a16_noalloc': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    'art_decode_attention_rope_split': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_void_p]),
    'art_gemv_w4a16_attn': (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    'art_gemv_w4a16_attn_sumsq': (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p,
                                          c_void_p, c_void_p]),
    'art_rope_qkv_store_rows': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    'art_prefill_attention': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_longlong, c_void_p]),
    'art_greedy_next': (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    'art_gemm_w4a16': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    'art_gemv_gptq': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    'art_partition_even_first_i32': (c_int, [c_void_p, c_void_p, c_longlong, c_void_p]),
    'art_w4_prepack_bytes': (c_size_t, [c_int, c_int]),
    'art_w4_prepack': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    'art_gemv_w4p': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_float, c_void_p, c_int, c_void_p]),
    'art_gemv_w4a16_fused': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_float, c_void_p,
                                     c_int, c_void_p]),
    'art_gemv_w4a16_fused_sumsq': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_float,
                                           c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    'art_decode_attention_rope': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p]),
    'art_rope_qkv_store': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    'art_gemm_f16': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    'art_gemm_f16_tuned': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    'art_gemm_f32': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    'art_gemm_f32_batched': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    'art_gemm_f32_ex': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    'art_rmsnorm': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_float, c_int, c_int, c_int, c_void_p]),
    'art_rotary': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_longlong, c_int, c_int, c_int, c_int,
                           c_void_p]),
    'art_decode_attention': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int,
                                     c_int, c_void_p]),
}

_lib = None


def exported_symbols():
    return list(_SIGNATURES)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ArtError(f'{LIB_PATH} is missing: build it with `python -m antares_amd.build` '
                           '(there is no CPU fallback)')
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype, fn.argtypes = res, args
        _lib = l
    return _lib


def check(rc: int):
    if rc != 0:
        raise ArtError(lib().art_last_error().decode(errors='replace'))


_inited = set()


def init(device: int = 0):
    if device not in _inited:
        check(lib().art_init(device))
        _inited.add(device)


def device_props() -> dict:
    p = ArtProps()
    check(lib().art_device_props(byref(p)))
    return {f: (getattr(p, f).decode() if isinstance(getattr(p, f), bytes) else getattr(p, f)) for f, _ in p._fields_}


def compile_hip(source: str, arch: str = 'gfx950') -> bytes:
    """HIP source -> code object bytes (in-process, no GPU needed)."""
    blob, size = c_void_p(), c_size_t()
    check(lib().art_module_compile(source.encode(), arch.encode(), byref(blob), byref(size)))
    try:
        return ctypes.string_at(blob, size.value)
    finally:
        lib().art_blob_free(blob)


class Module:
    def __init__(self, image: bytes):
        self._image = image            # keep alive: the loader may reference it
        h = c_void_p()
        check(lib().art_module_load(image, len(image), byref(h)))
        self.handle = h
        self._funcs = {}

    def function(self, name: str) -> c_void_p:
        f = self._funcs.get(name)
        if f is None:
            f = c_void_p()
            check(lib().art_get_function(self.handle, name.encode(), byref(f)))
            self._funcs[name] = f
        return f


_loaded_modules = {}


def shared_module(image: bytes) -> Module:
    """The loaded code object for this image, loaded once per process: an operator that drops a per-shape kernel set
    from its table and meets the shape again gets the module that is already on the device instead of loading a
    second copy.  Modules stay loaded for the life of the process (a recorded graph may still launch from them), as the
    reference's do (graph_evaluator/execute_module.hpp:274-319)."""
    import hashlib
    key = hashlib.sha256(image).digest()
    m = _loaded_modules.get(key)
    if m is None:
        m = _loaded_modules[key] = Module(image)
    return m


def launch(func, grid, block, stream: int, args, lds: int = 0):
    n = len(args)
    arr = (c_uint64 * n)(*[a & 0xFFFFFFFFFFFFFFFF for a in args])
    check(lib().art_launch(func, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds,
                           c_void_p(stream), arr, n))


class Event:
    def __init__(self):
        self.h = c_void_p()
        check(lib().art_event_create(byref(self.h)))

    def record(self, stream: int):
        check(lib().art_event_record(self.h, c_void_p(stream)))

    def elapsed_ms(self, stop: 'Event') -> float:
        ms = c_float()
        check(lib().art_event_elapsed_ms(self.h, stop.h, byref(ms)))
        return ms.value

    def __del__(self):
        try:
            lib().art_event_destroy(self.h)
        except Exception:
            pass
