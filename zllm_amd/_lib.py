"""Loads libzllm_hip.so and declares the C ABI of include/zllm_hip.h.

There is no fallback: if the library is missing the import fails loudly.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libzllm_hip.so")

# Every entry point include/zllm_hip.h declares.
EXPORTS = (
    "zhip_create", "zhip_destroy", "zhip_get_caps", "zhip_supports_prefill", "zhip_set_file", "zhip_execute",
    "zhip_profile_start", "zhip_profile_stop", "zhip_profile_read", "zhip_last_submit", "zhip_replayed_submits", "zhip_last_error",
    "zhip_force_loss", "zhip_kernel_artifact", "zhip_backend_source", "zhip_kernel_ordinal",
    "zhip_matmul_q8_0_float_no_alloc", "zhip_no_alloc_capacity",
)


class Options(C.Structure):
    _fields_ = [("device_index", C.c_uint32), ("flags", C.c_uint32)]


class Caps(C.Structure):
    _fields_ = [
        ("abi_version", C.c_uint32), ("compute_units", C.c_uint32), ("wavefront", C.c_uint32), ("lds_bytes", C.c_uint32),
        ("memory_bytes", C.c_uint64), ("memory_free", C.c_uint64), ("max_binding", C.c_uint64), ("offset_align", C.c_uint64),
        ("name", C.c_char * 128), ("arch", C.c_char * 32),
    ]


class CCompletion(C.Structure):
    _fields_ = [("token", C.c_uint32), ("status", C.c_uint32)]


class CTiming(C.Structure):
    _fields_ = [("pipeline", C.c_uint32), ("grid", C.c_uint32 * 3), ("ns", C.c_uint64), ("count", C.c_uint64)]


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is not built: run `python -m zllm_amd.build` (hipcc, gfx950). There is no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    ctx = C.c_void_p
    lib.zhip_create.restype = C.c_int32
    lib.zhip_create.argtypes = [C.POINTER(Options), C.POINTER(ctx)]
    lib.zhip_destroy.restype = C.c_int32
    lib.zhip_destroy.argtypes = [ctx]
    lib.zhip_get_caps.restype = C.c_int32
    lib.zhip_get_caps.argtypes = [ctx, C.POINTER(Caps)]
    lib.zhip_supports_prefill.restype = C.c_int32
    lib.zhip_supports_prefill.argtypes = [ctx, C.c_uint32]
    lib.zhip_set_file.restype = C.c_int32
    lib.zhip_set_file.argtypes = [ctx, C.c_void_p, C.c_size_t]
    lib.zhip_execute.restype = C.c_int32
    lib.zhip_execute.argtypes = [ctx, C.c_void_p, C.c_size_t, C.POINTER(CCompletion), C.c_size_t, C.POINTER(C.c_size_t)]
    lib.zhip_profile_start.restype = C.c_int32
    lib.zhip_profile_start.argtypes = [ctx]
    lib.zhip_profile_stop.restype = C.c_int32
    lib.zhip_profile_stop.argtypes = [ctx]
    lib.zhip_profile_read.restype = C.c_int32
    lib.zhip_profile_read.argtypes = [ctx, C.POINTER(CTiming), C.c_size_t, C.POINTER(C.c_size_t), C.POINTER(C.c_uint64)]
    lib.zhip_last_submit.restype = C.c_int32
    lib.zhip_last_submit.argtypes = [ctx, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
    lib.zhip_replayed_submits.restype = C.c_int32
    lib.zhip_replayed_submits.argtypes = [ctx, C.POINTER(C.c_uint64)]
    lib.zhip_last_error.restype = C.c_size_t
    lib.zhip_last_error.argtypes = [ctx, C.c_char_p, C.c_size_t]
    lib.zhip_force_loss.restype = C.c_int32
    lib.zhip_force_loss.argtypes = [ctx]
    lib.zhip_kernel_artifact.restype = C.c_size_t
    lib.zhip_kernel_artifact.argtypes = [C.c_char_p, C.c_uint32, C.c_char_p, C.c_size_t]
    lib.zhip_backend_source.restype = C.c_size_t
    lib.zhip_backend_source.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t]
    lib.zhip_kernel_ordinal.restype = C.c_int32
    lib.zhip_kernel_ordinal.argtypes = [C.c_char_p]
    lib.zhip_matmul_q8_0_float_no_alloc.restype = C.c_int32
    lib.zhip_matmul_q8_0_float_no_alloc.argtypes = [ctx, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_uint32] * 6
    lib.zhip_no_alloc_capacity.restype = C.c_uint64
    lib.zhip_no_alloc_capacity.argtypes = []
    return lib


lib = _load()


def kernel_artifact(name: str, variant: int) -> bytes:
    buf = C.create_string_buffer(128)
    n = lib.zhip_kernel_artifact(name.encode(), variant, buf, len(buf))
    return buf.raw[:n]


def backend_source(name: str) -> bytes:
    buf = C.create_string_buffer(256)
    n = lib.zhip_backend_source(name.encode(), buf, len(buf))
    return buf.raw[:n]


def kernel_ordinal(name: str) -> int:
    return lib.zhip_kernel_ordinal(name.encode())
