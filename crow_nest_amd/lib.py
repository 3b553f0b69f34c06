"""ctypes binding of libcrow_hip.so (the C ABI of include/crow_hip.h).

``build()`` compiles the library for gfx950 with the Makefile in ``csrc/``; ``lib()`` loads what is
built.  Nothing here computes anything on the CPU: a missing library or a failing call raises.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.environ.get("CROW_HIP_LIBRARY") or os.path.join(_HERE, "libcrow_hip.so")
_lib = None


class CrowHipError(RuntimeError):
    def __init__(self, code: int, what: str):
        self.code = code
        super().__init__(f"{what}: {error_string(code)} ({code})")


class Dims(C.Structure):
    _fields_ = [("gx", C.c_uint32), ("gy", C.c_uint32), ("gz", C.c_uint32), ("bx", C.c_uint32)]


def library_path() -> str:
    return _SO


def build(force: bool = True) -> None:
    cmd = ["make", "-C", os.path.join(_HERE, "csrc")] + (["-B"] if force else [])
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building libcrow_hip.so failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])


def lib():
    """The loaded library (not initialised: see ``init``)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        raise FileNotFoundError(f"{_SO} is not built (run __graft_entry__.build() or make -C crow_nest_amd/csrc)")
    L = C.CDLL(_SO)
    vp, u32, u64p, sz = C.c_void_p, C.c_uint32, C.POINTER(C.c_uint64), C.c_size_t
    sig = {
        "crow_hip_init": (C.c_int, [C.c_int]),
        "crow_hip_shutdown": (C.c_int, []),
        "crow_hip_error_string": (C.c_char_p, [C.c_int]),
        "crow_hip_device_name": (C.c_int, [C.c_char_p, sz]),
        "crow_hip_module_load": (C.c_int, [C.POINTER(vp)]),
        "crow_hip_module_unload": (C.c_int, [vp]),
        "crow_hip_module_get": (C.c_int, [vp, C.c_char_p, C.POINTER(vp)]),
        "crow_hip_get_function": (C.c_int, [C.c_char_p, C.POINTER(vp)]),
        "crow_hip_function_count": (C.c_int, []),
        "crow_hip_function_name": (C.c_char_p, [C.c_int]),
        "crow_hip_function_arg_count": (C.c_int, [vp]),
        "crow_hip_set_geo": (C.c_int, [C.c_int] * 4),
        "crow_hip_launch": (C.c_int, [vp, u32, u32, u32, u32, u64p, u32, vp]),
        "crow_hip_launch_noalloc": (C.c_int, [vp, u32, u32, u32, u32, u64p, u32, vp]),
        "crow_hip_launch_dims": (C.c_int, [C.c_char_p, u32, u32, u32, C.POINTER(Dims)]),
        "crow_hip_gemm_kernel": (C.c_char_p, [u32, u32]),
        "crow_hip_launch_dims_split": (C.c_int, [C.c_char_p, u32, u32, u32, u32, u32, C.POINTER(Dims)]),
        "crow_hip_status": (C.c_int, []),
        "crow_hip_reset_workspace": (C.c_int, []),
        "crow_hip_set_stream": (None, [vp]),
        "crow_hip_cur_stream": (vp, []),
        "crow_hip_sync": (C.c_int, []),
        "crow_hip_alloc": (C.c_int, [sz, C.POINTER(vp)]),
        "crow_hip_free": (C.c_int, [vp]),
        "crow_hip_upload": (C.c_int, [vp, vp, sz]),
        "crow_hip_download": (C.c_int, [vp, vp, sz]),
        "crow_hip_event_create": (C.c_int, [C.POINTER(vp)]),
        "crow_hip_event_record": (C.c_int, [vp]),
        "crow_hip_event_elapsed_ms": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
        "crow_hip_event_destroy": (C.c_int, [vp]),
        "crow_hip_time_launches": (C.c_int, [vp, u32, u32, u32, u32, u64p, u32, u32, u32, C.POINTER(C.c_float)]),
        "crow_hip_time_sequence": (C.c_int, [u32, C.POINTER(vp), C.POINTER(Dims), C.POINTER(u32), u64p, u32, u32, C.POINTER(C.c_float)]),
        "crow_hip_stream_create": (C.c_int, [C.POINTER(vp)]),
        "crow_hip_stream_destroy": (C.c_int, [vp]),
        "crow_hip_begin_capture": (C.c_int, [vp]),
        "crow_hip_end_capture_instantiate": (C.c_int, [vp, C.POINTER(vp)]),
        "crow_hip_launch_graph": (C.c_int, [vp, vp]),
        "crow_hip_graph_exec_destroy": (C.c_int, [vp]),
        "crow_hip_time_graph": (C.c_int, [vp, vp, u32, C.POINTER(C.c_float)]),
        "crow_hip_time_pure_read": (C.c_int, [u64p, u32, sz, u32, u32, u32, u32, C.POINTER(C.c_float)]),
        "crow_hip_container_bytes": (sz, [u32, u32]),
        "crow_hip_tiled_bytes": (sz, [u32, u32]),
        "crow_hip_tile_code_offset": (u32, [u32, u32]),
        "crow_hip_tile_scale_offset": (u32, [u32, u32]),
        "crow_hip_repack_nvfp4": (C.c_int, [vp, u32, u32, vp]),
        "crow_hip_unpack_nvfp4": (C.c_int, [vp, u32, u32, vp]),
        "crow_hip_dequant_tiled": (C.c_int, [vp, vp, u32, u32, vp]),
        "crow_hip_quantize_nvfp4": (C.c_int, [vp, sz, vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)  # AttributeError here = the library does not export what the header declares
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


# include/crow_hip_bench.h: timing loops and the forced GEMV split, for bench.py and the tests (not part of the drop-in ABI)
BENCH_EXPORTS = ["crow_hip_launch_dims_split", "crow_hip_time_launches", "crow_hip_time_sequence", "crow_hip_time_graph", "crow_hip_time_pure_read"]

EXPORTS = [
    "crow_hip_init", "crow_hip_shutdown", "crow_hip_error_string", "crow_hip_device_name", "crow_hip_module_load",
    "crow_hip_module_unload", "crow_hip_module_get", "crow_hip_get_function", "crow_hip_function_count",
    "crow_hip_function_name", "crow_hip_function_arg_count", "crow_hip_set_geo", "crow_hip_launch", "crow_hip_launch_noalloc",
    "crow_hip_launch_dims", "crow_hip_gemm_kernel", "crow_hip_status", "crow_hip_reset_workspace", "crow_hip_set_stream", "crow_hip_cur_stream",
    "crow_hip_sync", "crow_hip_event_create", "crow_hip_event_record", "crow_hip_event_elapsed_ms", "crow_hip_event_destroy", "crow_hip_alloc", "crow_hip_free", "crow_hip_upload", "crow_hip_download",
    "crow_hip_stream_create", "crow_hip_stream_destroy", "crow_hip_begin_capture", "crow_hip_end_capture_instantiate",
    "crow_hip_launch_graph", "crow_hip_graph_exec_destroy",
    "crow_hip_container_bytes", "crow_hip_tiled_bytes", "crow_hip_tile_code_offset", "crow_hip_tile_scale_offset", "crow_hip_repack_nvfp4", "crow_hip_unpack_nvfp4",
    "crow_hip_dequant_tiled", "crow_hip_quantize_nvfp4",
]


def error_string(code: int) -> str:
    try:
        return lib().crow_hip_error_string(code).decode()
    except Exception:  # the library itself is missing
        return "libcrow_hip.so not loaded"


def check(code: int, what: str) -> None:
    if code != 0:
        raise CrowHipError(code, what)


_inited = False


def init(device: int = 0) -> None:
    """``Ctx::init`` of the reference (engine/src/cuda.rs:435): device, workspace, kernel table."""
    global _inited
    check(lib().crow_hip_init(device), "crow_hip_init")
    _inited = True


def ensure_init() -> None:
    if not _inited:
        init(0)
