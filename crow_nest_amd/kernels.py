"""Host-side mirror of the reference's kernel table and launch shim for the NVFP4 path.

Reference interface (engine/src/kernels.rs:5128-5348, engine/src/cuda.rs:274-284,485-509):

    let module = cuda::compile(&kgeo.source());      ->  module = compile(geo)
    let k = Kernels::new(&module, p2);               ->  k = Kernels(module)
    launch_v(k.f("gemv_nvfp4_w"), gx, gy, gz, bx, &[w, x, gs, y, k_p, rows_p]);
                                                      ->  launch_v(k.f("gemv_nvfp4_w"), gx, gy, gz, bx, [w, x, gs, y, k_p, rows_p])

Same names, same argument meaning (every value a device address), same failure behaviour: a missing
name raises ``KernelMissing("kernel missing: <name>")`` where the reference panics with that text; a
HIP error raises where the reference's ``cuda::ck`` panics.  Grid and block come from
``launch_dims`` so that wave64 geometry stays inside the library.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

from . import lib as _l


class KernelMissing(KeyError):
    pass


# crow_hip.h: CROW_DIMS_COUNT_FROM_MEMORY - launch_dims(name, rows, k, COUNT_FROM_MEMORY | capacity): the launch reads its row
# count from the device word behind m_p / t_p (the reference's convention: a fixed grid, the word rewritten per step)
COUNT_FROM_MEMORY = 0x80000000


@dataclass(frozen=True)
class KernelGeo:
    """The geometry the reference bakes into its kernel source (kernels.rs:5040-5125, CN_* defines)."""
    experts: int = 0
    topk: int = 0
    hidden: int = 0
    inter: int = 0


class Module:
    """``cuda::Module``: the loaded code objects (here: the ahead-of-time gfx950 objects in the library)."""

    def __init__(self, handle: int):
        self.handle = handle

    def get(self, name: str) -> int:
        out = C.c_void_p()
        rc = _l.lib().crow_hip_module_get(self.handle, name.encode(), C.byref(out))
        if rc == -2:
            raise KernelMissing(f"kernel missing: {name}")
        _l.check(rc, f"Module::get({name})")
        return out.value

    def unload(self) -> None:
        if self.handle:
            _l.check(_l.lib().crow_hip_module_unload(self.handle), "Module::unload")
            self.handle = 0


def compile(geo: KernelGeo | None = None) -> Module:  # noqa: A001 - the reference's name
    """``cuda::compile``: nothing is compiled at run time; loads the module and writes the geometry."""
    _l.ensure_init()
    out = C.c_void_p()
    _l.check(_l.lib().crow_hip_module_load(C.byref(out)), "crow_hip_module_load")
    if geo is not None:
        set_geo(geo)
    return Module(out.value)


def set_geo(geo: KernelGeo) -> None:
    _l.ensure_init()
    _l.check(_l.lib().crow_hip_set_geo(geo.experts, geo.topk, geo.hidden, geo.inter), "crow_hip_set_geo")


class Kernels:
    """``Kernels::new`` resolves every launched name once; ``f`` looks one up."""

    def __init__(self, module: Module):
        L = _l.lib()
        self.map = {}
        for i in range(L.crow_hip_function_count()):
            name = L.crow_hip_function_name(i).decode()
            self.map[name] = module.get(name)

    def f(self, name: str) -> int:
        try:
            return self.map[name]
        except KeyError:
            raise KernelMissing(f"kernel missing: {name}") from None


def launch_v(f: int, gx: int, gy: int, gz: int, bx: int, vals) -> None:
    """``launch_v``: asynchronous launch on the current stream; every value is a device address."""
    n = len(vals)
    arr = (C.c_uint64 * n)(*[int(v) for v in vals])
    _l.check(_l.lib().crow_hip_launch(f, gx, gy, gz, bx, arr, n, None), "launch_v")


def launch_noalloc(f: int, gx: int, gy: int, gz: int, bx: int, vals) -> None:
    """``launch_v`` for callers that may not allocate device memory: the kernels' scratch (split-K partial sums, arrival
    counters, status, the head's key) is a fixed array inside the library; a split beyond its size raises."""
    n = len(vals)
    arr = (C.c_uint64 * n)(*[int(v) for v in vals])
    _l.check(_l.lib().crow_hip_launch_noalloc(f, gx, gy, gz, bx, arr, n, None), "launch_noalloc")


def sync() -> None:
    _l.check(_l.lib().crow_hip_sync(), "sync")


def launch_sync(f: int, gx: int, gy: int, gz: int, bx: int, vals) -> None:
    launch_v(f, gx, gy, gz, bx, vals)
    sync()


def status() -> None:
    """Raise if a launch since the last call refused its shape or did not fit the workspace."""
    _l.check(_l.lib().crow_hip_status(), "kernel status")


def launch_dims(name: str, rows: int, k_dim: int, z: int = 1, split: tuple[int, int] = (0, 0)) -> tuple[int, int, int, int]:
    """Grid and block the library chooses; `split` = (column slices per strip, waves per block and tensor) forces a GEMV split."""
    d = _l.Dims()
    rc = _l.lib().crow_hip_launch_dims_split(name.encode(), rows, k_dim, z, split[0], split[1], C.byref(d))
    if rc == -2:
        raise KernelMissing(f"kernel missing: {name}")
    _l.check(rc, f"launch_dims({name}, {rows}, {k_dim}, {z})")
    return d.gx, d.gy, d.gz, d.bx


def time_launches(f: int, gx: int, gy: int, gz: int, bx: int, arg_sets, iters: int) -> float:
    """Mean microseconds per launch over `iters` back-to-back launches that rotate over `arg_sets`
    (the loop runs inside the library, between two HIP events on the launch stream)."""
    n = len(arg_sets[0])
    flat = [int(v) for s in arg_sets for v in s]
    arr = (C.c_uint64 * len(flat))(*flat)
    us = C.c_float()
    _l.check(_l.lib().crow_hip_time_launches(f, gx, gy, gz, bx, arr, n, len(arg_sets), iters, C.byref(us)), "crow_hip_time_launches")
    return float(us.value)


def time_pure_read(buffers, nbytes: int, blocks: int, threads: int, iters: int, pattern: int = 0) -> float:
    """Mean microseconds per launch of a kernel that only READS `nbytes` (a multiple of 2304) of each of the device
    `buffers` in turn: the chip's ceiling for that many bytes (measurement only).  pattern 0 = the GEMVs' own requests
    (2304-byte groups, four in flight per wave), 1 = 16 contiguous bytes per lane, non-temporal, 2 = the same, plain loads."""
    arr = (C.c_uint64 * len(buffers))(*[int(b) for b in buffers])
    us = C.c_float()
    _l.check(_l.lib().crow_hip_time_pure_read(arr, len(buffers), nbytes, blocks, threads, pattern, iters, C.byref(us)), "crow_hip_time_pure_read")
    return float(us.value)


def time_sequence(kernels, n_sets: int, iters: int) -> float:
    """Mean microseconds per iteration of a launch SEQUENCE.  `kernels` = [(f, (gx, gy, gz, bx), arg_sets), ...];
    every kernel has `n_sets` argument sets (a kernel with one set repeats it); iteration i uses set i % n_sets."""
    nk = len(kernels)
    fns = (C.c_void_p * nk)(*[k[0] for k in kernels])
    dims = (_l.Dims * nk)(*[_l.Dims(*k[1]) for k in kernels])
    nv = (C.c_uint32 * nk)(*[len(k[2][0]) for k in kernels])
    flat = []
    for s in range(n_sets):
        for _, _, sets in kernels:
            flat.extend(int(v) for v in sets[s % len(sets)])
    arr = (C.c_uint64 * len(flat))(*flat)
    us = C.c_float()
    _l.check(_l.lib().crow_hip_time_sequence(nk, fns, dims, nv, arr, n_sets, iters, C.byref(us)), "crow_hip_time_sequence")
    return float(us.value)


class Graph:
    """A captured launch sequence (the reference's CROW_GRAPH path, engine/src/cuda.rs:113-203):

        g = Graph()
        with g.capture():           # begin_capture on the graph's own non-blocking stream; launch_v records
            launch_v(...); launch_v(...)
        g.launch()                  # launch_graph on that stream
    """

    def __init__(self):
        _l.ensure_init()
        s = C.c_void_p()
        _l.check(_l.lib().crow_hip_stream_create(C.byref(s)), "crow_hip_stream_create")
        self.stream = s
        self.exec = C.c_void_p()

    class _Capture:
        def __init__(self, g):
            self.g = g

        def __enter__(self):
            self.prev = _l.lib().crow_hip_cur_stream()
            _l.check(_l.lib().crow_hip_begin_capture(self.g.stream), "crow_hip_begin_capture")
            return self.g

        def __exit__(self, et, ev, tb):
            rc = _l.lib().crow_hip_end_capture_instantiate(self.g.stream, C.byref(self.g.exec))
            _l.lib().crow_hip_set_stream(self.prev)
            if et is None:
                _l.check(rc, "crow_hip_end_capture_instantiate")
            return False

    def capture(self):
        return Graph._Capture(self)

    def launch(self) -> None:
        _l.check(_l.lib().crow_hip_launch_graph(self.exec, self.stream), "crow_hip_launch_graph")

    def sync(self) -> None:
        import torch
        torch.cuda.synchronize()

    def time(self, iters: int) -> float:
        us = C.c_float()
        _l.check(_l.lib().crow_hip_time_graph(self.exec, self.stream, iters, C.byref(us)), "crow_hip_time_graph")
        return float(us.value)

    def close(self) -> None:
        if self.exec:
            _l.lib().crow_hip_graph_exec_destroy(self.exec)
            self.exec = C.c_void_p()
        if self.stream:
            _l.lib().crow_hip_stream_destroy(self.stream)
            self.stream = C.c_void_p()


class Event:
    """A HIP event on the library's current stream (the stream every launch_v goes to)."""

    def __init__(self):
        h = C.c_void_p()
        _l.check(_l.lib().crow_hip_event_create(C.byref(h)), "crow_hip_event_create")
        self.h = h

    def record(self) -> "Event":
        _l.check(_l.lib().crow_hip_event_record(self.h), "crow_hip_event_record")
        return self

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        _l.check(_l.lib().crow_hip_event_elapsed_ms(self.h, stop.h, C.byref(ms)), "crow_hip_event_elapsed_ms")
        return float(ms.value)

    def __del__(self):
        try:
            _l.lib().crow_hip_event_destroy(self.h)
        except Exception:
            pass
