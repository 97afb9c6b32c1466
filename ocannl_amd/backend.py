"""Host-side mirror of OCANNL's ``Lowered_backend`` for the MI355X library (ctypes over the
C ABI in ``include/ocannl_hip.h``).

Names, argument meaning and error behaviour follow ``Backend_impl.Lowered_backend``
(arrayjit/lib/backend_impl.ml:292-367) and the included ``Backend_device_common`` /
``Slab_alloc`` signatures (arrayjit/lib/backend_intf.ml:22-37,206-266): ``compile``, ``link``,
``from_host``, ``to_host``, ``device_to_device``, ``alloc_pool``, ``free_pool``, ``memset_zero``,
``sync``, ``is_done``, ``will_wait_for``, ``all_work``, ``await_``, ``is_idle``, ``get_device``,
``num_devices``, ``get_used_memory``, ``static_properties``.  This is what an OCaml
``hip_backend.ml`` does through ``Foreign.foreign``; the tests drive the same entry points.

:class:`Context` is the small part of the shared layer above the boundary that the tests and the
benchmark need: pool planning and zero-initialisation as ``Backends.allocate_delta`` does
(arrayjit/lib/backends.ml:22-51,529-614), and host transfers as ``Context.set_values`` /
``get_values`` do (arrayjit/lib/context.ml:322-401).

There is no CPU fallback: a missing or unloadable library raises at import of the symbols.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Iterable, List, Mapping, Optional, Sequence

import numpy as np

from . import llir as L

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libocannl_hip.so")


class User_error(Exception):
    """``Utils.User_error``: a user mistake (bad static index, node missing from context...)."""


class Invalid_argument(ValueError):
    """OCaml ``Invalid_argument``: misuse of the interface or malformed IR."""


class Failure(RuntimeError):
    """OCaml ``Failure``: the HIP runtime or hiprtc failed."""


class _NodeLoc(ctypes.Structure):
    _fields_ = [("node_id", ctypes.c_int32), ("pool_id", ctypes.c_int32), ("offset", ctypes.c_uint64)]


class _Kparam(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("id", ctypes.c_int32), ("size_bytes", ctypes.c_int64)]


class KernelInfo(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("coop_lanes", ctypes.c_int32), ("flops", ctypes.c_double),
                ("bytes", ctypes.c_double), ("m", ctypes.c_int64), ("n", ctypes.c_int64),
                ("k", ctypes.c_int64), ("batch", ctypes.c_int64), ("name", ctypes.c_char * 96),
                ("queue", ctypes.c_int32), ("reserved", ctypes.c_int32)]

    KINDS = ("generated", "fill", "mfma")

    def as_dict(self):
        return {"kind": self.KINDS[self.kind], "coop_lanes": self.coop_lanes, "flops": self.flops,
                "bytes": self.bytes, "m": self.m, "n": self.n, "k": self.k, "batch": self.batch,
                "name": self.name.decode(), "queue": self.queue}


# every symbol include/ocannl_hip.h declares
EXPORTS = (
    "ocannl_hip_last_error", "ocannl_hip_init", "ocannl_hip_num_devices", "ocannl_hip_get_device",
    "ocannl_hip_get_name", "ocannl_hip_static_properties", "ocannl_hip_get_used_memory",
    "ocannl_hip_get_debug_info", "ocannl_hip_get_global_debug_info", "ocannl_hip_await", "ocannl_hip_is_idle", "ocannl_hip_all_work",
    "ocannl_hip_sync", "ocannl_hip_is_done", "ocannl_hip_will_wait_for", "ocannl_hip_event_free",
    "ocannl_hip_alloc_pool", "ocannl_hip_free_pool", "ocannl_hip_memset_zero", "ocannl_hip_from_host",
    "ocannl_hip_to_host", "ocannl_hip_device_to_device", "ocannl_hip_compile",
    "ocannl_hip_compile_opts", "ocannl_hip_code_free", "ocannl_hip_code_num_routines",
    "ocannl_hip_code_routine_name", "ocannl_hip_code_kparams", "ocannl_hip_code_source", "ocannl_hip_code_object",
    "ocannl_hip_code_num_kernels", "ocannl_hip_code_kernel_info", "ocannl_hip_link",
    "ocannl_hip_routine_free", "ocannl_hip_routine_set_static", "ocannl_hip_routine_run",
    "ocannl_hip_routine_run_static_scratch", "ocannl_hip_routine_log_id", "ocannl_hip_routine_run_timed",
    "ocannl_hip_routine_profile_kernel", "ocannl_hip_routine_profile_read",
)

_lib = None


def load_library() -> ctypes.CDLL:
    """dlopen the in-tree library; fails loudly when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise Failure(f"{LIB_PATH} is missing: build it with `make -C ocannl_amd/csrc` "
                      "(there is no CPU fallback for the hip backend)")
    lib = ctypes.CDLL(LIB_PATH)
    vp, i32, u64, i64, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_int64, ctypes.c_size_t
    P = ctypes.POINTER
    sigs = {
        "ocannl_hip_last_error": (ctypes.c_char_p, []),
        "ocannl_hip_init": (i32, []),
        "ocannl_hip_num_devices": (i32, [P(i32)]),
        "ocannl_hip_get_device": (i32, [i32, P(vp)]),
        "ocannl_hip_get_name": (i32, [vp, ctypes.c_char_p, sz]),
        "ocannl_hip_static_properties": (i32, [ctypes.c_char_p, sz]),
        "ocannl_hip_get_used_memory": (i32, [vp, P(u64)]),
        "ocannl_hip_get_debug_info": (i32, [vp, ctypes.c_char_p, sz]),
        "ocannl_hip_get_global_debug_info": (i32, [ctypes.c_char_p, sz]),
        "ocannl_hip_await": (i32, [vp]),
        "ocannl_hip_is_idle": (i32, [vp, P(i32)]),
        "ocannl_hip_all_work": (i32, [vp, P(vp)]),
        "ocannl_hip_sync": (i32, [vp]),
        "ocannl_hip_is_done": (i32, [vp, P(i32)]),
        "ocannl_hip_will_wait_for": (i32, [vp, vp]),
        "ocannl_hip_event_free": (None, [vp]),
        "ocannl_hip_alloc_pool": (i32, [vp, i32, u64, u64]),
        "ocannl_hip_free_pool": (i32, [vp, i32]),
        "ocannl_hip_memset_zero": (i32, [vp, i32, u64, u64]),
        "ocannl_hip_from_host": (i32, [vp, i32, u64, vp, u64]),
        "ocannl_hip_to_host": (i32, [vp, i32, u64, vp, u64]),
        "ocannl_hip_device_to_device": (i32, [vp, i32, u64, vp, i32, u64, u64]),
        "ocannl_hip_compile": (i32, [ctypes.c_char_p, sz, P(vp)]),
        "ocannl_hip_compile_opts": (i32, [ctypes.c_char_p, sz, ctypes.c_char_p, P(vp)]),
        "ocannl_hip_code_free": (None, [vp]),
        "ocannl_hip_code_num_routines": (i32, [vp, P(i32)]),
        "ocannl_hip_code_routine_name": (i32, [vp, i32, ctypes.c_char_p, sz]),
        "ocannl_hip_code_kparams": (i32, [vp, i32, P(_Kparam), i32, P(i32)]),
        "ocannl_hip_code_source": (i32, [vp, ctypes.c_char_p, sz, P(sz)]),
        "ocannl_hip_code_object": (i32, [vp, i32, ctypes.c_char_p, sz, P(sz)]),
        "ocannl_hip_code_num_kernels": (i32, [vp, i32, P(i32)]),
        "ocannl_hip_code_kernel_info": (i32, [vp, i32, i32, P(KernelInfo)]),
        "ocannl_hip_link": (i32, [vp, vp, i32, P(_NodeLoc), i32, P(vp)]),
        "ocannl_hip_routine_free": (None, [vp]),
        "ocannl_hip_routine_set_static": (i32, [vp, i32, i64]),
        "ocannl_hip_routine_run": (i32, [vp]),
        "ocannl_hip_routine_run_static_scratch": (i32, [vp]),
        "ocannl_hip_routine_log_id": (i32, [vp, P(i32)]),
        "ocannl_hip_routine_run_timed": (i32, [vp, P(ctypes.c_float), i32]),
        "ocannl_hip_routine_profile_kernel": (i32, [vp, i32]),
        "ocannl_hip_routine_profile_read": (i32, [vp, P(ctypes.c_double), P(i64)]),
    }
    for name in EXPORTS:
        fn = getattr(lib, name)   # AttributeError if the library lacks a declared symbol
        fn.restype, fn.argtypes = sigs[name]
    _lib = lib
    return lib


def _check(rc: int) -> None:
    if rc == 0:
        return
    msg = load_library().ocannl_hip_last_error().decode(errors="replace")
    if rc == -1:
        raise User_error(msg)
    if rc == -2:
        raise Invalid_argument(msg)
    raise Failure(msg)


# ----------------------------------------------------------------------------------------------
# Lowered_backend
# ----------------------------------------------------------------------------------------------

class Event:
    def __init__(self, handle):
        self._h = handle

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.ocannl_hip_event_free(self._h)
            self._h = None


class Device:
    def __init__(self, handle, ordinal):
        self._h = handle
        self.ordinal = ordinal


def initialize() -> None:
    _check(load_library().ocannl_hip_init())


def num_devices() -> int:
    n = ctypes.c_int()
    _check(load_library().ocannl_hip_num_devices(ctypes.byref(n)))
    return n.value


def get_device(ordinal: int = 0) -> Device:
    h = ctypes.c_void_p()
    _check(load_library().ocannl_hip_get_device(ordinal, ctypes.byref(h)))
    return Device(h, ordinal)


def get_name(dev: Device) -> str:
    buf = ctypes.create_string_buffer(64)
    _check(load_library().ocannl_hip_get_name(dev._h, buf, 64))
    return buf.value.decode()


def static_properties() -> str:
    buf = ctypes.create_string_buffer(1 << 16)
    _check(load_library().ocannl_hip_static_properties(buf, 1 << 16))
    return buf.value.decode()


def get_used_memory(dev: Device) -> int:
    n = ctypes.c_uint64()
    _check(load_library().ocannl_hip_get_used_memory(dev._h, ctypes.byref(n)))
    return n.value


def get_debug_info(dev: Device) -> str:
    buf = ctypes.create_string_buffer(4096)
    _check(load_library().ocannl_hip_get_debug_info(dev._h, buf, 4096))
    return buf.value.decode()


def get_global_debug_info() -> str:
    """``get_global_debug_info`` (backend_intf.ml:242; cuda_backend.ml:1088-1090): process-wide counters."""
    buf = ctypes.create_string_buffer(4096)
    _check(load_library().ocannl_hip_get_global_debug_info(buf, 4096))
    return buf.value.decode()


def await_(dev: Device) -> None:
    _check(load_library().ocannl_hip_await(dev._h))


def is_idle(dev: Device) -> bool:
    v = ctypes.c_int()
    _check(load_library().ocannl_hip_is_idle(dev._h, ctypes.byref(v)))
    return bool(v.value)


def all_work(dev: Device) -> Event:
    h = ctypes.c_void_p()
    _check(load_library().ocannl_hip_all_work(dev._h, ctypes.byref(h)))
    return Event(h)


def sync(ev: Event) -> None:
    _check(load_library().ocannl_hip_sync(ev._h))


def is_done(ev: Event) -> bool:
    v = ctypes.c_int()
    _check(load_library().ocannl_hip_is_done(ev._h, ctypes.byref(v)))
    return bool(v.value)


def will_wait_for(dev: Device, ev: Event) -> None:
    _check(load_library().ocannl_hip_will_wait_for(dev._h, ev._h))


def alloc_pool(dev: Device, *, pool_id: int, size_in_bytes: int, alignment: int = 256) -> None:
    _check(load_library().ocannl_hip_alloc_pool(dev._h, pool_id, size_in_bytes, alignment))


def free_pool(dev: Device, *, pool_id: int) -> None:
    _check(load_library().ocannl_hip_free_pool(dev._h, pool_id))


def memset_zero(dev: Device, *, pool_id: int, offset: int, size_in_bytes: int) -> None:
    _check(load_library().ocannl_hip_memset_zero(dev._h, pool_id, offset, size_in_bytes))


def from_host(dev: Device, *, pool_id: int, offset: int, src: np.ndarray) -> None:
    assert src.flags["C_CONTIGUOUS"]
    _check(load_library().ocannl_hip_from_host(dev._h, pool_id, offset, src.ctypes.data, src.nbytes))


def to_host(dev: Device, *, pool_id: int, offset: int, dst: np.ndarray) -> None:
    assert dst.flags["C_CONTIGUOUS"] and dst.flags["WRITEABLE"]
    _check(load_library().ocannl_hip_to_host(dev._h, pool_id, offset, dst.ctypes.data, dst.nbytes))


def device_to_device(*, dst: Device, dst_pool_id: int, dst_offset: int, src: Device, src_pool_id: int,
                     src_offset: int, size_in_bytes: int) -> None:
    _check(load_library().ocannl_hip_device_to_device(dst._h, dst_pool_id, dst_offset, src._h,
                                                      src_pool_id, src_offset, size_in_bytes))


class Code:
    """``Lowered_backend.code`` / ``code_batch``."""

    def __init__(self, handle, routines: Sequence[L.Routine]):
        self._h = handle
        self.routines = list(routines)

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.ocannl_hip_code_free(self._h)
            self._h = None

    def index_of(self, name: str) -> int:
        for i, r in enumerate(self.routines):
            if r.name == name:
                return i
        raise Invalid_argument(f"no routine named {name}")

    def source(self) -> str:
        need = ctypes.c_size_t()
        _check(load_library().ocannl_hip_code_source(self._h, None, 0, ctypes.byref(need)))
        buf = ctypes.create_string_buffer(need.value)
        _check(load_library().ocannl_hip_code_source(self._h, buf, need.value, None))
        return buf.value.decode()

    def code_object(self, index: int = 0) -> bytes:
        """The gfx950 code object of the routine's generated kernels (the ``.ptx`` dump of
        cuda_backend.ml:193-202 under ``output_debug_files_in_build_directory``)."""
        need = ctypes.c_size_t()
        _check(load_library().ocannl_hip_code_object(self._h, index, None, 0, ctypes.byref(need)))
        buf = ctypes.create_string_buffer(max(need.value, 1))
        _check(load_library().ocannl_hip_code_object(self._h, index, buf, need.value, None))
        return buf.raw[:need.value]

    def kernels(self, index: int = 0) -> List[dict]:
        n = ctypes.c_int()
        _check(load_library().ocannl_hip_code_num_kernels(self._h, index, ctypes.byref(n)))
        out = []
        for k in range(n.value):
            info = KernelInfo()
            _check(load_library().ocannl_hip_code_kernel_info(self._h, index, k, ctypes.byref(info)))
            out.append(info.as_dict())
        return out

    def kparams(self, index: int = 0) -> List[tuple]:
        n = ctypes.c_int()
        _check(load_library().ocannl_hip_code_kparams(self._h, index, None, 0, ctypes.byref(n)))
        arr = (_Kparam * max(n.value, 1))()
        _check(load_library().ocannl_hip_code_kparams(self._h, index, arr, n.value, ctypes.byref(n)))
        kinds = ("ptr", "static_idx", "merge_buffer")
        return [(kinds[arr[i].kind], arr[i].id, arr[i].size_bytes) for i in range(n.value)]


def compile(routine: L.Routine, options: Optional[str] = None) -> Code:  # noqa: A001
    """``Lowered_backend.compile ~name bindings optimized`` (backend_impl.ml:347)."""
    return compile_batch([routine], options)


def compile_batch(routines: Sequence[L.Routine], options: Optional[str] = None) -> Code:
    """``Lowered_backend.compile_batch`` (backend_impl.ml:349-353)."""
    # with debug_log=1 every Set carries its text, as Low_level.Set's `debug` field does
    # (the option is read as the library reads it: any value but "0" switches logging on)
    debug = any(kv.split("=", 1)[0].strip() == "debug_log" and kv.split("=", 1)[1].strip() != "0"
                for kv in (options or "").split(";") if "=" in kv)
    text = "".join(L.to_wire(r, debug=debug) for r in routines).encode()
    h = ctypes.c_void_p()
    lib = load_library()
    if options is None:
        _check(lib.ocannl_hip_compile(text, len(text), ctypes.byref(h)))
    else:
        _check(lib.ocannl_hip_compile_opts(text, len(text), options.encode(), ctypes.byref(h)))
    return Code(h, routines)


class Routine:
    """The linked launch closure: ``lowered_bindings * Task.t`` (backend_impl.ml:355)."""

    def __init__(self, handle, code: Code, index: int, dev: Device):
        self._h = handle
        self.code = code   # context_lifetime: keep the code alive
        self.index = index
        self.dev = dev
        self.llir = code.routines[index]

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.ocannl_hip_routine_free(self._h)
            self._h = None

    def set_static(self, sym: int, value: int) -> None:
        _check(load_library().ocannl_hip_routine_set_static(self._h, sym, value))

    def run(self) -> None:
        """``Task.run``: checks static indices, enqueues the kernels; asynchronous."""
        _check(load_library().ocannl_hip_routine_run(self._h))

    def run_static_scratch(self) -> None:
        """``run`` with the routine's scratch memory taken from the library's static device array:
        allocates nothing; refuses (``User_error``) a routine whose scratch needs exceed it."""
        _check(load_library().ocannl_hip_routine_run_static_scratch(self._h))

    def log_id(self) -> int:
        """The prefix of the log lines of this routine's latest run (``debug_log=1``)."""
        v = ctypes.c_int()
        _check(load_library().ocannl_hip_routine_log_id(self._h, ctypes.byref(v)))
        return v.value

    def profile_kernel(self, kernel_index: int) -> None:
        _check(load_library().ocannl_hip_routine_profile_kernel(self._h, kernel_index))

    def profile_read(self):
        ms, n = ctypes.c_double(), ctypes.c_int64()
        _check(load_library().ocannl_hip_routine_profile_read(self._h, ctypes.byref(ms), ctypes.byref(n)))
        return ms.value, n.value

    def run_timed(self) -> List[float]:
        n = len(self.code.kernels(self.index))
        arr = (ctypes.c_float * max(n, 1))()
        _check(load_library().ocannl_hip_routine_run_timed(self._h, arr, n))
        return [arr[i] for i in range(n)]


def link(dev: Device, code: Code, ctx_buffers: Mapping[int, tuple], index: int = 0) -> Routine:
    """``Lowered_backend.link context code ctx_buffers``; ``ctx_buffers`` maps node id ->
    ``(pool_id, offset)`` (``Backend_intf.buffer_loc``)."""
    locs = (_NodeLoc * max(len(ctx_buffers), 1))()
    for i, (nid, (pool, off)) in enumerate(ctx_buffers.items()):
        locs[i] = _NodeLoc(nid, pool, off)
    h = ctypes.c_void_p()
    _check(load_library().ocannl_hip_link(dev._h, code._h, index, locs, len(ctx_buffers), ctypes.byref(h)))
    return Routine(h, code, index, dev)


# ----------------------------------------------------------------------------------------------
# the slice of the shared layer the tests need
# ----------------------------------------------------------------------------------------------

NP_DTYPE = {
    "byte": np.uint8, "uint16": np.uint16, "int32": np.int32, "uint32": np.uint32,
    "int64": np.int64, "uint64": np.uint64, "half": np.float16, "bfloat16": np.uint16,
    "fp8": np.uint8, "single": np.float32, "double": np.float64,
}


def plan_pool_segments(items: Sequence[tuple], cap: int = 1 << 62):
    """``Backends.plan_pool_segments`` (backends.ml:22-51): bump-pack (size, align) items into
    pools, opening a new pool when the cap would be exceeded."""
    def align_up(off, a):
        return off if a <= 1 else (off + a - 1) // a * a

    seg, bump, closed, out = 0, 0, [], []
    for size, align in items:
        if size > cap:
            raise User_error(f"tensor node needs {size} bytes, over the {cap}-byte per-pool cap")
        off = align_up(bump, align)
        if off + size > cap:
            closed.append(bump)
            seg += 1
            bump = size
            out.append((seg, 0))
        else:
            bump = off + size
            out.append((seg, off))
    sizes = (closed + [bump]) if items else []
    return out, sizes


class Context:
    """Device buffers for a set of tensor nodes, one bump-packed pool per allocation round, zeroed
    at allocation (backends.ml:529-614), with host access as ``Context.set_values/get_values``."""

    _next_pool = [1]   # pool 0 is the merge buffer (cuda_backend.ml:71-76)

    def __init__(self, dev: Optional[Device] = None):
        self.dev = dev or get_device(0)
        self.ctx_buffers: Dict[int, tuple] = {}
        self.nodes: Dict[int, L.Node] = {}
        self.pools: List[int] = []

    def allocate(self, nodes: Iterable[L.Node]) -> None:
        new = [n for n in nodes if n.mode == "ctx" and n.id not in self.ctx_buffers]
        if not new:
            return
        assign, sizes = plan_pool_segments([(n.size_in_bytes, 256) for n in new])
        base = self._next_pool[0]
        for k, size in enumerate(sizes):
            alloc_pool(self.dev, pool_id=base + k, size_in_bytes=size, alignment=256)
            memset_zero(self.dev, pool_id=base + k, offset=0, size_in_bytes=size)
            self.pools.append(base + k)
        self._next_pool[0] += len(sizes)
        for n, (seg, off) in zip(new, assign):
            self.ctx_buffers[n.id] = (base + seg, off)
            self.nodes[n.id] = n

    def link(self, code: Code, index: int = 0) -> Routine:
        r = code.routines[index]
        self.allocate(r.param_nodes())
        need = {n.id: self.ctx_buffers[n.id] for n in r.param_nodes()}
        return link(self.dev, code, need, index)

    def set_values(self, node: L.Node, values: np.ndarray) -> None:
        self.allocate([node])
        pool, off = self.ctx_buffers[node.id]
        a = np.ascontiguousarray(values)
        assert a.nbytes == node.size_in_bytes, (node, a.shape, a.dtype)
        from_host(self.dev, pool_id=pool, offset=off, src=a)
        await_(self.dev)

    def get_values(self, node: L.Node) -> np.ndarray:
        pool, off = self.ctx_buffers[node.id]
        if node.prec == "uint4x32":
            out = np.empty(node.dims + (4,), np.uint32)
        else:
            out = np.empty(node.dims, NP_DTYPE[node.prec])
        await_(self.dev)
        to_host(self.dev, pool_id=pool, offset=off, dst=out)
        await_(self.dev)
        return out

    def free(self) -> None:
        await_(self.dev)
        for p in self.pools:
            free_pool(self.dev, pool_id=p)
        self.pools = []
        self.ctx_buffers = {}


class HipRun:
    """One routine compiled, given a context of its own with the given initial values, and linked:
    what a test or a benchmark steps (``Train.to_routine`` + ``Context.run``, lib/train.ml:108-170)."""

    def __init__(self, routine: L.Routine, init: Mapping[int, np.ndarray], options: Optional[str] = None):
        import sys
        self.B = sys.modules[__name__]   # the backend module, for callers that hold only the run
        self.routine = routine
        self.code = compile(routine, options)
        self.ctx = Context()
        self.ctx.allocate(routine.param_nodes())
        for n in routine.param_nodes():
            if n.id in init:
                self.ctx.set_values(n, init[n.id])
        self.rt = self.ctx.link(self.code)

    def step(self, static: Optional[Mapping[int, int]] = None, static_scratch: bool = False):
        for sym, v in (static or {}).items():
            self.rt.set_static(sym, v)
        if static_scratch:
            self.rt.run_static_scratch()
        else:
            self.rt.run()

    def get(self, node: L.Node) -> np.ndarray:
        return self.ctx.get_values(node)

    def close(self):
        await_(self.ctx.dev)
        del self.rt
        self.ctx.free()


def routine_log_lines(stdout_text: str, log_id: int) -> List[str]:
    """The log of one run out of captured standard output: the lines that start with ``<log_id>: ``,
    prefix removed, ``$`` turned back into line ends (``Utils.log_debug_routine_logs``)."""
    prefix = f"{log_id}: "
    out: List[str] = []
    for chunk in stdout_text.split("$"):
        chunk = chunk.rsplit("\n", 1)[-1]   # (other output of the process may sit between two log lines)
        if chunk.startswith(prefix):
            out.append(chunk[len(prefix):])
    return out
