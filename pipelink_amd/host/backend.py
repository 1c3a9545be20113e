"""ctypes binding of the C-ABI launch layer (``include/plk_hip.h``).

``HipBackend`` offers the method set of the reference's ``CudaBackend``
(pipec/src/pipec2/host/cuda.py:118-265): allocate / free / zero / upload / readback /
synchronize / event_* / launch, so session code written against that class carries over.
There is no CPU fallback: a missing library or a failing HIP call raises ``PlkError``.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, byref, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint32, c_uint64, c_void_p

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG, "libplk_hip.so")

STATUS_NAMES = {0: "PLK_OK", 1: "PLK_E_VERSION", 2: "PLK_E_CAPACITY", 3: "PLK_E_ARGUMENT", 4: "PLK_E_CONTRACT",
                5: "PLK_E_RESOURCE", 6: "PLK_E_BUILD", 7: "PLK_E_RELEASE"}


class PlkError(RuntimeError):
    def __init__(self, status: int, message: str):
        self.status = status
        super().__init__(f"{STATUS_NAMES.get(status, status)}: {message}")


class DeviceInfo(ctypes.Structure):
    _fields_ = [("compute_units", c_int32), ("wavefront_size", c_int32), ("max_lds_per_workgroup", c_int32),
                ("max_threads_per_workgroup", c_int32), ("clock_khz", c_int32), ("memory_clock_khz", c_int32),
                ("l2_bytes", c_int32), ("reserved", c_int32), ("total_memory", c_int64), ("arch", ctypes.c_char * 64)]


class MokLinkInfo(ctypes.Structure):
    _fields_ = [(n, c_uint32) for n in ("struct_bytes", "params_bytes", "framework_offset", "gemm_offset",
                                        "act_offset", "threads", "dyn_lds_bytes", "workgroups_per_cu")]


class MokProblem(ctypes.Structure):
    _fields_ = [("struct_bytes", c_uint32), ("num_tokens", c_int32), ("hidden", c_int32), ("intermediate", c_int32),
                ("num_experts", c_int32), ("routed_rows", c_int32), ("ld_sc_h", c_int32), ("ld_sc_i", c_int32),
                ("ld_q_h", c_int32), ("ld_q_i", c_int32), ("swiglu_limit", c_float), ("reserved", c_int32)] + \
               [(n, c_uint64) for n in ("x_q", "x_sc", "row_token", "tokens_per_expert", "w_gate_q", "w_gate_sc",
                                        "w_up_q", "w_up_sc", "w_down_q", "w_down_sc", "hidden_q", "hidden_sc", "y")]


# every entry point include/plk_hip.h and include/plk_mok.h declare: (restype, argtypes)
SIGNATURES = {
    "plk_hip_last_error": (c_char_p, []),
    "plk_hip_device_count": (c_int, [POINTER(c_int32)]),
    "plk_hip_set_device": (c_int, [c_int32]),
    "plk_hip_device_info_get": (c_int, [c_int32, POINTER(DeviceInfo)]),
    "plk_hip_alloc": (c_int, [c_size_t, POINTER(c_uint64)]),
    "plk_hip_free": (c_int, [c_uint64]),
    "plk_hip_zero": (c_int, [c_uint64, c_size_t, c_void_p]),
    "plk_hip_fill_u8": (c_int, [c_uint64, c_int, c_size_t, c_void_p]),
    "plk_hip_upload": (c_int, [c_uint64, c_void_p, c_size_t, c_void_p]),
    "plk_hip_readback": (c_int, [c_void_p, c_uint64, c_size_t, c_void_p]),
    "plk_hip_synchronize": (c_int, [c_void_p]),
    "plk_hip_stream_create": (c_int, [POINTER(c_void_p)]),
    "plk_hip_stream_destroy": (c_int, [c_void_p]),
    "plk_hip_graph_begin": (c_int, [c_void_p]),
    "plk_hip_graph_end": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p)]),
    "plk_hip_graph_abort": (c_int, [c_void_p]),
    "plk_hip_graph_launch": (c_int, [c_void_p, c_void_p]),
    "plk_hip_graph_destroy": (c_int, [c_void_p, c_void_p]),
    "plk_hip_event_create": (c_int, [POINTER(c_void_p)]),
    "plk_hip_event_record": (c_int, [c_void_p, c_void_p]),
    "plk_hip_event_synchronize": (c_int, [c_void_p]),
    "plk_hip_event_elapsed_ms": (c_int, [c_void_p, c_void_p, POINTER(c_float)]),
    "plk_hip_event_destroy": (c_int, [c_void_p]),
    "plk_hip_module_load": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "plk_hip_module_unload": (c_int, [c_void_p]),
    "plk_hip_module_function": (c_int, [c_void_p, c_char_p, c_uint32, POINTER(c_void_p)]),
    "plk_hip_launch": (c_int, [c_void_p, POINTER(c_uint32 * 3), POINTER(c_uint32 * 3), c_uint32, c_void_p, c_uint64]),
    "plk_mok_session_create": (c_int, [c_void_p, c_size_t, POINTER(MokLinkInfo), POINTER(c_void_p)]),
    "plk_mok_session_destroy": (c_int, [c_void_p]),
    "plk_mok_forward": (c_int, [c_void_p, POINTER(MokProblem), c_void_p]),
    "plk_mok_forward_pass": (c_int, [c_void_p, POINTER(MokProblem), c_int, c_void_p]),
    "plk_mok_forward_static": (c_int, [c_void_p, POINTER(MokProblem), c_void_p]),
    "plk_mok_status": (c_int, [c_void_p, c_void_p, POINTER(ctypes.c_uint32)]),
    "plk_mok_session_launches": (c_int, [c_void_p, c_int]),
    "plk_mxfp8_scales_to_slot_major": (c_int, [c_uint64, c_int64, c_int32, c_int32, c_uint64, c_void_p]),
    "plk_mxfp8_codes_to_k64_tiled": (c_int, [c_uint64, c_int64, c_int32, c_int64, c_uint64, c_void_p]),
    "plk_mxfp8_quantize": (c_int, [c_uint64, c_int, c_int64, c_int32, c_uint64, c_int32, c_uint64, c_int32, c_void_p]),
}

_lib = None


def load_library(path: str | None = None) -> ctypes.CDLL:
    """Load ``libplk_hip.so`` (built in-tree by ``__graft_entry__.build()``); raises if absent."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise PlkError(6, f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = the library does not export what the headers declare
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(lib, status: int) -> None:
    if status != 0:
        raise PlkError(status, (lib.plk_hip_last_error() or b"").decode("utf-8", "replace"))


class _Current:
    """What HipBackend.current() returns: the device is already current; usable as ``with backend.current():``."""

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


class Graph:
    """An instantiated graph replaying exactly the work captured on one stream (host/cuda.py:358-388 in the reference)."""

    def __init__(self, backend: "HipBackend", graph: int, executable: int):
        self._backend, self._graph, self.executable, self.closed = backend, graph, executable, False

    def launch(self, stream: int | None = None) -> None:
        check(self._backend.lib, self._backend.lib.plk_hip_graph_launch(self.executable, self._backend._s(stream)))

    def close(self) -> None:
        if self.closed:
            return
        self.closed = True
        self._backend._graphs.remove(self)
        if not self._backend.lost:
            check(self._backend.lib, self._backend.lib.plk_hip_graph_destroy(self._graph, self.executable))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


class HipBackend:
    """Device memory, events, launches and graph capture on one GPU; ``stream`` is a raw ``hipStream_t`` (0 = default).

    The method set is the reference's ``CudaBackend`` (host/cuda.py:118-356): allocate / free / zero / upload /
    readback / synchronize / event_* / launch / capture / current / abandon / close, ``stream_token``,
    ``observations``."""

    def __init__(self, device: int = 0, stream: int = 0):
        self.lib = load_library()
        self.device = device
        self.stream_token = stream
        self.lost = self.closed = False
        check(self.lib, self.lib.plk_hip_set_device(device))
        self._allocations: set[int] = set()
        self._graphs: list[Graph] = []
        self._streams: list[int] = []
        info = self.info()
        self.observations: dict = {"device_ordinal": device, "arch": info.arch.decode().split(":")[0],
                                   "observed_cu_count": info.compute_units, "wavefront_size": info.wavefront_size,
                                   "max_lds_per_workgroup": info.max_lds_per_workgroup,
                                   "max_threads": info.max_threads_per_workgroup, "l2_bytes": info.l2_bytes,
                                   "total_memory": info.total_memory}

    # -- CudaBackend.current(): one device, one context -- making it current is setting the device
    def current(self) -> _Current:
        check(self.lib, self.lib.plk_hip_set_device(self.device))
        return _Current()

    def stream_create(self) -> int:
        """A stream of default priority that close() destroys (graph capture needs one: stream 0 cannot be captured)."""
        s = c_void_p()
        check(self.lib, self.lib.plk_hip_stream_create(byref(s)))
        self._streams.append(s.value)
        return s.value

    def capture(self, stream: int, body) -> Graph:
        """Record what ``body()`` enqueues on ``stream`` and instantiate it.  Fills issued in the body are recorded as
        kernels; an upload or a readback in the body fails the capture."""
        check(self.lib, self.lib.plk_hip_graph_begin(c_void_p(stream)))
        try:
            body()
        except BaseException:
            self.lib.plk_hip_graph_abort(c_void_p(stream))
            raise
        graph, executable = c_void_p(), c_void_p()
        check(self.lib, self.lib.plk_hip_graph_end(c_void_p(stream), byref(graph), byref(executable)))
        result = Graph(self, graph.value, executable.value)
        self._graphs.append(result)
        return result

    def abandon(self) -> None:
        """After a failed synchronisation: nothing this backend allocated is reused or freed."""
        self.lost = True

    def info(self) -> DeviceInfo:
        out = DeviceInfo()
        check(self.lib, self.lib.plk_hip_device_info_get(self.device, byref(out)))
        return out

    def allocate(self, size: int, align: int = 256) -> int:
        if align > 256 or align & (align - 1):
            raise PlkError(3, f"alignment {align} is not a power of two <= 256")
        addr = c_uint64()
        check(self.lib, self.lib.plk_hip_alloc(size, byref(addr)))
        self._allocations.add(addr.value)
        return addr.value

    def free(self, addr: int) -> None:
        self._allocations.discard(addr)
        check(self.lib, self.lib.plk_hip_free(addr))

    def zero(self, addr: int, size: int, stream: int | None = None) -> None:
        check(self.lib, self.lib.plk_hip_zero(addr, size, self._s(stream)))

    def fill(self, addr: int, value: int, size: int, stream: int | None = None) -> None:
        check(self.lib, self.lib.plk_hip_fill_u8(addr, value, size, self._s(stream)))

    def upload(self, addr: int, data: bytes | bytearray | memoryview, stream: int | None = None) -> None:
        buf = (ctypes.c_char * len(data)).from_buffer_copy(data)
        check(self.lib, self.lib.plk_hip_upload(addr, buf, len(data), self._s(stream)))

    def readback(self, addr: int, size: int, stream: int | None = None) -> bytes:
        buf = ctypes.create_string_buffer(size)
        check(self.lib, self.lib.plk_hip_readback(buf, addr, size, self._s(stream)))
        return buf.raw

    def synchronize(self, stream: int | None = None) -> None:
        check(self.lib, self.lib.plk_hip_synchronize(self._s(stream)))

    def event_create(self) -> int:
        ev = c_void_p()
        check(self.lib, self.lib.plk_hip_event_create(byref(ev)))
        return ev.value

    def event_record(self, event: int, stream: int | None = None) -> None:
        check(self.lib, self.lib.plk_hip_event_record(event, self._s(stream)))

    def event_synchronize(self, event: int) -> None:
        check(self.lib, self.lib.plk_hip_event_synchronize(event))

    def event_elapsed_time(self, start: int, stop: int) -> float:
        ms = c_float()
        check(self.lib, self.lib.plk_hip_event_elapsed_ms(start, stop, byref(ms)))
        return ms.value

    def event_destroy(self, event: int) -> None:
        check(self.lib, self.lib.plk_hip_event_destroy(event))

    def module_load(self, image: bytes) -> int:
        mod = c_void_p()
        buf = ctypes.create_string_buffer(image, len(image))
        check(self.lib, self.lib.plk_hip_module_load(buf, len(image), byref(mod)))
        return mod.value

    def module_unload(self, module: int) -> None:
        check(self.lib, self.lib.plk_hip_module_unload(module))

    def module_function(self, module: int, name: str, dyn_lds_bytes: int = 0) -> int:
        fn = c_void_p()
        check(self.lib, self.lib.plk_hip_module_function(module, name.encode(), dyn_lds_bytes, byref(fn)))
        return fn.value

    def launch(self, function: int, params_addr: int, grid, block, dyn_lds_bytes: int, stream: int | None = None):
        """One launch; the kernel's only argument is the address of its params image."""
        g = (c_uint32 * 3)(*grid)
        b = (c_uint32 * 3)(*block)
        check(self.lib, self.lib.plk_hip_launch(function, byref(g), byref(b), dyn_lds_bytes, self._s(stream), params_addr))

    def close(self) -> None:
        if self.closed:
            return
        self.closed = True
        for graph in list(self._graphs):
            graph.close()
        if not self.lost:
            for addr in sorted(self._allocations):
                self.lib.plk_hip_free(addr)
            for stream in self._streams:
                self.lib.plk_hip_stream_destroy(c_void_p(stream))
        self._allocations.clear()
        self._streams.clear()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _s(self, stream):
        return c_void_p(self.stream_token if stream is None else stream)
