"""Host-less launch of a linked pipeline: no provider libraries, the caller supplies buffers and
a function that turns their device addresses into per-stage params blobs.

Mirrors pipec/src/pipec2/launcher.py:107-333 of the reference: ``open_hostless`` allocates and
uploads (arrays) or zeroes (shape/dtype specs) every buffer *before* ``params(addresses)`` runs,
checks that the returned blobs cover exactly the non-empty entries of ``link.json``'s
``params.entries`` (else ``L-PARAMS`` at ``launch.params``), copies them to their linked offsets
and returns a ``HostlessSession`` with ``launch / synchronize / read / write / time / with_image /
close``.  ``with_image`` loads a second code object that shares buffers, params and stream --
the linked-versus-one-unit A/B switch.  The backend is anything with the ``HipBackend`` method
set, so the CPU tests drive it with an in-memory fake."""
from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Callable

import numpy as np

from .clauses import ClauseFailure, LaunchError


def _fail(clause: str, path: str, message: str, **detail: Any):
    raise LaunchError([ClauseFailure(clause, path, message, detail)])


class HostlessSession:
    def __init__(self, backend, link: dict[str, Any], function: int, module: int, buffers: dict[str, tuple[int, int, Any]],
                 params_addr: int, grid: tuple[int, int, int], owns: bool = True):
        self.backend, self.link, self._fn, self._module = backend, link, function, module
        self.buffers, self.params_addr, self.grid, self._owns = buffers, params_addr, grid, owns
        self._children: list[HostlessSession] = []

    def launch(self) -> None:
        self.backend.launch(self._fn, self.params_addr, self.grid, (self.link["threads"], 1, 1), self.link["dyn_smem_bytes"])

    def synchronize(self) -> None:
        self.backend.synchronize()

    def read(self, name: str) -> np.ndarray:
        addr, size, spec = self.buffers[name]
        shape, dtype = spec
        return np.frombuffer(self.backend.readback(addr, size), dtype=dtype).reshape(shape).copy()

    def write(self, name: str, array: np.ndarray) -> None:
        addr, size, spec = self.buffers[name]
        data = np.ascontiguousarray(array, dtype=spec[1])
        if data.nbytes != size:
            _fail("L-LAUNCH", f"launch.buffers.{name}", "array size differs from the buffer's")
        self.backend.upload(addr, data.tobytes())

    def time(self, n: int) -> float:
        """Milliseconds per launch over n back-to-back launches (one event pair)."""
        if n <= 0:
            _fail("L-LAUNCH", "launch.time", "launch count must be positive")
        e0, e1 = self.backend.event_create(), self.backend.event_create()
        self.backend.event_record(e0)
        for _ in range(n):
            self.launch()
        self.backend.event_record(e1)
        self.backend.event_synchronize(e1)
        ms = self.backend.event_elapsed_time(e0, e1) / n
        self.backend.event_destroy(e0)
        self.backend.event_destroy(e1)
        if not (ms > 0 and np.isfinite(ms)):
            _fail("L-LAUNCH", "launch.time", "measured time is not finite and positive")
        return ms

    def with_image(self, image_path: str | Path) -> "HostlessSession":
        module = self.backend.module_load(Path(image_path).read_bytes())
        fn = self.backend.module_function(module, self.link["kernel_symbol"], self.link["dyn_smem_bytes"])
        child = HostlessSession(self.backend, self.link, fn, module, self.buffers, self.params_addr, self.grid, owns=False)
        self._children.append(child)
        return child

    def close(self) -> None:
        for c in self._children:
            c.close()
        self._children.clear()
        self.backend.module_unload(self._module)
        if self._owns:
            for addr, _, _ in self.buffers.values():
                self.backend.free(addr)
            self.backend.free(self.params_addr)


def open_hostless(link_json: str | Path | dict, *, buffers: dict[str, Any], params: Callable[[dict[str, int]], dict[str, bytes]],
                  grid: tuple[int, ...], backend=None, image: str | Path | None = None, device: int = 0) -> HostlessSession:
    if isinstance(link_json, dict):
        link, base = link_json, Path(".")
    else:
        link, base = json.loads(Path(link_json).read_text()), Path(link_json).parent
    if link.get("host"):
        _fail("L-LAUNCH", "launch.host", "link carries a host section: open it through its providers")
    if backend is None:
        from ..host.backend import HipBackend
        backend = HipBackend(device)
    backend.current()
    placed: dict[str, tuple[int, int, Any]] = {}
    owned: list[int] = []   # device allocations of this call: given back if the session cannot be opened
    try:
        return _open_placed(link, base, buffers, params, grid, backend, image, placed, owned)
    except BaseException:
        for addr in owned:
            backend.free(addr)
        raise


def _open_placed(link, base, buffers, params, grid, backend, image, placed, owned) -> HostlessSession:
    for name, spec in buffers.items():
        if isinstance(spec, np.ndarray):
            data = np.ascontiguousarray(spec)
            addr = backend.allocate(max(data.nbytes, 1))
            owned.append(addr)
            backend.upload(addr, data.tobytes())
            placed[name] = (addr, data.nbytes, (data.shape, data.dtype))
        else:
            shape, dtype = spec
            size = int(np.prod(shape)) * np.dtype(dtype).itemsize
            addr = backend.allocate(max(size, 1))
            owned.append(addr)
            backend.zero(addr, size)
            placed[name] = (addr, size, (tuple(shape), np.dtype(dtype)))
    backend.synchronize()
    blobs = params({n: a for n, (a, _, _) in placed.items()})
    entries = {e["stage_id"]: e for e in link["params"]["entries"] if e["bytes"]}
    if set(blobs) != set(entries):
        _fail("L-PARAMS", "launch.params", "params blobs do not cover exactly the linked params entries",
              expected=sorted(entries), actual=sorted(blobs))
    image_bytes = bytearray(max(link["params"]["total_bytes"], 16))
    for sid, blob in blobs.items():
        e = entries[sid]
        if len(blob) != e["bytes"]:
            _fail("L-PARAMS", f"launch.params.{sid}", "params blob size differs from the packed layout",
                  expected=e["bytes"], actual=len(blob))
        image_bytes[e["offset"]:e["offset"] + e["bytes"]] = blob
    params_addr = backend.allocate(len(image_bytes))
    owned.append(params_addr)
    backend.upload(params_addr, bytes(image_bytes))
    path = Path(image) if image else base / link["target"]["image"]
    module = backend.module_load(path.read_bytes())
    fn = backend.module_function(module, link["kernel_symbol"], link["dyn_smem_bytes"])
    g = tuple(grid) + (1,) * (3 - len(grid))
    return HostlessSession(backend, link, fn, module, placed, params_addr, g)


def run_hostless(link_json, *, buffers, params, grid, outputs: list[str], **kw) -> dict[str, np.ndarray]:
    s = open_hostless(link_json, buffers=buffers, params=params, grid=grid, **kw)
    try:
        s.launch()
        s.synchronize()
        return {n: s.read(n) for n in outputs}
    finally:
        s.close()


def _parse_buffer(spec: str):
    """``FILE.npy`` or ``SHAPE:DTYPE`` (e.g. ``64x64:float32``, a zeroed buffer)."""
    if spec.endswith(".npy"):
        return np.load(spec, allow_pickle=False)
    shape, _, dtype = spec.partition(":")
    try:
        return tuple(int(d) for d in shape.split("x")), np.dtype(dtype)
    except (ValueError, TypeError):
        _fail("L-LAUNCH", "launch.buffers", "buffer spec must be FILE.npy or SHAPE:DTYPE", spec=spec)


def _load_params_function(spec: str) -> Callable[[dict[str, int]], dict[str, bytes]]:
    """``PY_FILE:FUNCTION`` -> the function (the file is executed as a module of its own)."""
    import importlib.util

    path, _, name = spec.rpartition(":")
    if not path or not name:
        _fail("L-LAUNCH", "launch.params", "params builder must be PY_FILE:FUNCTION", spec=spec)
    module_spec = importlib.util.spec_from_file_location("pipec_launch_params", path)
    if module_spec is None or module_spec.loader is None:
        _fail("L-LAUNCH", "launch.params", "params builder file cannot be loaded", path=path)
    module = importlib.util.module_from_spec(module_spec)
    module_spec.loader.exec_module(module)
    if not callable(getattr(module, name, None)):
        _fail("L-LAUNCH", "launch.params", "params builder function not found", function=name)
    return getattr(module, name)


def launch(link_json: str | Path, *, grid: tuple[int, ...] | None, buffers: dict[str, str] | None = None,
           params: str | None = None, blobs: dict[str, str | Path] | None = None, outputs: dict[str, str | Path] | None = None,
           providers: dict[str, str] | None = None, host_inputs: str | Path | None = None, device: int = 0,
           backend=None) -> dict[str, Any]:
    """One launch, as ``pipec launch`` runs it (pipec/src/pipec2/launcher.py:284-333 in the reference).  A link with
    a host section goes through its providers (``providers`` = params group -> shared library, ``host_inputs`` = the
    caller's scalars and buffers, see ``host.fixture.load_inputs``).  Any other link takes the host-less route: buffers from ``NAME -> FILE.npy | SHAPE:DTYPE``, params either from a Python
    builder ``PY_FILE:FUNCTION`` (device addresses -> stage bytes) or from ready-made blobs
    ``STAGE_ID -> file``; named buffers are saved as .npy afterwards.  Returns the report the CLI prints."""
    link_obj = json.loads(Path(link_json).read_text())
    if link_obj.get("host") or providers or host_inputs:
        return _launch_host(Path(link_json), link_obj, providers or {}, host_inputs, device, backend, grid, buffers, params, blobs)
    if grid is None:
        _fail("L-LAUNCH", "launch.grid", "host-less launch requires a grid")
    if params is not None and blobs:
        _fail("L-LAUNCH", "launch.params", "params builder and blob paths are mutually exclusive")
    builder = _load_params_function(params) if params is not None else (
        lambda addresses: {sid: Path(path).read_bytes() for sid, path in (blobs or {}).items()})
    parsed = {name: _parse_buffer(spec) for name, spec in (buffers or {}).items()}
    unknown = sorted(set(outputs or {}) - set(parsed))
    if unknown:
        _fail("L-LAUNCH", "launch.outputs", "output names a buffer that was not declared", names=unknown)
    result = run_hostless(link_json, buffers=parsed, params=builder, grid=tuple(grid), outputs=list(outputs or {}),
                          backend=backend, device=device)
    for name, path in (outputs or {}).items():
        with Path(path).open("wb") as stream:
            np.save(stream, result[name], allow_pickle=False)
    link = json.loads(Path(link_json).read_text())
    g = tuple(grid) + (1,) * (3 - len(grid))
    return {"geometry": {"grid": list(g), "block": [link["threads"], 1, 1], "dynamic_smem_bytes": link["dyn_smem_bytes"]},
            "outputs": {name: str(path) for name, path in (outputs or {}).items()}}


def _launch_host(link_path: Path, link: dict[str, Any], providers: dict[str, str], host_inputs, device: int, backend, grid,
                 buffers, params, blobs) -> dict[str, Any]:
    """The provider route of ``pipec launch``: report / query / build through the named libraries, one launch, outputs
    written as raw bytes to the files the inputs name."""
    import ctypes

    from ..host import broker
    from ..host.backend import HipBackend, PlkError
    from ..host.fixture import Fixture, load_inputs

    if not link.get("host"):
        _fail("L-LAUNCH", "launch.providers", "this link has no host section: it takes --grid / --buffer / --params")
    if grid is not None or buffers or params is not None or blobs:
        _fail("L-LAUNCH", "launch.host", "a link with a host section takes --provider and --host-inputs only")
    if host_inputs is None:
        _fail("L-LAUNCH", "launch.host_inputs", "a link with a host section needs --host-inputs")
    groups = link["host"]["groups"]
    expected = sorted(g["params_group"] for g in groups)
    if sorted(providers) != expected:
        _fail("L-HOSTABI", "launch.providers", "provider maps must exactly resolve params groups", expected=expected,
              actual=sorted(providers))
    image = (link_path.parent / link["target"]["image"]).read_bytes()
    libs = {}
    for group, so in providers.items():
        try:
            libs[group] = ctypes.CDLL(str(so))
        except OSError as err:
            _fail("L-HOSTABI", f"launch.providers.{group}", f"cannot load provider: {err}")
    be = backend or HipBackend(device)
    try:
        with Fixture(be) as fixture:
            scalars, output_paths = load_inputs(host_inputs, fixture)
            resources = {g["owner"]: {c["name"]: fixture.resources[c["name"]] for c in g["channels"] if c["name"] in fixture.resources}
                         for g in groups}
            try:
                with broker.open_host(link, image, resources, scalars, be, providers=libs) as session:
                    session.launch()
                    be.synchronize()
                    geometry = session.geometry
            except PlkError as err:
                _fail("L-HOSTABI", "launch.host", str(err))
            for name, data in fixture.readback().items():
                output_paths[name].write_bytes(data)
    finally:
        if backend is None:
            be.close()
    return {"geometry": {"grid": list(geometry["grid"]), "block": list(geometry["block"]), "dynamic_smem_bytes": geometry["dyn_lds"]},
            "outputs": {name: str(path) for name, path in output_paths.items()}}
