"""Caller-owned tensor loans for the provider route (the reference's ``pipec2.host.fixture``:
``Resource``, ``Domain``, ``Fixture``; pipec/src/pipec2/host/fixture.py:14-96).

A provider only ever sees addresses and sizes.  Who allocated a buffer, what was uploaded into it and when
its contents are read back stays on this side of the C seam: a ``Fixture`` owns fabricated buffers from
its backend until the host session that borrowed them has closed."""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, NamedTuple


class Domain(NamedTuple):
    """This rank's place in a caller-named communication domain.  The owners built here declare no
    domain (one GPU): the type exists so that a caller written against the reference's fixture
    module finds it."""
    rank: int
    world: int


@dataclass
class Resource:
    """One caller-owned device allocation lent to an owner for a session."""
    address: int
    allocation_bytes: int
    origin_byte_offset: int = 0


class Fixture:
    """Allocate, upload and later read back caller buffers on one backend; frees them on exit unless the
    backend was abandoned.  Inputs are uploaded synchronously at fabrication, so they are ready on whichever
    stream the caller launches on."""

    def __init__(self, backend: Any):
        self.backend = backend
        self.resources: dict[str, Resource] = {}
        self.outputs: dict[str, bytes] = {}
        self._outputs: list[str] = []
        self._allocations: list[int] = []

    def tensor(self, name: str, *, data: bytes | None, allocation_bytes: int, alignment: int = 256, output: bool = False,
               origin_byte_offset: int = 0) -> Resource:
        if name in self.resources:
            raise ValueError(f"duplicate fixture resource {name!r}")
        if allocation_bytes < 0 or (data is not None and len(data) != allocation_bytes):
            raise ValueError("fixture data must cover the declared allocation")
        address = self.backend.allocate(max(allocation_bytes, 1), alignment)
        self._allocations.append(address)
        if data:
            self.backend.upload(address, data)
        elif allocation_bytes:
            self.backend.zero(address, allocation_bytes)
        resource = Resource(address, allocation_bytes, origin_byte_offset)
        self.resources[name] = resource
        if output:
            self._outputs.append(name)
        return resource

    def readback(self) -> dict[str, bytes]:
        """Copy every output allocation to host memory; the caller synchronised first."""
        for name in self._outputs:
            resource = self.resources[name]
            self.outputs[name] = self.backend.readback(resource.address, resource.allocation_bytes)
        return self.outputs

    def __enter__(self) -> "Fixture":
        return self

    def __exit__(self, *_: Any) -> None:
        if not getattr(self.backend, "lost", False):
            self.backend.synchronize()
            for address in reversed(self._allocations):
                self.backend.free(address)
        self._allocations.clear()


def load_inputs(path: str | Path, fixture: Fixture) -> tuple[dict[str, Any], dict[str, Path]]:
    """Caller scalars and buffers for ``pipec launch --host-inputs`` (the reference's ``load_inputs``,
    host/fixture.py:122-156): ``{"scalars": {...}, "resources": {name: {"data": FILE | null, "allocation_bytes": n,
    ["alignment": a,] ["origin_byte_offset": o,] ["output": FILE]}}}``, paths relative to the JSON.  A resource
    without data is zeroed; one that names an output file is read back after the launch.  The tensor metadata the
    reference's records carry besides (extents, strides, dtype) is accepted and not needed: the link states every
    channel's extents.  Returns (scalars, {name: output path})."""
    path = Path(path)
    obj = json.loads(path.read_text())
    if not isinstance(obj, dict) or set(obj) != {"scalars", "resources"}:
        raise ValueError("host inputs require exactly scalars and resources objects")
    if not isinstance(obj["scalars"], dict) or not isinstance(obj["resources"], dict):
        raise ValueError("host scalars/resources must be objects")
    known = {"data", "allocation_bytes", "extents", "bit_strides", "dtype_id", "alignment", "origin_byte_offset",
             "origin_bit_offset", "output"}
    outputs: dict[str, Path] = {}
    for name, item in obj["resources"].items():
        if not isinstance(item, dict) or not {"data", "allocation_bytes"} <= set(item) or set(item) - known:
            raise ValueError(f"invalid fixture declaration for {name}")
        data = None if item["data"] is None else (path.parent / item["data"]).read_bytes()
        fixture.tensor(name, data=data, allocation_bytes=item["allocation_bytes"], alignment=item.get("alignment", 256),
                       origin_byte_offset=item.get("origin_byte_offset", 0), output=item.get("output") is not None)
        if item.get("output") is not None:
            outputs[name] = path.parent / item["output"]
    return obj["scalars"], outputs
