"""Caller-owned tensor loans for the provider route (the reference's ``pipec2.host.fixture``:
``Resource``, ``Domain``, ``Fixture``; pipec/src/pipec2/host/fixture.py:14-96).

A provider only ever sees addresses and sizes.  Who allocated a buffer, what was uploaded into it and when
its contents are read back stays on this side of the C seam: a ``Fixture`` owns fabricated buffers from
its backend until the host session that borrowed them has closed."""
from __future__ import annotations

from dataclasses import dataclass
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
