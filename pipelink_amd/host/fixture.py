"""Buffers a caller lends to the provider route.

The public names -- ``Resource``, ``Domain``, ``Fixture`` with ``tensor`` / ``readback``, and ``load_inputs`` --
are the ones a caller of the reference's ``pipec2.host.fixture`` module uses (pipec/src/pipec2/host/fixture.py:14-156);
what they promise is the contract below, and the code is written from it.

Contract.  An owner's provider is handed addresses and byte counts, nothing else.  Everything about a buffer's
life stays with the caller: a ``Fixture`` gets device memory from its backend, fills it (bytes the caller supplies,
or zeros), remembers which buffers the caller wants back after the launch, and returns all of it to the backend
when the ``with`` block ends -- last lent first, after the device has drained -- unless the backend reports that
it lost its device, in which case nothing is handed back for reuse."""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, NamedTuple


class Domain(NamedTuple):
    """Rank and size of a communication domain the caller names.  No owner built here declares one (one GPU);
    the type is part of the module's surface."""
    rank: int
    world: int


@dataclass
class Resource:
    """A device allocation on loan: where it is, how long it is, and where the tensor's origin sits in it."""
    address: int
    allocation_bytes: int
    origin_byte_offset: int = 0


@dataclass
class _Loan:
    name: str
    resource: Resource
    wanted_back: bool = field(default=False)


class Fixture:
    """The lender.  ``tensor`` lends one named buffer, ``readback`` fetches the ones marked as outputs (after the
    caller has synchronised), leaving the ``with`` block gives the memory back."""

    def __init__(self, backend: Any):
        self.backend = backend
        self.resources: dict[str, Resource] = {}   # by name, in lending order
        self.outputs: dict[str, bytes] = {}        # filled by readback()
        self._loans: list[_Loan] = []

    def tensor(self, name: str, *, data: bytes | None, allocation_bytes: int, alignment: int = 256, output: bool = False,
               origin_byte_offset: int = 0) -> Resource:
        """Lend ``allocation_bytes`` of device memory under ``name``: a copy of ``data`` (which must be exactly
        that long), or zeros when ``data`` is None.  The copy is synchronous, so the bytes are in place whatever
        stream the launch uses."""
        if name in self.resources:
            raise ValueError(f"{name!r} is already on loan from this fixture")
        if allocation_bytes < 0:
            raise ValueError(f"{name!r}: a negative allocation ({allocation_bytes} bytes)")
        if data is not None and len(data) != allocation_bytes:
            raise ValueError(f"{name!r}: {len(data)} bytes of data for an allocation of {allocation_bytes}")
        # the backend hands out at least one byte, so an empty tensor still has an address of its own
        address = self.backend.allocate(allocation_bytes or 1, alignment)
        loan = _Loan(name, Resource(address, allocation_bytes, origin_byte_offset), output)
        self._loans.append(loan)  # on the books before anything can fail: the exit path frees it
        if allocation_bytes:
            if data is None:
                self.backend.zero(address, allocation_bytes)
            else:
                self.backend.upload(address, data)
        self.resources[name] = loan.resource
        return loan.resource

    def readback(self) -> dict[str, bytes]:
        """Host copies of every output buffer, by name (also kept in ``outputs``)."""
        self.outputs.update((loan.name, self.backend.readback(loan.resource.address, loan.resource.allocation_bytes))
                            for loan in self._loans if loan.wanted_back)
        return self.outputs

    def __enter__(self) -> "Fixture":
        return self

    def __exit__(self, *_: Any) -> None:
        loans, self._loans = self._loans, []
        if getattr(self.backend, "lost", False):
            return  # the device is gone: its memory is not handed back for reuse
        self.backend.synchronize()
        while loans:
            self.backend.free(loans.pop().resource.address)


# keys of one resource record in a host-inputs file: required ones first
_REQUIRED = ("data", "allocation_bytes")
_OPTIONAL = ("alignment", "origin_byte_offset", "output",
             # tensor metadata the reference's records carry; the link states every channel's extents, so it is only accepted
             "extents", "bit_strides", "dtype_id", "origin_bit_offset")


def load_inputs(path: str | Path, fixture: Fixture) -> tuple[dict[str, Any], dict[str, Path]]:
    """Read the file ``pipec launch --host-inputs`` names and lend its buffers from ``fixture``.

    The file is one JSON object with two members: ``scalars`` (name -> number, passed on untouched) and ``resources``
    (name -> record).  A record has ``data`` (a file beside the JSON, or null for zeros) and ``allocation_bytes``,
    and may have ``alignment`` (default 256), ``origin_byte_offset`` (default 0), ``output`` (a file to write the
    buffer to after the launch) and tensor metadata.  Returns the scalars and {name: output path}."""
    path = Path(path)
    doc = json.loads(path.read_text())
    members = set(doc) if isinstance(doc, dict) else None
    if members != {"scalars", "resources"}:
        raise ValueError(f"{path.name}: expected an object with members 'scalars' and 'resources', found {sorted(members or [])}")
    scalars, records = doc["scalars"], doc["resources"]
    if not isinstance(scalars, dict):
        raise ValueError(f"{path.name}: 'scalars' is not an object")
    if not isinstance(records, dict):
        raise ValueError(f"{path.name}: 'resources' is not an object")
    write_to: dict[str, Path] = {}
    for name, record in records.items():
        if not isinstance(record, dict):
            raise ValueError(f"{path.name}: resource {name!r} is not an object")
        missing = [k for k in _REQUIRED if k not in record]
        unknown = sorted(set(record) - set(_REQUIRED) - set(_OPTIONAL))
        if missing or unknown:
            raise ValueError(f"{path.name}: resource {name!r} lacks {missing} / has unknown members {unknown}")
        source, target = record["data"], record.get("output")
        fixture.tensor(name,
                       data=(path.parent / source).read_bytes() if source is not None else None,
                       allocation_bytes=record["allocation_bytes"],
                       alignment=record.get("alignment", 256),
                       origin_byte_offset=record.get("origin_byte_offset", 0),
                       output=target is not None)
        if target is not None:
            write_to[name] = path.parent / target
    return scalars, write_to
