"""Named diagnostics.  Every rejection anywhere in pack / link / launch is a list of
``ClauseFailure(clause_id, path, message, detail)`` carried by a ``PipeLinkError``; the CLI
prints them as ``pipec: [ID] path: message; [ID] ...``.

Same registry, ids, phases and message format as pipec/src/pipec2/model.py:44-93,226-252
(the contract-gallery checker of the reference greps that exact prefix,
examples/contract-gallery/check.py:24-25)."""
from __future__ import annotations

import re
from dataclasses import dataclass, field
from typing import Any

PHASES = ("load", "pack", "layout", "protocol", "solve", "link", "launch")
_ID = re.compile(r"[A-Z][A-Z0-9]*(?:-[A-Z0-9]+)*\Z")

CLAUSES: dict[str, str] = {}        # id -> description
CLAUSE_PHASES: dict[str, str] = {}  # id -> primary phase


def register_clause(clause_id: str, *, phase: str, description: str = "") -> None:
    if not isinstance(clause_id, str) or not _ID.match(clause_id):
        raise ValueError(f"invalid clause ID {clause_id!r}")
    if phase not in PHASES:
        raise ValueError(f"unknown clause phase {phase!r}")
    if clause_id in CLAUSES:
        raise ValueError(f"duplicate clause ID {clause_id!r}")
    CLAUSES[clause_id] = description
    CLAUSE_PHASES[clause_id] = phase


_CORE = """
L-ALIGN solve claim bindings satisfy native and physical alignment
L-BUDGET solve solver finds a feasible layout within its deterministic work limit
L8 layout paired endpoints have equal canonical physical layout identity
L-ENTRYABI load stage entry ABI is supported by the live linker
L-HANDLE load handle declarations and references are complete and consistent
L-HOSTCHAN link host declarations and selected resource contracts agree
L-HOSTABI launch native host provider ABI agrees with the declared inventory
L-LINK link artifact linking and dispatch generation complete successfully
L-OVERLAP solve physical intervals do not overlap without valid alias or lifetime exclusion
L-OWNER solve every allocation handle has exactly one owning claim
L-PAIR link each channel has one compatible producer and consumer
L-PARAMS link stage and aggregate parameter layouts satisfy the target ABI
L-PHASE solve claim phases and pairwise exclusions are finite and valid
L-PROTO protocol paired endpoint protocols expand consistently
L-REGS solve register groups and the register pool are legal
L-SYM link artifact symbols and normalized prefixes are unique
L-TOPO solve stage topology constraints have a legal intersection
L-STUB link generated binding stubs and trampolines are well formed
L-LAUNCH launch launch geometry, buffers and params blobs match the link result
P-IMPORT pack artifact imports are declared PipeLink symbols
P-CONTAINER pack artifact containers and payload declarations are readable and well formed
P-COMPILE pack stage sources compile for the target and emit a registry
P-SYM pack stage symbols carry the normalised stage prefix
P-INIT pack counter rings name an initialising role
T-CONTRACT load tensor contracts and explicit connection references are valid
"""
for _line in _CORE.strip().splitlines():
    _cid, _phase, _desc = _line.split(" ", 2)
    register_clause(_cid, phase=_phase, description=_desc)


@dataclass(frozen=True)
class ClauseFailure:
    clause_id: str
    path: str
    message: str
    detail: dict[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        if self.clause_id not in CLAUSES:
            raise ValueError(f"unknown clause ID {self.clause_id!r}")

    def to_json_obj(self) -> dict[str, Any]:
        return {"clause_id": self.clause_id, "path": self.path, "message": self.message, "detail": self.detail}


class PipeLinkError(RuntimeError):
    """Deterministic failure of one phase; ``failures`` is sorted by (clause_id, path)."""

    def __init__(self, failures: list[ClauseFailure]):
        self.failures = sorted(failures, key=lambda f: (f.clause_id, f.path))
        super().__init__("; ".join(f"[{f.clause_id}] {f.path}: {f.message}" for f in self.failures)
                         or type(self).__name__)

    @property
    def clause_ids(self) -> set[str]:
        return {f.clause_id for f in self.failures}


class SchemaError(PipeLinkError):
    pass


class PackError(PipeLinkError):
    pass


class SolveError(PipeLinkError):
    pass


class LinkError(PipeLinkError):
    pass


class LaunchError(PipeLinkError):
    pass


def reject(kind: type[PipeLinkError], clause_id: str, path: str, message: str, **detail: Any):
    raise kind([ClauseFailure(clause_id, path, message, detail)])
