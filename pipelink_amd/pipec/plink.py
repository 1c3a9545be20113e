"""The ``.plink`` package: canonical JSON manifest + one payload member.

Byte-compatible with the reference's container (pipec/src/pipec2/container.py:14-18,31-62,
canonjson.py:8-11): a ZIP with exactly ``manifest.json`` then ``stage.o``, DEFLATE level 9,
timestamp 1980-01-01 00:00:00, create_system 3, external_attr 0o600 << 16, no extra fields or
comments; the manifest is JSON with sorted keys, ``(",", ":")`` separators, no NaN, one
trailing line feed, and carries ``payload = {"file": "stage.o", "sha256": ...}`` computed
here (a source-supplied digest is refused).  On gfx950 the payload is AMDGPU LLVM bitcode."""
from __future__ import annotations

import copy
import hashlib
import io
import json
import zipfile
from pathlib import Path
from typing import Any

from .clauses import PackError, reject

MEMBERS = ("manifest.json", "stage.o")
_EPOCH = (1980, 1, 1, 0, 0, 0)


def canonical_dumps(obj: Any) -> str:
    return json.dumps(obj, sort_keys=True, separators=(",", ":"), allow_nan=False) + "\n"


def canonical_bytes(obj: Any) -> bytes:
    return canonical_dumps(obj).encode("utf-8")


def sha256_hex(data: bytes) -> str:
    return hashlib.sha256(data).hexdigest()


def _zip_bytes(parts: list[tuple[str, bytes]]) -> bytes:
    buf = io.BytesIO()
    with zipfile.ZipFile(buf, "w", compression=zipfile.ZIP_DEFLATED, compresslevel=9) as zf:
        zf.comment = b""
        for name, data in parts:
            info = zipfile.ZipInfo(name, date_time=_EPOCH)
            info.compress_type = zipfile.ZIP_DEFLATED
            info.create_system = 3
            info.external_attr = 0o600 << 16
            info.internal_attr = 0
            info.flag_bits = 0
            info.extra = b""
            info.comment = b""
            zf.writestr(info, data, compresslevel=9)
    return buf.getvalue()


def pack(manifest: dict[str, Any], payload: bytes, out: str | Path) -> dict[str, Any]:
    """Write the container; returns its digests (artifact, manifest, payload)."""
    if not isinstance(manifest, dict):
        reject(PackError, "P-CONTAINER", "$", "manifest root must be an object")
    if not isinstance(payload, (bytes, bytearray)):
        reject(PackError, "P-CONTAINER", "stage.o", "object payload must be bytes")
    m = copy.deepcopy(manifest)
    decl = m.get("payload")
    if not isinstance(decl, dict):
        reject(PackError, "P-CONTAINER", "$.payload", "source manifest payload must be an object")
    extra = sorted(set(decl) - {"file", "sha256"})
    if extra:
        reject(PackError, "P-CONTAINER", f"$.payload.{extra[0]}", "unknown payload field")
    if decl.get("file") != MEMBERS[1]:
        reject(PackError, "P-CONTAINER", "$.payload.file", "payload file must be 'stage.o'")
    if "sha256" in decl:
        reject(PackError, "P-CONTAINER", "$.payload.sha256",
               "source-supplied payload digest is forbidden; pack computes it")
    decl["sha256"] = sha256_hex(bytes(payload))
    try:
        mbytes = canonical_bytes(m)
    except (TypeError, ValueError) as exc:
        reject(PackError, "P-CONTAINER", "$", f"cannot encode canonical artifact: {exc}")
    blob = _zip_bytes([(MEMBERS[0], mbytes), (MEMBERS[1], bytes(payload))])
    try:
        Path(out).write_bytes(blob)
    except OSError as exc:
        reject(PackError, "P-CONTAINER", str(out), f"cannot write artifact: {exc}")
    return {"artifact_sha256": sha256_hex(blob), "manifest_sha256": sha256_hex(mbytes),
            "payload": {"file": MEMBERS[1], "sha256": decl["sha256"], "size": len(payload)}}


def read(path: str | Path) -> tuple[dict[str, Any], bytes]:
    """Return (manifest, payload bytes); checks that the payload matches its recorded digest."""
    try:
        with zipfile.ZipFile(Path(path)) as zf:
            mbytes = zf.read(MEMBERS[0])
            payload = zf.read(MEMBERS[1])
    except (zipfile.BadZipFile, OSError, RuntimeError, ValueError, KeyError) as exc:
        reject(PackError, "P-CONTAINER", "zip", f"invalid ZIP container: {exc}")
    try:
        manifest = json.loads(mbytes.decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as exc:
        reject(PackError, "P-CONTAINER", "$.manifest.json", f"manifest is not UTF-8 JSON: {exc}")
    if not isinstance(manifest, dict):
        reject(PackError, "P-CONTAINER", "$", "manifest root must be an object")
    want = (manifest.get("payload") or {}).get("sha256")
    if want is not None and want != sha256_hex(payload):
        reject(PackError, "P-CONTAINER", "$.payload.sha256", "payload bytes do not match the recorded digest")
    return manifest, payload
