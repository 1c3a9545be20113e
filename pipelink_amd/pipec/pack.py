"""``pipec pack``: one annotated HIP stage source -> one ``.plink``.

Steps (the reference's pipec/src/pipec2/pack/__init__.py:10-55 with hipcc in nvcc's place):
1. emit program -- the source is compiled for the *host* with ``-DPIPELINK_EMIT`` and run; it
   prints the annotation registry as JSON (pack/emit.py:54-114);
2. device object -- ``hipcc --offload-arch=gfx950 -fgpu-rdc --cuda-device-only -emit-llvm``
   gives AMDGPU LLVM bitcode, the LTO payload (the reference ships an NVVM-LTO ELF);
3. assemble -- registry -> manifest: call seams become ``call`` endpoints carrying the
   declaration text and its digest, counters become ``counter`` endpoints, claims, variants,
   topology, params (+ layout probe digest), published facts (pack/assemble.py:199-379);
4. observe -- defined symbols of the bitcode must carry the normalised stage prefix
   (``P-SYM``, pack/objectfacts.py:55-74);
5. container -- ``plink.pack``."""
from __future__ import annotations

import json
import os
import re
import subprocess
import tempfile
from pathlib import Path
from typing import Any

from . import plink
from .channels import call_symbol, declaration_digest
from .clauses import ClauseFailure, PackError
from .gfx950 import get_profile
from .manifest import load_stage_manifest, normalise_prefix

INCLUDE_DIR = Path(__file__).resolve().parent / "include"
LLVM_BIN = Path(os.environ.get("PIPEC_LLVM_BIN", "/opt/rocm/lib/llvm/bin"))
HIPCC = os.environ.get("PIPEC_HIPCC", "/opt/rocm/bin/hipcc")
TOOLKIT = "rocm-7.2.0"

# Math mode and code-generation flags are part of the target stamp: the final link and the
# one-unit control re-apply exactly these (the reference records nvcc's math mode the same
# way, pipec/src/pipec2/link.py:565-590).  Packed FP32 VALU forms are switched off.
DEVICE_FLAGS = ["-O3", "-std=c++17", "-ffp-contract=fast", "-fgpu-flush-denormals-to-zero",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _fail(clause: str, path: str, message: str, **detail: Any):
    raise PackError([ClauseFailure(clause, path, message, detail)])


def _run(cmd: list[str], what: str, cwd: str | None = None) -> subprocess.CompletedProcess:
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=cwd)
    if proc.returncode != 0:
        _fail("P-COMPILE", what, f"{Path(cmd[0]).name} failed: {proc.stderr.strip()[-2000:]}", argv=cmd)
    return proc


def emit_registry(source: Path, include_dirs: list[Path]) -> dict[str, Any]:
    with tempfile.TemporaryDirectory(prefix="pipec-emit-") as tmp:
        exe = Path(tmp) / "emit"
        inc = [f"-I{d}" for d in [INCLUDE_DIR, *include_dirs]]
        _run(["g++", "-std=c++17", "-x", "c++", "-DPIPELINK_EMIT", *inc, str(source), "-o", str(exe)], "emit.compile")
        out = _run([str(exe)], "emit.run").stdout
    try:
        return json.loads(out)
    except json.JSONDecodeError as exc:
        _fail("P-COMPILE", "emit.run", f"registry is not JSON: {exc}")


def compile_bitcode(source: Path, include_dirs: list[Path], arch: str, out: Path, defines: list[str] | None = None) -> None:
    inc = [f"-I{d}" for d in [INCLUDE_DIR, *include_dirs]]
    _run([HIPCC, f"--offload-arch={arch}", "-x", "hip", "-fgpu-rdc", "--cuda-device-only", "-emit-llvm", "-c",
          *DEVICE_FLAGS, *[f"-D{d}" for d in (defines or [])], *inc, str(source), "-o", str(out)], "device.compile")


_DEFINE = re.compile(r"^define\s+(?P<attrs>[^@]*)@(?P<name>[A-Za-z_$.][\w$.]*)\(", re.M)


def defined_symbols(bitcode: Path) -> list[str]:
    """Strong external definitions of a bitcode module (read from its textual IR)."""
    text = _run([str(LLVM_BIN / "llvm-dis"), str(bitcode), "-o", "-"], "device.symbols").stdout
    names = []
    for m in _DEFINE.finditer(text):
        attrs = m.group("attrs").split()
        if any(a in ("internal", "private", "linkonce_odr", "linkonce", "weak", "weak_odr", "available_externally")
               for a in attrs):
            continue
        names.append(m.group("name"))
    return sorted(names)


def _prelude(path: Path) -> dict[str, str]:
    if not path.exists():
        _fail("P-COMPILE", "$.hints.preludes", f"prelude header {path} does not exist")
    text = path.read_text()
    return {"name": path.name, "text": text, "sha256": plink.sha256_hex(text.encode())}


def assemble(registry: dict[str, Any], profile_name: str, source: Path) -> dict[str, Any]:
    """Registry records -> manifest object (without the payload digest)."""
    profile = get_profile(profile_name)
    if len(registry.get("stage", [])) != 1:
        _fail("P-COMPILE", "$.stage", "a stage source carries exactly one PL_STAGE")
    stage = registry["stage"][0]
    prefix = normalise_prefix(stage["id"])
    params = (registry.get("params") or [{"type": "void", "bytes": 0, "align": 1}])[0]
    roles = {r["name"]: {"entry": r["entry"], "warps": r["warps"]} for r in registry.get("roles", [])}
    exports = {}
    for e in registry.get("exports", []):
        if not e["symbol"].startswith(prefix):
            _fail("P-SYM", f"$.stage.exports.{e['name']}", "export symbol does not carry the normalised stage prefix",
                  symbol=e["symbol"], prefix=prefix)
        exports[e["name"]] = {"symbol": e["symbol"], "decl": e["decl"], "decl_sha256": declaration_digest(e["decl"])}
    for name, r in roles.items():
        if not r["entry"].startswith(prefix):
            _fail("P-SYM", f"$.stage.roles.{name}.entry", "role entry does not carry the normalised stage prefix")
    endpoints = []
    for c in registry.get("calls", []):
        if c["direction"] == "produce":
            decl = c["decl"]
            if call_symbol(c["channel"]) not in decl:
                _fail("P-SYM", f"$.endpoints.{c['channel']}", "caller declaration must declare the channel trampoline")
        else:
            if c["export"] not in exports:
                _fail("P-SYM", f"$.endpoints.{c['channel']}", "served export is not declared with PL_EXPORT")
            decl = exports[c["export"]]["decl"]
        endpoints.append({
            "name": c["channel"], "direction": c["direction"],
            "owner_role": next(iter(roles), None) if c["direction"] == "produce" else None,
            "space": "reg", "scope": "cta", "proxy": "generic", "tile": {"dtype": "s32", "shape": [1]},
            "layout": {"encoding": "pl-layout-v2", "elem_bits": 32, "shape": [1], "stride": [1]},
            "protocol": {"kind": "call", "export": c["export"], "decl": decl, "decl_sha256": declaration_digest(decl)},
            "binds": {}})
    for c in registry.get("counters", []):
        endpoints.append({
            "name": c["name"], "direction": c["direction"], "owner_role": None, "exports": c["exports"],
            "space": "gmem", "scope": "grid", "proxy": "generic", "tile": {"dtype": "i32", "shape": [1]},
            "layout": {"encoding": "pl-layout-v2", "elem_bits": 32, "shape": [1], "stride": [1]},
            "protocol": {"kind": "counter", "slot": c["slot"], "release": "atomic_add.release.agent",
                         "acquire": "load.acquire.agent"},
            "binds": {}})
    def count(text: str):
        return int(text) if text.isdigit() else text

    for r in registry.get("rings", []):
        endpoints.append({
            "name": r["name"], "direction": r["direction"], "owner_role": r["owner_role"],
            "space": "smem", "scope": "cta", "proxy": "async", "tile": {"dtype": r["dtype"], "shape": [r["rows"], r["cols"]]},
            "layout": {"encoding": "pl-layout-v2", "elem_bits": r["elem_bits"], "shape": [[r["rows"]], [r["cols"]]],
                       "stride": [[r["cols"]], [1]]},
            "ring": {"depth": {"handle": r["depth"]}, "stage_stride_bytes": r["stride"]},
            "protocol": {"kind": "mbarrier",
                         "full": {"slots": r["full"], "arrive": {"count": count(r["full_count"]), "by": r["full_by"]},
                                  "tx_bytes": "tile"},
                         "empty": {"slots": r["empty"], "arrive": {"count": count(r["empty_count"]), "by": r["empty_by"]},
                                   "tx_bytes": 0},
                         "init": {"owner": r["init_owner"], "materializer": "dispatch", "phase": 0},
                         "release": "once-per-acquire"},
            "binds": {"full": r["full"], "empty": r["empty"]}})
    topo = (registry.get("topology") or [{"persistent": False, "scheduler": "static"}])[0]
    variants = sorted(registry.get("variants") or [{"index": 0, "key": {}}], key=lambda v: v["index"])
    probe = plink.sha256_hex(plink.canonical_bytes({"type": params["type"], "bytes": params["bytes"],
                                                    "align": params["align"]}))
    tensor = {}
    if registry.get("tensor_exports") or registry.get("tensor_imports"):
        tensor = {"tensor": {"schema": "tensor-v1", "exports": registry.get("tensor_exports", []),
                             "imports": registry.get("tensor_imports", [])}}
    host = {}
    if registry.get("host_group"):
        group = registry["host_group"][0]
        channels = sorted(registry.get("host_channels", []), key=lambda c: c["id"])
        if [c["id"] for c in channels] != list(range(1, len(channels) + 1)):
            _fail("L-HOSTCHAN", "$.host.channels", "host channel ids must be 1..n without gaps", ids=[c["id"] for c in channels])
        if params["bytes"] == 0:
            _fail("L-HOSTCHAN", "$.host.params_group", "a stage without params cannot own a params group")
        host = {"host": {"schema": "host-v2", "params_group": group["params_group"], "provider": group["provider"],
                         "abi_types": sorted(registry.get("host_types", []), key=lambda t: t["id"]),
                         "scalars": sorted(registry.get("host_scalars", []), key=lambda t: t["id"]),
                         "channels": channels}}
    return {
        **tensor,
        **host,
        "pipelink_abi": {"schema": "3.0", "target": {
            "profile": profile.name, "lto_arch": profile.lto_arch, "toolkit": TOOLKIT,
            "math": {"flags": DEVICE_FLAGS}}},
        "stage": {"id": stage["id"], "version": stage["version"], "symbol_prefix": prefix, "entry_abi": "v2",
                  "entry_signature": "void(const void* params, unsigned variant)", "roles": roles, "exports": exports,
                  "variants": [{"key": v["key"], "index": v["index"]} for v in variants]},
        "endpoints": endpoints,
        "claims": registry.get("claims", []),
        "topology": {"cta_group": {"fixed": 1}, "cluster": {"compiled": [1, 1, 1], "launch": {"x_multiple_of": 1, "max": [1, 1, 1]}},
                     "multicast": [], "persistent": topo["persistent"], "scheduler": topo["scheduler"]},
        "params": {"type": params["type"], "bytes": params["bytes"], "align": params["align"],
                   "sha256_of_layout_probe": probe},
        "facts": {f["name"]: f["value"] for f in registry.get("facts", [])},
        "hints": {"uses": sorted(registry.get("uses", [])),
                  "preludes": [_prelude(source.parent / rel) for rel in registry.get("preludes", [])]},
        "provenance": {"source": str(source), "source_sha256": plink.sha256_hex(source.read_bytes())},
        "payload": {"file": "stage.o"},
    }


def pack_stage(source: str | Path, out: str | Path, *, include_dirs: list[str | Path] | None = None,
               profile: str = "gfx950", defines: list[str] | None = None) -> dict[str, Any]:
    """Compile, describe and package one stage.  Returns the pack report."""
    source = Path(source).resolve()
    dirs = [Path(d).resolve() for d in (include_dirs or [])]
    registry = emit_registry(source, dirs)
    manifest = assemble(registry, profile, source)
    load_stage_manifest(manifest)  # the packer never writes a manifest its own loader refuses
    with tempfile.TemporaryDirectory(prefix="pipec-pack-") as tmp:
        bc = Path(tmp) / "stage.bc"
        compile_bitcode(source, dirs, profile, bc, defines)
        symbols = defined_symbols(bc)
        prefix = manifest["stage"]["symbol_prefix"]
        for sym in symbols:
            if not sym.startswith(prefix) and not sym.startswith("_Z"):
                _fail("P-SYM", "$.symbols.defined_strong", "defined symbol does not carry the normalised stage prefix",
                      symbol=sym, prefix=prefix)
        manifest["symbols"] = {"defined_strong": symbols}
        report = plink.pack(manifest, bc.read_bytes(), out)
    report["stage_id"] = manifest["stage"]["id"]
    return report
