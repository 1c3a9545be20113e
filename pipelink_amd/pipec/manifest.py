"""Strict loaders for stage manifests and ``pipeline.json`` and the cross-object checks that
run before anything is solved.

Accepts the grammar the reference's own fixtures use (pipec/tests/pipec2/
test_negative_fixtures.py:46-224; schema in pipec/src/pipec2/schema.py:1033-1202 for stages,
:1390-1486 for pipelines, :1489-1826 for ``validate_assembly``) and raises the same named
clauses at the same paths:

* ``L-ENTRYABI``  unsupported schema / entry ABI / profile
* ``L-HANDLE``    incomplete variant key, undeclared or malformed handle, bad forced binding
* ``L-PARAMS``    one stage's params blob beyond the target limit
* ``L-PHASE``     exclusivity pair or claim lifetime naming an undeclared phase
* ``L-TOPO``      stage vs pipeline persistence / scheduler
* ``L-OWNER``     allocation handle without exactly one owning claim
* ``L-SYM``       symbol prefix not the normalised stage id

Manifests stay plain dicts (they are hashed and re-serialised canonically); the loaders
return light wrappers with the lookups the later phases need."""
from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Any

from .clauses import ClauseFailure, SchemaError
from .gfx950 import Profile, get_profile

SCHEMA_VERSIONS = ("3.0", "2.0-draft")  # 2.0-draft: the legacy stage schema, which has no tensor section
TENSOR_SCHEMA_VERSIONS = ("3.0",)
_STAGE_ID = re.compile(r"[a-z][a-z0-9_-]*(\.[a-z0-9][a-z0-9_-]*)+\Z")
_HANDLE = re.compile(r"pipelink_[a-z0-9_]+\Z")
_IDENT = re.compile(r"[A-Za-z_][A-Za-z0-9_]*\Z")
_STAGE_KEYS = {"pipelink_abi", "stage", "endpoints", "claims", "topology", "params", "hints", "payload", "symbols",
               "host", "tensor", "provenance", "facts"}
_PIPELINE_KEYS = {"name", "stages", "handles", "phases", "exclusive", "domains", "depth_priority", "regs_priority",
                  "forced_bindings", "topology", "tensor_connections", "math", "facts"}
HANDLE_CLASSES = ("depth", "regs", "base", "variant")
BINDINGS = ("bind", "fixed", "launch")
PROTOCOL_KINDS = ("mbarrier", "call", "counter", "named_barrier")


def normalise_prefix(stage_id: str) -> str:
    return stage_id.replace(".", "_").replace("-", "_") + "_"


class _Collector:
    def __init__(self) -> None:
        self.failures: list[ClauseFailure] = []

    def add(self, clause: str, path: str, message: str, **detail: Any) -> None:
        self.failures.append(ClauseFailure(clause, path, message, detail))

    def finish(self) -> None:
        if self.failures:
            raise SchemaError(self.failures)


def _is_int(v: Any) -> bool:
    return type(v) is int


def _abi(obj: Any, c: _Collector) -> Profile | None:
    abi = obj.get("pipelink_abi") if isinstance(obj, dict) else None
    if not isinstance(abi, dict):
        c.add("L-ENTRYABI", "$.pipelink_abi", "pipelink_abi must be an object")
        return None
    if abi.get("schema", "3.0") not in SCHEMA_VERSIONS:
        c.add("L-ENTRYABI", "$.pipelink_abi.schema", "unsupported manifest schema", actual=abi.get("schema"))
    target = abi.get("target")
    if not isinstance(target, dict) or not isinstance(target.get("profile"), str):
        c.add("L-ENTRYABI", "$.pipelink_abi.target", "target must name a profile")
        return None
    try:
        return get_profile(target["profile"])
    except SchemaError as err:
        c.failures.extend(err.failures)
        return None


@dataclass
class Stage:
    manifest: dict[str, Any]
    profile: Profile

    @property
    def id(self) -> str:
        return self.manifest["stage"]["id"]

    @property
    def prefix(self) -> str:
        return self.manifest["stage"]["symbol_prefix"]

    @property
    def roles(self) -> dict[str, dict[str, Any]]:
        return self.manifest["stage"]["roles"]

    @property
    def exports(self) -> dict[str, dict[str, Any]]:
        return self.manifest["stage"].get("exports", {})

    @property
    def variants(self) -> list[dict[str, Any]]:
        return self.manifest["stage"]["variants"]

    @property
    def endpoints(self) -> list[dict[str, Any]]:
        return self.manifest["endpoints"]

    @property
    def claims(self) -> list[dict[str, Any]]:
        return self.manifest["claims"]

    @property
    def topology(self) -> dict[str, Any]:
        return self.manifest["topology"]

    @property
    def params(self) -> dict[str, Any]:
        return self.manifest["params"]


@dataclass
class Pipeline:
    document: dict[str, Any]
    profile: Profile

    @property
    def body(self) -> dict[str, Any]:
        return self.document["pipeline"]

    @property
    def name(self) -> str:
        return self.body["name"]

    @property
    def handles(self) -> dict[str, dict[str, Any]]:
        return self.body["handles"]

    @property
    def phases(self) -> list[str]:
        return self.body["phases"]

    @property
    def stage_ids(self) -> list[str]:
        return [s["stage_id"] for s in self.body["stages"]]


def _check_endpoint(ep: Any, i: int, roles: dict[str, Any], c: _Collector) -> None:
    path = f"$.endpoints[{i}]"
    if not isinstance(ep, dict):
        c.add("L-PAIR", path, "endpoint must be an object")
        return
    if not isinstance(ep.get("name"), str) or not _IDENT.match(ep["name"]):
        c.add("L-PAIR", f"{path}.name", "endpoint name must be an identifier")
    if ep.get("direction") not in ("produce", "consume"):
        c.add("L-PAIR", f"{path}.direction", "direction must be 'produce' or 'consume'")
    proto = ep.get("protocol")
    if not isinstance(proto, dict) or proto.get("kind") not in PROTOCOL_KINDS:
        c.add("L-PROTO", f"{path}.protocol.kind", "unsupported protocol kind",
              actual=proto.get("kind") if isinstance(proto, dict) else None)
        return
    role = ep.get("owner_role")
    if role is not None and role not in roles:
        c.add("L-PAIR", f"{path}.owner_role", "endpoint owner role is not a role of this stage")
    if proto["kind"] == "mbarrier":
        for side in ("full", "empty"):
            s = proto.get(side)
            if s is None:
                continue
            if isinstance(s, dict) and isinstance(s.get("tx_bytes"), dict):
                names = s["tx_bytes"].get("sum")
                if isinstance(names, list) and len(set(names)) != len(names):
                    c.add("L-PROTO", f"{path}.protocol.{side}.tx_bytes.sum", "array entries must be unique")


def load_stage_manifest(obj: Any) -> Stage:
    """Validate one ``manifest.json`` object (schema.py:1033 in the reference)."""
    c = _Collector()
    if not isinstance(obj, dict):
        c.add("L-ENTRYABI", "$", "manifest root must be an object")
        c.finish()
    for key in sorted(set(obj) - _STAGE_KEYS):
        c.add("L-ENTRYABI", f"$.{key}", "unknown manifest field")
    profile = _abi(obj, c)
    stage = obj.get("stage")
    if not isinstance(stage, dict):
        c.add("L-ENTRYABI", "$.stage", "stage must be an object")
        c.finish()
    sid = stage.get("id")
    if not isinstance(sid, str) or not _STAGE_ID.match(sid):
        c.add("L-SYM", "$.stage.id", "stage id must be a lowercase reverse-DNS name")
        sid = str(sid)
    if stage.get("symbol_prefix") != normalise_prefix(sid):
        c.add("L-SYM", "$.stage.symbol_prefix", "symbol prefix must be the normalised stage id")
    if stage.get("entry_abi") != "v2":
        c.add("L-ENTRYABI", "$.stage.entry_abi", "stage entry ABI is not supported by this linker",
              actual=stage.get("entry_abi"))
    if stage.get("entry_signature") != "void(const void* params, unsigned variant)":
        c.add("L-ENTRYABI", "$.stage.entry_signature", "role entry signature must be the v2 signature")
    roles = stage.get("roles")
    if not isinstance(roles, dict):
        c.add("L-ENTRYABI", "$.stage.roles", "roles must be an object")
        roles = {}
    for name, role in roles.items():
        if not isinstance(role, dict) or not _is_int(role.get("warps")) or role["warps"] <= 0:
            c.add("L-TOPO", f"$.stage.roles.{name}.warps", "role must claim a positive number of warps")
        if not isinstance(role, dict) or not isinstance(role.get("entry"), str) or not _IDENT.match(role["entry"]):
            c.add("L-SYM", f"$.stage.roles.{name}.entry", "role entry must be an identifier")
    exports = stage.get("exports", {})
    if not isinstance(exports, dict):
        c.add("L-ENTRYABI", "$.stage.exports", "exports must be an object")
    variants = stage.get("variants")
    if not isinstance(variants, list) or not variants:
        c.add("L-HANDLE", "$.stage.variants", "a stage declares at least one variant")
        variants = []
    keyset = None
    seen_index: set[int] = set()
    for i, var in enumerate(variants):
        key = var.get("key") if isinstance(var, dict) else None
        if not isinstance(key, dict) or not all(_HANDLE.match(str(k)) and _is_int(v) for k, v in key.items()):
            c.add("L-HANDLE", f"$.stage.variants[{i}].key", "variant key must map pipelink_* handles to integers")
            continue
        if keyset is None:
            keyset = set(key)
        elif set(key) != keyset:
            c.add("L-HANDLE", f"$.stage.variants[{i}].key", "variant key is incomplete",
                  expected=sorted(keyset), actual=sorted(key))
        if not _is_int(var.get("index")) or var["index"] in seen_index:
            c.add("L-HANDLE", f"$.stage.variants[{i}].index", "variant index must be a unique integer")
        else:
            seen_index.add(var["index"])
    params = obj.get("params")
    if not isinstance(params, dict) or not _is_int(params.get("bytes")) or params["bytes"] < 0:
        c.add("L-PARAMS", "$.params", "params must give a byte size")
    else:
        align = params.get("align")
        if not _is_int(align) or align <= 0 or align & (align - 1):
            c.add("L-PARAMS", "$.params.align", "params alignment must be a power of two")
        if profile is not None and params["bytes"] > profile.param_limit_bytes:
            c.add("L-PARAMS", "$.params.bytes", "parameter blob exceeds the target parameter limit",
                  limit=profile.param_limit_bytes, actual=params["bytes"])
    endpoints = obj.get("endpoints")
    if not isinstance(endpoints, list):
        c.add("L-PAIR", "$.endpoints", "endpoints must be an array")
        endpoints = []
    for i, ep in enumerate(endpoints):
        _check_endpoint(ep, i, roles, c)
    claims = obj.get("claims")
    if not isinstance(claims, list):
        c.add("L-OWNER", "$.claims", "claims must be an array")
        claims = []
    for i, claim in enumerate(claims):
        path = f"$.claims[{i}]"
        if not isinstance(claim, dict) or not isinstance(claim.get("domain"), str):
            c.add("L-OWNER", path, "claim must name a domain")
            continue
        if not isinstance(claim.get("handle"), str) or not _HANDLE.match(claim["handle"]):
            c.add("L-HANDLE", f"{path}.handle", "claim handle must be a pipelink_* name")
        if claim["domain"] == "regs":
            continue
        ext = claim.get("extent")
        if not isinstance(ext, dict) or not _is_int(ext.get("const")) or not isinstance(ext.get("per", {}), dict):
            c.add("L-OVERLAP", f"{path}.extent", "claim extent must be {const, per}")
        al = claim.get("align", 1)
        if not _is_int(al) or al <= 0:
            c.add("L-ALIGN", f"{path}.align", "claim alignment must be positive")
    topo = obj.get("topology")
    if not isinstance(topo, dict) or not isinstance(topo.get("persistent"), bool) or \
            not isinstance(topo.get("scheduler"), str):
        c.add("L-TOPO", "$.topology", "topology must give persistent and scheduler")
    if "tensor" in obj:
        from .tensors import check_stage_tensor  # (tensors imports this module)

        schema = obj["pipelink_abi"].get("schema", "3.0") if isinstance(obj.get("pipelink_abi"), dict) else None
        for path, message, detail in check_stage_tensor(obj["tensor"], schema in TENSOR_SCHEMA_VERSIONS):
            c.add("T-CONTRACT", path, message, **detail)
    c.finish()
    return Stage(obj, profile)  # type: ignore[arg-type]


def load_pipeline(obj: Any) -> Pipeline:
    """Validate one ``pipeline.json`` object (schema.py:1390 in the reference)."""
    c = _Collector()
    if not isinstance(obj, dict) or not isinstance(obj.get("pipeline"), dict):
        c.add("L-ENTRYABI", "$.pipeline", "pipeline must be an object")
        c.finish()
    profile = _abi(obj, c)
    p = obj["pipeline"]
    for key in sorted(set(p) - _PIPELINE_KEYS):
        c.add("L-ENTRYABI", f"$.pipeline.{key}", "unknown pipeline field")
    if not isinstance(p.get("name"), str) or not p["name"]:
        c.add("L-ENTRYABI", "$.pipeline.name", "pipeline needs a name")
    stages = p.get("stages")
    if not isinstance(stages, list) or not stages:
        c.add("L-PAIR", "$.pipeline.stages", "pipeline lists at least one stage")
        stages = []
    seen: set[str] = set()
    for i, s in enumerate(stages):
        if not isinstance(s, dict) or not isinstance(s.get("stage_id"), str) or \
                not isinstance(s.get("artifact_path"), str):
            c.add("L-PAIR", f"$.pipeline.stages[{i}]", "stage entry needs artifact_path and stage_id")
        elif s["stage_id"] in seen:
            c.add("L-SYM", f"$.pipeline.stages[{i}].stage_id", "stage is listed twice")
        else:
            seen.add(s["stage_id"])
    handles = p.get("handles")
    if not isinstance(handles, dict):
        c.add("L-HANDLE", "$.pipeline.handles", "handles must be an object")
        handles = {}
    for name, h in handles.items():
        path = f"$.pipeline.handles.{name}"
        if not _HANDLE.match(str(name)):
            c.add("L-HANDLE", path, "handle names start with pipelink_")
        if not isinstance(h, dict) or h.get("class") not in HANDLE_CLASSES:
            c.add("L-HANDLE", f"{path}.class", "handle class must be depth, regs, base or variant")
            continue
        if h.get("binding") not in BINDINGS:
            c.add("L-HANDLE", f"{path}.binding", "handle binding must be bind, fixed or launch")
        if not isinstance(h.get("owner"), str) or ":" not in h["owner"]:
            c.add("L-OWNER", f"{path}.owner", "handle owner must be '<kind>:<name>'")
        if h["class"] in ("depth", "variant", "regs"):
            vals = h.get("values")
            if not isinstance(vals, list) or not vals or not all(_is_int(v) for v in vals):
                c.add("L-HANDLE", f"{path}.values", "finite handles list their candidate integer values")
        if h["class"] == "base" and not isinstance(h.get("domain"), str):
            c.add("L-HANDLE", f"{path}.domain", "base handles name their claim domain")
    phases = p.get("phases")
    if not isinstance(phases, list) or not phases or len(set(phases)) != len(phases) or \
            not all(isinstance(x, str) and _IDENT.match(x) for x in phases):
        c.add("L-PHASE", "$.pipeline.phases", "phases must be a non-empty list of unique identifiers")
        phases = []
    exclusive = p.get("exclusive", [])
    if not isinstance(exclusive, list):
        c.add("L-PHASE", "$.pipeline.exclusive", "exclusive must be a list of phase pairs")
        exclusive = []
    for i, pair in enumerate(exclusive):
        if not isinstance(pair, list) or len(pair) != 2:
            c.add("L-PHASE", f"$.pipeline.exclusive[{i}]", "exclusivity entries are pairs of phases")
            continue
        for j, ph in enumerate(pair):
            if ph not in phases:
                c.add("L-PHASE", f"$.pipeline.exclusive[{i}][{j}]", "unknown phase", actual=ph)
        if pair[0] == pair[1]:
            c.add("L-PHASE", f"$.pipeline.exclusive[{i}]", "a phase cannot exclude itself")
    for key, cls in (("depth_priority", "depth"), ("regs_priority", "regs")):
        for i, name in enumerate(p.get(key, [])):
            if name not in handles or handles[name].get("class") != cls:
                c.add("L-HANDLE", f"$.pipeline.{key}[{i}]", f"priority entry is not a declared {cls} handle")
    for name, value in (p.get("forced_bindings") or {}).items():
        h = handles.get(name)
        if h is None:
            c.add("L-HANDLE", f"$.pipeline.forced_bindings.{name}", "forced binding names an undeclared handle")
        elif "values" in h and value not in h["values"]:
            c.add("L-HANDLE", f"$.pipeline.forced_bindings.{name}", "forced value is not one of the handle's values",
                  values=h["values"], actual=value)
    topo = p.get("topology")
    if not isinstance(topo, dict) or not isinstance(topo.get("persistent"), bool) or \
            not isinstance(topo.get("scheduler"), str):
        c.add("L-TOPO", "$.pipeline.topology", "pipeline topology must give persistent and scheduler")
    domains = p.get("domains", {})
    if not isinstance(domains, dict):
        c.add("L-OVERLAP", "$.pipeline.domains", "domains must be an object")
    c.finish()
    return Pipeline(obj, profile)  # type: ignore[arg-type]


def endpoint_handle_refs(ep: dict[str, Any]) -> list[tuple[str, str]]:
    """(path suffix, handle name) for every pipelink_* handle an endpoint mentions."""
    refs: list[tuple[str, str]] = []
    ring = ep.get("ring")
    if isinstance(ring, dict) and isinstance(ring.get("depth"), dict) and "handle" in ring["depth"]:
        refs.append(("ring.depth.handle", ring["depth"]["handle"]))
    proto = ep.get("protocol", {})
    for side in ("full", "empty"):
        s = proto.get(side)
        if isinstance(s, dict) and isinstance(s.get("slots"), str):
            refs.append((f"protocol.{side}.slots", s["slots"]))
    if proto.get("kind") == "counter" and isinstance(proto.get("slot"), str):
        refs.append(("protocol.slot", proto["slot"]))
    if proto.get("kind") == "named_barrier" and isinstance(proto.get("id"), str):
        refs.append(("protocol.id", proto["id"]))
    for key, name in (ep.get("binds") or {}).items():
        refs.append((f"binds.{key}", name))
    return refs


def validate_assembly(pipeline: Pipeline, stages: list[Stage]) -> list[ClauseFailure]:
    """Checks that need the pipeline and every stage together (schema.py:1489 in the reference).
    Returns the failures; an empty list means the assembly is admissible."""
    out: list[ClauseFailure] = []
    handles = pipeline.handles
    by_id = {s.id: s for s in stages}
    for sid in pipeline.stage_ids:
        if sid not in by_id:
            out.append(ClauseFailure("L-PAIR", f"pipeline.stages.{sid}", "listed stage has no artifact"))
    for s in stages:
        if s.id not in pipeline.stage_ids:
            out.append(ClauseFailure("L-PAIR", f"stages.{s.id}", "artifact is not listed by the pipeline"))
        if s.profile.name != pipeline.profile.name:
            out.append(ClauseFailure("L-ENTRYABI", f"stages.{s.id}.pipelink_abi.target.profile",
                                     "stage and pipeline target profiles disagree"))
        ptopo = pipeline.body["topology"]
        if s.topology["persistent"] != ptopo["persistent"]:
            out.append(ClauseFailure("L-TOPO", f"stages.{s.id}.topology.persistent",
                                     "stage and pipeline persistence disagree"))
        if s.topology["scheduler"] != ptopo["scheduler"]:
            out.append(ClauseFailure("L-TOPO", f"stages.{s.id}.topology.scheduler",
                                     "stage and pipeline scheduler disagree"))
        for ep in s.endpoints:
            for suffix, name in endpoint_handle_refs(ep):
                if name not in handles:
                    out.append(ClauseFailure(
                        "L-HANDLE", f"stages.{s.id}.endpoints.{ep['name']}.{suffix}",
                        "referenced pipelink_* handle is not declared in pipeline scope", {"handle": name}))
        for claim in s.claims:
            cpath = f"stages.{s.id}.claims.{claim['domain']}.{claim['handle']}"
            if claim["handle"] not in handles:
                out.append(ClauseFailure("L-HANDLE", f"{cpath}.handle",
                                         "referenced pipelink_* handle is not declared in pipeline scope",
                                         {"handle": claim["handle"]}))
            for dep in (claim.get("extent") or {}).get("per", {}):
                if dep not in handles or handles[dep]["class"] != "depth":
                    out.append(ClauseFailure("L-HANDLE", f"{cpath}.extent.per.{dep}",
                                             "claim extent depends on an undeclared depth handle"))
            life = claim.get("lifetime", "kernel")
            if life != "kernel":
                if not isinstance(life, str) or not life.startswith("phase:") or life[6:] not in pipeline.phases:
                    out.append(ClauseFailure("L-PHASE", f"{cpath}.lifetime",
                                             "claim lifetime names an undeclared phase", {"lifetime": life}))
        for i, var in enumerate(s.variants):
            for name in var["key"]:
                if name not in handles:
                    out.append(ClauseFailure("L-HANDLE", f"stages.{s.id}.stage.variants[{i}].key.{name}",
                                             "referenced pipelink_* handle is not declared in pipeline scope"))
    # every base handle is allocated by exactly one claim (identical claims under one alias aside)
    owners: dict[str, list[str]] = {}
    for s in stages:
        for claim in s.claims:
            if claim["domain"] != "regs":
                owners.setdefault(claim["handle"], []).append(s.id)
    for name, h in handles.items():
        if h["class"] == "base" and h["binding"] == "bind":
            n = len(owners.get(name, []))
            if n != 1:
                out.append(ClauseFailure("L-OWNER", f"pipeline.handles.{name}",
                                         "allocation handle needs exactly one owning claim", {"claims": n}))
    return sorted(out, key=lambda f: (f.clause_id, f.path))
