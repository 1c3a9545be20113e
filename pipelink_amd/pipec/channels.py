"""Channel pairing and protocol expansion: every channel has one producer and one consumer
endpoint, and the two sides must have declared the same protocol.  Every disagreement is an
``L-PROTO`` failure at ``channels.<name>...`` with the reference's wording
(pipec/src/pipec2/protocol.py:27-28 ``_reject``; expansion :511-818, counter :821-853; pairing
link.py:263-307 ``L-PAIR``), because its contract gallery greps those lines verbatim
(docs/tutorials/T3-contract-gallery.md:92-94).

Protocol kinds:
* ``mbarrier``  a full/empty counter ring.  On gfx950 the slots are 16-byte LDS cells holding
  32-bit counters; arrive counts are compared as expressions, ``threads(role)`` expands with
  the profile's wave width (64), ``tx_bytes: "tile"`` to the tile's byte footprint.
* ``call``      a cross-package function call; both sides carry the declaration text and its
  digest, the consumer must export the named symbol.
* ``counter``   a global-memory counter slot (release add / acquire load).
* ``named_barrier``  the workgroup barrier.
"""
from __future__ import annotations

import hashlib
import re
from dataclasses import dataclass, field
from typing import Any

from .clauses import ClauseFailure, LinkError, SolveError
from .manifest import Pipeline, Stage

DTYPE_BITS = {"bf16": 16, "f16": 16, "f32": 32, "s32": 32, "i32": 32, "u32": 32, "u8": 8, "s8": 8, "e4m3": 8,
              "e8m0": 8, "f64": 64}


def _reject(path: str, message: str, **detail: Any):
    raise SolveError([ClauseFailure("L-PROTO", path, message, detail)])


# ---- declarations -------------------------------------------------------------------------
_COMMENT = re.compile(r"//[^\n]*|/\*.*?\*/", re.S)
_TOKEN = re.compile(r'"(?:\\.|[^"\\])*"|\'(?:\\.|[^\'\\])*\'|\s+|[^\s"\']+')


def normalize_declaration(text: str) -> str:
    """Comments become whitespace, whitespace runs one space, literals stay untouched."""
    text = _COMMENT.sub(" ", text)
    out = []
    for tok in _TOKEN.findall(text):
        out.append(" " if tok.isspace() else tok)
    return "".join(out).strip()


def declaration_digest(text: str) -> str:
    return hashlib.sha256(normalize_declaration(text).encode("utf-8")).hexdigest()


def call_symbol(channel: str) -> str:
    return f"pipelink_call_{channel}"


# ---- pairing ------------------------------------------------------------------------------
@dataclass
class Channel:
    name: str
    producer_stage: Stage
    producer: dict[str, Any]
    consumer_stage: Stage
    consumer: dict[str, Any]


def pair_channels(stages: list[Stage]) -> dict[str, Channel]:
    sides: dict[str, dict[str, list[tuple[Stage, dict[str, Any]]]]] = {}
    for s in stages:
        for ep in s.endpoints:
            sides.setdefault(ep["name"], {"produce": [], "consume": []})[ep["direction"]].append((s, ep))
    failures = []
    out: dict[str, Channel] = {}
    for name in sorted(sides):
        prod, cons = sides[name]["produce"], sides[name]["consume"]
        if len(prod) != 1 or len(cons) != 1:
            failures.append(ClauseFailure("L-PAIR", f"channels.{name}",
                                          "channel needs exactly one producer and one consumer",
                                          {"producers": len(prod), "consumers": len(cons)}))
            continue
        (ps, pe), (cs, ce) = prod[0], cons[0]
        for key in ("space", "scope", "proxy"):
            if pe.get(key) != ce.get(key):
                failures.append(ClauseFailure("L-PAIR", f"channels.{name}.{key}",
                                              f"producer and consumer {key} disagree"))
        if pe.get("tile") != ce.get("tile"):
            failures.append(ClauseFailure("L-PAIR", f"channels.{name}.tile", "producer and consumer tiles disagree"))
        if pe.get("layout") != ce.get("layout"):
            failures.append(ClauseFailure("L8", f"channels.{name}.layout",
                                          "producer and consumer physical layouts disagree"))
        out[name] = Channel(name, ps, pe, cs, ce)
    if failures:
        raise LinkError(failures)
    return out


# ---- expansion ----------------------------------------------------------------------------
@dataclass
class Expansion:
    channel: str
    kind: str
    tx_full: int | None = None
    tx_empty: int | None = None
    arrive_full: int | None = None
    arrive_empty: int | None = None
    init_owner: str | None = None
    init_materializer: str | None = None
    slots: tuple[str, str] | None = None
    depth: str | int | None = None
    call: tuple[str, str, str] | None = None      # (export symbol, declaration, digest)
    named_barrier: tuple[str, int] | None = None
    counter: dict[str, Any] | None = None
    detail: dict[str, Any] = field(default_factory=dict)

    def to_json_obj(self) -> dict[str, Any]:
        return {k: (list(v) if isinstance(v, tuple) else v) for k, v in self.__dict__.items()
                if v not in (None, {}) or k in ("channel", "kind")}


def tile_bytes(ep: dict[str, Any], path: str) -> int:
    tile = ep.get("tile") or {}
    bits = DTYPE_BITS.get(tile.get("dtype"))
    if bits is None or not isinstance(tile.get("shape"), list):
        _reject(path, "tile footprint is not defined for this dtype")
    n = 1
    for d in tile["shape"]:
        n *= int(d)
    return n * bits // 8


_TERM = re.compile(r"(?:(\d+)\*)?(threads|warps)\(([A-Za-z_][A-Za-z0-9_]*)\)\Z")


def arrive_count(expr: Any, roles: dict[str, int], wave: int, path: str) -> int:
    """int > 0, or '+'-joined terms [k*]threads(role) / [k*]warps(role)."""
    if type(expr) is int:
        if expr <= 0:
            _reject(path, "arrive count must be positive")
        return expr
    if not isinstance(expr, str) or not expr:
        _reject(path, "invalid arrive count expression")
    if expr.isdigit():
        return arrive_count(int(expr), roles, wave, path)
    total = 0
    for term in expr.replace(" ", "").split("+"):
        m = _TERM.match(term)
        if not m:
            _reject(path, "invalid arrive count expression", term=term)
        k, fn, role = int(m.group(1) or 1), m.group(2), m.group(3)
        if role not in roles:
            _reject(path, "arrive count names a role that is not launched", role=role)
        total += k * roles[role] * (wave if fn == "threads" else 1)
    if total <= 0:
        _reject(path, "arrive count must be positive")
    return total


def _ring_identity(ep: dict[str, Any]):
    ring = ep.get("ring")
    if not isinstance(ring, dict):
        return None
    depth = ring.get("depth", {})
    ident = depth.get("handle") if "handle" in depth else ("fixed", depth.get("fixed"))
    return ident, ring.get("stage_stride_bytes")


def _check_slots(handle: str, depth_ident, pipeline: Pipeline, claims: dict[str, dict[str, Any]], path: str):
    decl = pipeline.handles.get(handle)
    if decl is None or decl.get("class") != "base" or decl.get("domain") != "mbarrier":
        _reject(path, "barrier slots handle is not declared in the mbarrier domain", handle=handle)
    claim = claims.get(handle)
    if claim is None:
        _reject(path, "barrier slots handle has no allocation claim", handle=handle)
    ext = claim["extent"]
    if isinstance(depth_ident, tuple):
        ok = ext.get("const") == depth_ident[1] and not ext.get("per")
    else:
        ok = ext.get("const") == 0 and ext.get("per") == {depth_ident: 1}
    if not ok:
        _reject(path, "barrier slots extent must equal the ring depth", handle=handle)


def shared_completion(channels: dict[str, Channel]) -> dict[tuple[str, str], str]:
    """(channel, side) -> the channel whose barrier side it completes on (``member_of``).

    Several tiles that always arrive together may share one counter: one channel's side is the *root* (it owns the
    slots and the arrival count, and states the bytes one completion stands for as ``tx_bytes: {"sum": [...]}`` over
    itself and its members), the others name it with ``member_of`` and state only their own tile.  A member may only
    name a root: membership does not chain."""
    member: dict[tuple[str, str], str] = {}
    for name, ch in channels.items():
        pp, cp = ch.producer["protocol"], ch.consumer["protocol"]
        if pp.get("kind") != "mbarrier" or cp.get("kind") != "mbarrier":
            continue
        for side in ("full", "empty"):
            ps, cs = pp.get(side), cp.get(side)
            if isinstance(ps, dict) and isinstance(cs, dict) and ("member_of" in ps or "member_of" in cs):
                if ps.get("member_of") != cs.get("member_of") or not isinstance(ps.get("member_of"), str):
                    _reject(f"channels.{name}.protocol.{side}.member_of", "producer and consumer name different roots")
                member[(name, side)] = ps["member_of"]
    for (name, side), root in sorted(member.items()):
        target = channels.get(root)
        target_side = target.producer["protocol"].get(side) if target and target.producer["protocol"].get("kind") == "mbarrier" else None
        if not isinstance(target_side, dict) or (root, side) in member:
            _reject(f"channels.{root}.protocol.{side}", "member_of may only target a root barrier side", member=name)
    return member


def expand(channel: Channel, pipeline: Pipeline, stages: list[Stage], seen_inits: dict[tuple, tuple] | None = None,
           channels: dict[str, Channel] | None = None, member: dict[tuple[str, str], str] | None = None) -> Expansion:
    """Expand one paired channel or raise ``SolveError`` with ``L-PROTO`` failures.  ``channels`` and ``member``
    (``shared_completion``) are needed by a channel that takes part in a shared completion."""
    name = channel.name
    path = f"channels.{name}"
    pp, cp = channel.producer["protocol"], channel.consumer["protocol"]
    if pp.get("kind") != cp.get("kind"):
        _reject(f"{path}.protocol.kind", "producer and consumer protocol kinds disagree")
    kind = pp["kind"]
    wave = pipeline.profile.wave_size
    roles = {r: v["warps"] for s in stages for r, v in s.roles.items()}
    claims = {c["handle"]: c for s in stages for c in s.claims}

    if kind == "mbarrier":
        if _ring_identity(channel.producer) != _ring_identity(channel.consumer) or _ring_identity(channel.producer) is None:
            _reject(f"{path}.ring", "mbarrier endpoint ring declarations disagree")
        if pp.get("release") != cp.get("release"):
            _reject(f"{path}.protocol.release", "mbarrier release declarations disagree")
        depth_ident = _ring_identity(channel.producer)[0]
        result: dict[str, Any] = {}
        for side in ("full", "empty"):
            ps, cs = pp.get(side), cp.get(side)
            spath = f"{path}.protocol.{side}"
            if not isinstance(ps, dict) or not isinstance(cs, dict):
                _reject(spath, "barrier side is missing")
            root = (member or {}).get((name, side))
            if root is None and ("member_of" in ps or "member_of" in cs):
                _reject(spath, "shared-completion sides need the assembly's other channels to expand")
            if root is not None:
                # slots and arrivals are the root's; the member only states its own tile
                ps = dict(channels[root].producer["protocol"][side], tx_bytes=ps.get("tx_bytes", 0))
                cs = dict(channels[root].consumer["protocol"][side], tx_bytes=cs.get("tx_bytes", 0))
            if ps.get("slots") != cs.get("slots"):
                _reject(f"{spath}.slots", "producer and consumer slot handles disagree")
            if ps.get("arrive") != cs.get("arrive"):
                _reject(f"{spath}.arrive", "producer and consumer arrival declarations disagree",
                        producer=ps.get("arrive"), consumer=cs.get("arrive"))
            arr = ps.get("arrive") or {}
            if arr.get("by") not in roles:
                _reject(f"{spath}.arrive.count", "arrive count names a role that is not launched", role=arr.get("by"))
            count = arrive_count(arr.get("count"), roles, wave, f"{spath}.arrive.count")
            members = sorted(m for (m, sd), r in (member or {}).items() if r == name and sd == side)
            tx = []
            for ep, proto_side in ((channel.producer, ps), (channel.consumer, cs)):
                t = proto_side.get("tx_bytes", 0)
                if members or isinstance(t, dict):
                    # a root: one completion stands for its own tile and every direct member's
                    if not isinstance(t, dict) or sorted(t.get("sum") or []) != sorted([name] + members):
                        _reject(f"{spath}.tx_bytes.sum", "root sum must name exactly the root and all direct members",
                                members=members, actual=t.get("sum") if isinstance(t, dict) else t)
                    pick = (lambda c: c.producer) if ep is channel.producer else (lambda c: c.consumer)
                    t = sum(tile_bytes(pick(channels[n] if n != name else channel), f"{spath}.tx_bytes") for n in [name] + members)
                if t == "tile":
                    t = tile_bytes(ep, f"{spath}.tx_bytes")
                if type(t) is not int or t < 0:
                    _reject(f"{spath}.tx_bytes", "transaction bytes must be 'tile' or a non-negative integer")
                tx.append(t)
            if tx[0] != tx[1]:
                _reject(f"{spath}.tx_bytes", "producer and consumer transaction-byte expansions disagree",
                        producer=tx[0], consumer=tx[1])
            _check_slots(ps["slots"], depth_ident, pipeline, claims, f"{spath}.slots")
            result[side] = (ps["slots"], count, tx[0])
        if result["full"][0] == result["empty"][0]:
            _reject(f"{path}.protocol", "full and empty barrier slots may not use the same handle")
        pi, ci = pp.get("init"), cp.get("init")
        if not isinstance(pi, dict) or not isinstance(ci, dict):
            _reject(f"{path}.protocol.init", "mbarrier endpoints require init declarations on both sides")
        if pi.get("materializer") not in ("stage", "dispatch"):
            _reject(f"{path}.protocol.init", "init materializer must be 'stage' or 'dispatch'")
        if pi != ci:
            _reject(f"{path}.protocol.init", "producer and consumer init declarations disagree")
        if pi.get("owner") is None and pi.get("warp") is None:
            _reject(f"{path}.protocol.init", "init requires an owner or a physical initializing warp")
        if seen_inits is not None:
            # several channels may ride one physical ring of slots, but it is initialised once
            key = (result["full"][0], result["empty"][0])
            if key in seen_inits and seen_inits[key][1] != pi:
                _reject(f"channels.{seen_inits[key][0]}.protocol.init",
                        "barrier ring has more than one init owner or materializer", expected=pi, actual=seen_inits[key][1])
            seen_inits.setdefault(key, (name, pi))
        shared = {sd: r for (m, sd), r in (member or {}).items() if m == name}
        return Expansion(name, kind, tx_full=result["full"][2], tx_empty=result["empty"][2],
                         arrive_full=result["full"][1], arrive_empty=result["empty"][1], init_owner=pi.get("owner"),
                         init_materializer=pi["materializer"], slots=(result["full"][0], result["empty"][0]),
                         depth=depth_ident if not isinstance(depth_ident, tuple) else depth_ident[1],
                         detail={"member_of": shared} if shared else {})

    if kind == "call":
        if pp.get("export") != cp.get("export"):
            _reject(f"{path}.protocol.export", "call endpoints name different exports")
        for side, item in (("producer", pp), ("consumer", cp)):
            if not isinstance(item.get("decl"), str) or item.get("decl_sha256") != declaration_digest(item["decl"]):
                _reject(f"{path}.protocol.decl_sha256", f"{side} call declaration hash does not match normalized text")
        exported = channel.consumer_stage.exports.get(cp["export"])
        if exported is None:
            _reject(f"{path}.protocol.export", "consumer stage does not declare the export", export=cp["export"])
        if (normalize_declaration(exported.get("decl", "")), exported.get("decl_sha256")) != \
                (normalize_declaration(cp["decl"]), cp["decl_sha256"]):
            _reject(f"{path}.protocol", "consumer export declaration bytes or hash disagree with the channel")
        # apart from the declarator identifier the caller's trampoline declaration is the export's
        caller = normalize_declaration(pp["decl"]).replace(call_symbol(name), "\0")
        callee = normalize_declaration(exported["decl"]).replace(exported["symbol"], "\0")
        if caller != callee:
            _reject(f"{path}.protocol.decl", "caller and export declarations differ outside the declarator identifier")
        return Expansion(name, kind, call=(exported["symbol"], exported["decl"], exported["decl_sha256"]))

    if kind == "named_barrier":
        if (pp.get("id"), pp.get("count")) != (cp.get("id"), cp.get("count")):
            _reject(f"{path}.protocol", "named-barrier id handle or thread count disagrees")
        decl = pipeline.handles.get(pp.get("id"))
        if decl is None or decl.get("class") != "base" or decl.get("domain") != "named_barrier":
            _reject(f"{path}.protocol", "named-barrier id handle is not declared in the named_barrier domain")
        return Expansion(name, kind, named_barrier=(pp["id"], arrive_count(pp.get("count"), roles, wave, f"{path}.protocol.count")))

    if kind == "counter":
        decl = pipeline.handles.get(pp.get("slot"))
        if decl is None or decl.get("class") != "base" or decl.get("domain") != "gmem_counter":
            _reject(f"{path}.protocol", "counter slot handle is not declared in the gmem_counter domain")
        if channel.producer.get("space") != "gmem":
            _reject(f"{path}.protocol", "counter channels must use gmem space")
        keys = ("slot", "release", "acquire")
        if tuple(pp.get(k) for k in keys) != tuple(cp.get(k) for k in keys) or \
                channel.producer.get("scope") != channel.consumer.get("scope"):
            _reject(f"{path}.protocol", "counter scope, slot or release operation disagree")
        return Expansion(name, kind, counter={k: pp.get(k) for k in keys})

    _reject(f"{path}.protocol.kind", "unsupported protocol kind", actual=kind)


def expand_all(channels: dict[str, Channel], pipeline: Pipeline, stages: list[Stage]) -> list[Expansion]:
    seen: dict[tuple, tuple] = {}
    member = shared_completion(channels)
    return [expand(channels[name], pipeline, stages, seen, channels, member) for name in sorted(channels)]
