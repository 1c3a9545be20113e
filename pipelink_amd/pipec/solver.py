"""Deterministic resource and role solver in gfx950 units (no SMT solver involved).

Reproduces the decision procedure of pipec/src/pipec2/solve.py:815-1007 by enumeration: the
finite handles (ring depths, register budgets, variants) span a tiny Cartesian product that is
walked best-first in the reference's lexicographic objective order (solve.py:492-517:
``depth:<h>`` max in ``depth_priority`` then name order, ``regs:<h>`` max, high-water of each
physical domain min, ``variant:<stage>`` index min, ``finite:<h>`` min); for each assignment
claims are packed per physical domain (permutation search with first fit for <= 7 claims,
size-descending first fit beyond) honouring alignment, fixed offsets and phase-exclusive
lifetimes; waves tile ``[0, launch_warps)``.  The first feasible assignment is the optimum of
the depth/regs/finite tiers; packing supplies the high-water tier.

Units: ``smem`` bytes of LDS (capacity 160 KiB per workgroup); ``mbarrier`` 16-byte counter
slots inside LDS (they compete with tile bytes for the same capacity, which is why a
two-stage 16 KiB ring solves to 2*16384 + 4*16 = 32832 bytes); ``warp`` = one 64-lane wave;
``gmem_counter`` slots of the pipeline's counter workspace.

Infeasibility is reported like the reference's unsat core: one ``SolveError`` at path
``solve`` whose clause is the first applicable of L-OVERLAP, L-HANDLE, L-TOPO, L-REGS, L-ALIGN,
L-PHASE (solve.py:494-497)."""
from __future__ import annotations

import itertools
from dataclasses import dataclass, field
from typing import Any

from .channels import Expansion
from .clauses import ClauseFailure, SolveError
from .manifest import Pipeline, Stage

PRECEDENCE = ("L-OVERLAP", "L-HANDLE", "L-TOPO", "L-REGS", "L-ALIGN", "L-PHASE", "L-OWNER", "L-PROTO")


@dataclass
class Interval:
    handle: str
    domain: str       # claim (native) domain
    physical: str
    lo: int           # physical units (bytes for smem)
    hi: int
    phase: str        # 'kernel' or a phase name
    stage: str

    def to_json_obj(self) -> dict[str, Any]:
        return {"handle": self.handle, "domain": self.domain, "lo": self.lo, "hi": self.hi, "phase": self.phase}


@dataclass
class Solution:
    bindings: dict[str, tuple[int, str]]                 # handle -> (value, source)
    intervals: dict[str, list[Interval]]                 # physical domain -> placed intervals
    variants: dict[str, dict[str, Any]]                  # stage id -> chosen variant row
    role_warps: dict[str, tuple[str, int, int]]          # role -> (stage id, first warp, warps)
    launch_warps: int
    threads: int
    dyn_smem_bytes: int
    regs_cap: int
    tiers: list[dict[str, Any]] = field(default_factory=list)

    def value(self, handle: str) -> int:
        return self.bindings[handle][0]

    def to_json_obj(self) -> dict[str, Any]:
        return {
            "bindings": {k: [v, src] for k, (v, src) in sorted(self.bindings.items())},
            "intervals": {d: [i.to_json_obj() for i in iv] for d, iv in sorted(self.intervals.items())},
            "variants": {s: v["key"] for s, v in sorted(self.variants.items())},
            "roles": {r: {"stage": s, "first_warp": lo, "warps": n} for r, (s, lo, n) in sorted(self.role_warps.items())},
            "threads": self.threads, "dyn_smem_bytes": self.dyn_smem_bytes, "regs_cap": self.regs_cap,
        }


def _fail(clause: str, message: str, **detail: Any):
    raise SolveError([ClauseFailure(clause, "solve", message, detail)])


def _exclusive(a: str, b: str, pairs: set[frozenset[str]]) -> bool:
    return a != "kernel" and b != "kernel" and a != b and frozenset((a, b)) in pairs


def _align_up(x: int, a: int) -> int:
    return (x + a - 1) // a * a


PIPELINE_SIZED = ("gmem_counter", "opcode")


def _first_fit(order, placed: list[Interval], pairs, capacity):
    """Place claims in the given order; returns (high water, intervals) or None."""
    out = list(placed)
    new = []
    for c in order:
        unit, size, align_bytes = c["unit"], c["size"], c["align"] * c["unit"]
        if c.get("fixed") is not None:
            lo = c["fixed"] * unit
            if lo % align_bytes:
                return None
            candidates = [lo]
        else:
            candidates = sorted({0} | {_align_up(iv.hi, align_bytes) for iv in out})
        pos = None
        for lo in candidates:
            lo = _align_up(lo, align_bytes)
            hi = lo + size
            if all(hi <= iv.lo or lo >= iv.hi or _exclusive(c["phase"], iv.phase, pairs) for iv in out):
                pos = lo
                break
        if pos is None or (capacity is not None and pos + size > capacity):
            return None
        iv = Interval(c["handle"], c["domain"], c["physical"], pos, pos + size, c["phase"], c["stage"])
        out.append(iv)
        new.append(iv)
    return max((iv.hi for iv in out), default=0), new


def _pack(claims: list[dict[str, Any]], pairs, capacity):
    if not claims:
        return 0, []
    base = sorted(claims, key=lambda c: (c.get("fixed") is None, -c["size"], c["handle"]))
    orders = itertools.permutations(base) if len(base) <= 7 else [base]
    best = None
    for order in orders:
        res = _first_fit(order, [], pairs, capacity)
        if res is not None and (best is None or res[0] < best[0]):
            best = res
    return best


def check_topology(stages: list[Stage], pipeline: Pipeline) -> None:
    prof = pipeline.profile
    groups = {s.topology.get("cta_group", {}).get("fixed", 1) for s in stages}
    if len(groups) > 1:
        raise SolveError([ClauseFailure("L-TOPO", "stages.topology.cta_group", "stages disagree on compiled cta_group",
                                        {"values": sorted(groups)})])
    if groups and next(iter(groups)) not in prof.cta_group_legal:
        raise SolveError([ClauseFailure("L-TOPO", "stages.topology.cta_group",
                                        "compiled cta_group is not legal on the target profile")])
    shapes = {tuple(s.topology.get("cluster", {}).get("compiled", [1, 1, 1])) for s in stages}
    if len(shapes) > 1:
        raise SolveError([ClauseFailure("L-TOPO", "stages.topology.cluster.compiled", "compiled cluster shapes disagree",
                                        {"values": sorted(shapes)})])
    if shapes and any(a > b for a, b in zip(next(iter(shapes)), prof.max_cluster)):
        raise SolveError([ClauseFailure("L-TOPO", "stages.topology.cluster.compiled",
                                        "compiled cluster shape exceeds the target profile")])


def solve(pipeline: Pipeline, stages: list[Stage], expansions: list[Expansion] | None = None) -> Solution:
    prof = pipeline.profile
    body = pipeline.body
    handles = pipeline.handles
    check_topology(stages, pipeline)
    pairs = {frozenset(p) for p in body.get("exclusive", [])}
    forced = dict(body.get("forced_bindings") or {})

    # ---- finite handles, best value first ------------------------------------------------
    depth_names = [h for h in body.get("depth_priority", [])]
    depth_names += sorted(n for n, h in handles.items() if h["class"] == "depth" and n not in depth_names)
    regs_names = [h for h in body.get("regs_priority", [])]
    regs_names += sorted(n for n, h in handles.items() if h["class"] == "regs" and n not in regs_names)
    variant_names = sorted(n for n, h in handles.items() if h["class"] == "variant")
    finite = depth_names + regs_names + variant_names

    def candidates(name: str) -> list[int]:
        h = handles[name]
        vals = list(h["values"])
        if name in forced:
            return [forced[name]] if forced[name] in vals else []
        if h["binding"] == "fixed":
            return vals[:1]
        return sorted(vals, reverse=h["class"] != "variant")

    cand = [candidates(n) for n in finite]
    if any(not c for c in cand):
        _fail("L-HANDLE", "no feasible joint binding and placement exists; conflicting set: [forced_bindings]")

    # ---- waves ----------------------------------------------------------------------------
    role_warps: dict[str, tuple[str, int, int]] = {}
    warp_claims = [(s, c) for s in stages for c in s.claims if c["domain"] == "warp"]
    claimed_roles = {r for _, c in warp_claims for r in c.get("roles", [])}
    cursor = 0
    for s, c in sorted(warp_claims, key=lambda sc: (sc[1].get("offset") is None, sc[1].get("offset", 0), sc[1]["handle"])):
        lo = c.get("offset", cursor) if c.get("offset") is not None else cursor
        if lo < cursor:
            _fail("L-TOPO", "no feasible joint binding and placement exists; conflicting set: [warp claims overlap]")
        inner = lo
        for r in c.get("roles", []):
            role_warps[r] = (s.id, inner, s.roles[r]["warps"])
            inner += s.roles[r]["warps"]
        if inner - lo != c["extent"]["const"]:
            _fail("L-TOPO", "no feasible joint binding and placement exists; conflicting set: [warp claim extent]",
                  handle=c["handle"])
        cursor = inner
    for s in stages:
        for r in sorted(s.roles):
            if r not in claimed_roles:
                role_warps[r] = (s.id, cursor, s.roles[r]["warps"])
                cursor += s.roles[r]["warps"]
    launch_warps = cursor
    ranges = sorted((lo, lo + n) for _, lo, n in role_warps.values())
    if launch_warps == 0 or ranges[0][0] != 0 or any(a[1] != b[0] for a, b in zip(ranges, ranges[1:])):
        _fail("L-TOPO", "no feasible joint binding and placement exists; conflicting set: [warps do not tile the launch]")
    if launch_warps > prof.max_waves_per_workgroup:
        _fail("L-TOPO", "no feasible joint binding and placement exists; conflicting set: [launch exceeds the workgroup limit]",
              warps=launch_warps, limit=prof.max_waves_per_workgroup)
    regs_cap = prof.regs_cap(launch_warps)

    # ---- walk assignments best-first ---------------------------------------------------------
    blocked: set[str] = set()
    for combo in itertools.product(*cand):
        values = dict(zip(finite, combo))
        if any(values[n] > regs_cap for n in regs_names):
            blocked.add("L-REGS")
            continue
        # one variant row per stage
        chosen: dict[str, dict[str, Any]] = {}
        ok = True
        for s in stages:
            rows = [v for v in s.variants if all(values.get(k, forced.get(k)) == val for k, val in v["key"].items())]
            if len(rows) != 1:
                ok = False
                break
            chosen[s.id] = rows[0]
        if not ok:
            blocked.add("L-HANDLE")
            continue
        # claims per physical domain
        per_phys: dict[str, list[dict[str, Any]]] = {}
        bad = None
        for s in stages:
            for c in s.claims:
                if c["domain"] in ("regs", "warp"):
                    continue
                phys = prof.physical(c["domain"])
                if phys is None:
                    bad = "L-OVERLAP"
                    break
                extent = c["extent"]["const"] + sum(k * values[h] for h, k in c["extent"].get("per", {}).items())
                if extent <= 0:
                    bad = "L-OVERLAP"
                    break
                life = c.get("lifetime", "kernel")
                per_phys.setdefault(phys[0], []).append({
                    "handle": c["handle"], "domain": c["domain"], "physical": phys[0], "unit": phys[1],
                    "size": extent * phys[1], "align": c.get("align", 1), "fixed": forced.get(c["handle"], c.get("at")),
                    "phase": "kernel" if life == "kernel" else life[6:], "stage": s.id})
        if bad:
            blocked.add(bad)
            continue
        intervals: dict[str, list[Interval]] = {}
        feasible = True
        for phys, claims in sorted(per_phys.items()):
            cap = prof.capacity(phys)
            if phys in PIPELINE_SIZED:  # storage the pipeline sizes, not the chip
                cap = (body.get("domains", {}).get(phys) or {}).get("capacity")
            res = _pack(claims, pairs, cap)
            if res is None:
                feasible = False
                blocked.add("L-OVERLAP")
                break
            intervals[phys] = sorted(res[1], key=lambda iv: (iv.lo, iv.handle))
        if not feasible:
            continue
        bindings: dict[str, tuple[int, str]] = {n: (v, "forced" if n in forced else "solved") for n, v in values.items()}
        for phys, ivs in intervals.items():
            for iv in ivs:
                unit = prof.physical(iv.domain)[1]
                bindings[iv.handle] = (iv.lo // unit, "forced" if iv.handle in forced else "solved")
        for s, c in warp_claims:
            first = min(role_warps[r][1] for r in c.get("roles", [])) if c.get("roles") else 0
            bindings[c["handle"]] = (first, "solved")
        dyn = max((iv.hi for iv in intervals.get("smem", [])), default=0)
        tiers = [{"name": f"depth:{n}", "value": values[n], "status": "proved"} for n in depth_names]
        tiers += [{"name": f"regs:{n}", "value": values[n], "status": "proved"} for n in regs_names]
        tiers += [{"name": f"high_water:{p}", "value": max((iv.hi for iv in ivs), default=0),
                   "status": "proved" if len(per_phys.get(p, [])) <= 7 else "bound_met"}
                  for p, ivs in sorted(intervals.items())]
        return Solution(bindings, intervals, chosen, role_warps, launch_warps, launch_warps * prof.wave_size, dyn,
                        regs_cap, tiers)
    clause = next((c for c in PRECEDENCE if c in blocked), "L-OVERLAP")
    _fail(clause, f"no feasible joint binding and placement exists; conflicting set: {sorted(blocked)}")
