"""Tensor connections: handing a producer's tile to a consumer that does not know where it lives.

A producer package exports a tensor (``PL_EXPORT_TENSOR``): its logical identity (result name, dtype,
per-participant shape) and its placement -- the *home* (``agpr``, ``vgpr`` or ``lds``) and the layout in
that home.  A consumer package imports one (``PL_IMPORT_TENSOR``): the same identity, the layout it wants
the elements in, and the name of a function it calls to get them.  The pipeline connects an export to an
import (``tensor_connections``); the linker checks the identities (``T-CONTRACT``), picks a route
(``T-PLAN`` if none exists) and *generates* the function, together with ``<fn>_ready()``,
``<fn>_done()`` and ``<fn>_block()`` (one 32 x 32 block at a time), into the binding stubs.  The consumer's source never changes with the producer's home.

The reference plans such routes with a model of typed transport primitives and a bounded search
(pipec/src/pipec2/tensor/plan.py:557 ``ConnectionPlanner``, lowering in tensor/lower.py:679; contract in
docs/reference/tensor-imports.md:40-142).  On gfx950 the homes an MFMA accumulator can have are three and
the primitives that read them are fixed, so the planner here is a route table:

    home   layout        route             what the generated function does per element
    vgpr   mfma32x32c    register_copy     a move the compiler folds away
    agpr   mfma32x32c    accvgpr_receipt   v_accvgpr_read_b32 from the accumulator register
    lds    row_major     lds_load          ds_read_b32 at row * pitch + 4 * column of the wave's tile

``mfma32x32c`` is the C/D fragment layout of the 32x32 MFMAs for a tile of rows x cols split into 32 x 32
blocks [i][j]: element (block i, block j, register r, lane l) is row 32 i + 8 (r / 4) + 4 (l / 32) + r % 4,
column 32 j + l % 32; in memory order it is word (i * (cols / 32) + j) * 16 + r of the lane's frame.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from .clauses import CLAUSES, ClauseFailure, LinkError, register_clause
from .manifest import Pipeline, Stage

for _cid, _desc in (("T-PLAN", "a transport route exists for every tensor connection"),):
    if _cid not in CLAUSES:
        register_clause(_cid, phase="link", description=_desc)

ROUTES = {("vgpr", "mfma32x32c"): "register_copy", ("agpr", "mfma32x32c"): "accvgpr_receipt", ("lds", "row_major"): "lds_load"}
WANTED_LAYOUTS = ("mfma32x32c",)
_IDENTITY = ("result", "dtype", "shape")


@dataclass(frozen=True)
class TensorPlan:
    name: str
    producer: str
    consumer: str
    export: dict[str, Any]
    imported: dict[str, Any]
    route: str

    def to_json_obj(self) -> dict[str, Any]:
        return {"name": self.name, "producer": self.producer, "consumer": self.consumer, "export": self.export["name"],
                "import": self.imported["name"], "function": self.imported["fn"], "home": self.export["home"],
                "route": self.route}


# What a consumer may promise about the place it calls an import from: a closed vocabulary (the generated function
# relies on exactly these; docs/reference/tensor-imports.md:96-118 in the reference).
SITE_GUARANTEES = ("enter_once", "converged", "full_warps", "no_early_return")
LEND_BINDINGS = ("fixed", "relocatable")


def check_stage_tensor(tensor: Any, schema_admits_tensor: bool) -> list[tuple[str, str, dict[str, Any]]]:
    """Load-time checks of a stage manifest's ``tensor`` section; returns (path, message, detail) per T-CONTRACT
    failure (the reference's load_stage_tensor, pipec/src/pipec2/tensor/contracts.py, reports the same paths).

    Besides the export and import records the planner reads, a section may carry
      ``sites``           [{name, role, guarantees: [...]}]: where the stage calls its imports from, and what it
                          promises there -- tokens of SITE_GUARANTEES only;
      ``imports[].lends`` [{name, binding, location: {handle, base}, ...}]: resources the consumer lends to the
                          generated function (scratch memory, a barrier, registers); names are local to the stage
                          and unique across its imports, and a relocatable lend names the handle the linker places
                          even when it also states a base.
    The route table of this linker needs nothing lent, so no stage here declares lends; they are part of the
    manifest format and are checked where present."""
    out: list[tuple[str, str, dict[str, Any]]] = []
    if not schema_admits_tensor:
        return [("$.tensor", "this stage schema has no tensor section", {})]
    if not isinstance(tensor, dict):
        return [("$.tensor", "tensor section must be an object", {})]
    for kind in ("exports", "imports", "sites"):
        if not isinstance(tensor.get(kind, []), list):
            out.append((f"$.tensor.{kind}", f"{kind} must be an array", {}))
    site_names: set[str] = set()
    for i, site in enumerate(tensor.get("sites", []) if isinstance(tensor.get("sites", []), list) else []):
        path = f"$.tensor.sites[{i}]"
        if not isinstance(site, dict) or not isinstance(site.get("name"), str):
            out.append((path, "a site is an object with a name", {}))
            continue
        if site["name"] in site_names:
            out.append((f"{path}.name", "site name is declared twice", {"name": site["name"]}))
        site_names.add(site["name"])
        promised = site.get("guarantees", [])
        if not isinstance(promised, list):
            out.append((f"{path}.guarantees", "guarantees must be an array", {}))
            continue
        for j, token in enumerate(promised):
            if token not in SITE_GUARANTEES:
                out.append((f"{path}.guarantees[{j}]", "unknown site guarantee", {"allowed": list(SITE_GUARANTEES), "actual": token}))
            elif token in promised[:j]:
                out.append((f"{path}.guarantees[{j}]", "site guarantee is listed twice", {"actual": token}))
    lent: set[str] = set()
    for i, imp in enumerate(tensor.get("imports", []) if isinstance(tensor.get("imports", []), list) else []):
        path = f"$.tensor.imports[{i}]"
        if not isinstance(imp, dict) or not isinstance(imp.get("name"), str):
            out.append((path, "an import is an object with a name", {}))
            continue
        for j, site in enumerate(imp.get("sites", []) or []):
            if site not in site_names:
                out.append((f"{path}.sites[{j}]", "import names a site the stage does not declare", {"actual": site}))
        lends = imp.get("lends", [])
        if not isinstance(lends, list):
            out.append((f"{path}.lends", "lends must be an array", {}))
            continue
        for j, lend in enumerate(lends):
            lp = f"{path}.lends[{j}]"
            if not isinstance(lend, dict) or not isinstance(lend.get("name"), str):
                out.append((lp, "a lend is an object with a name", {}))
                continue
            if lend["name"] in lent:
                out.append((f"{lp}.name", "two lends publish the same stage-local name", {"name": lend["name"]}))
            lent.add(lend["name"])
            if lend.get("binding") not in LEND_BINDINGS:
                out.append((f"{lp}.binding", "lend binding must be fixed or relocatable", {"actual": lend.get("binding")}))
            where = lend.get("location")
            if not isinstance(where, dict) or set(where) != {"handle", "base"}:
                out.append((f"{lp}.location", "lend location must give handle and base", {}))
            elif lend.get("binding") == "relocatable" and not isinstance(where["handle"], str):
                out.append((f"{lp}.location.handle", "a relocatable lend names the handle the linker places", {}))
            elif where["handle"] is None and where["base"] is None:
                out.append((f"{lp}.location", "a fixed lend states a handle or a base", {}))
    return out


def _records(stage: Stage, kind: str) -> dict[str, dict[str, Any]]:
    return {r["name"]: r for r in (stage.manifest.get("tensor") or {}).get(kind, [])}


def plan_connections(pipeline: Pipeline, stages: list[Stage]) -> list[TensorPlan]:
    """One plan per entry of ``pipeline.tensor_connections``; raises LinkError with T-CONTRACT / T-PLAN."""
    by_id = {s.id: s for s in stages}
    failures: list[ClauseFailure] = []
    plans: list[TensorPlan] = []
    seen_imports: set[tuple[str, str]] = set()
    for conn in pipeline.body.get("tensor_connections", []) or []:
        path = f"pipeline.tensor_connections.{conn.get('name', '?')}"

        def bad(clause: str, message: str, **detail: Any) -> None:
            failures.append(ClauseFailure(clause, path, message, detail))

        prod, cons = by_id.get(conn.get("producer")), by_id.get(conn.get("consumer"))
        if prod is None or cons is None:
            bad("T-CONTRACT", "connection names a stage that is not in the pipeline")
            continue
        exp = _records(prod, "exports").get(conn.get("export"))
        imp = _records(cons, "imports").get(conn.get("import"))
        if exp is None or imp is None:
            bad("T-CONTRACT", "connection names an export or import its stage does not declare",
                export=conn.get("export"), imported=conn.get("import"))
            continue
        if (cons.id, imp["name"]) in seen_imports:
            bad("T-CONTRACT", "an import is fed by more than one connection")
            continue
        seen_imports.add((cons.id, imp["name"]))
        differing = [k for k in _IDENTITY if exp.get(k) != imp.get(k)]
        if differing:
            bad("T-CONTRACT", "exported and imported tensor identities disagree",
                fields=differing, exported={k: exp.get(k) for k in differing}, imported={k: imp.get(k) for k in differing})
            continue
        rows, cols = exp["shape"]
        if imp["layout"] not in WANTED_LAYOUTS or rows % 32 or cols % 32:
            bad("T-PLAN", "no transport route delivers the demanded layout", wanted=imp["layout"], shape=exp["shape"])
            continue
        route = ROUTES.get((exp["home"], exp["layout"]))
        if route is None:
            bad("T-PLAN", "no transport route reads this home and layout", home=exp["home"], layout=exp["layout"])
            continue
        if route == "lds_load" and (exp.get("row_pitch_bytes", 0) < cols * 4 or exp["row_pitch_bytes"] % 4):
            bad("T-CONTRACT", "row pitch of the exported tile is smaller than a row or not a multiple of 4")
            continue
        plans.append(TensorPlan(conn["name"], prod.id, cons.id, exp, imp, route))
    declared = {(s.id, name) for s in stages for name in _records(s, "imports")}
    for sid, name in sorted(declared - seen_imports):
        failures.append(ClauseFailure("T-CONTRACT", f"stages.{sid}.tensor.imports.{name}",
                                      "import is not fed by any tensor connection"))
    if failures:
        raise LinkError(failures)
    return plans


def generate_adapters(plans: list[TensorPlan]) -> str:
    """HIP source of the generated import functions (appended to the binding stubs)."""
    out: list[str] = []
    for p in plans:
        fn = p.imported["fn"]
        rows, cols = p.export["shape"]
        bi, bj = rows // 32, cols // 32
        out += [f"// tensor connection {p.name}: {p.producer}.{p.export['name']} ({p.export['home']}, {p.export['layout']}) -> "
                f"{p.consumer}.{p.imported['name']} ({p.imported['layout']}); route {p.route}",
                f'extern "C" __device__ __attribute__((always_inline)) void {fn}_ready() {{ asm volatile("" ::: "memory"); }}']
        if p.route == "lds_load":
            out.append(f'extern "C" __device__ __attribute__((always_inline)) void {fn}_done() {{ '
                       '__builtin_amdgcn_s_waitcnt(0xC07F); asm volatile("" ::: "memory"); }  // the tile has been read')
        else:
            out.append(f'extern "C" __device__ __attribute__((always_inline)) void {fn}_done() {{ asm volatile("" ::: "memory"); }}')
        out.append(f'extern "C" __device__ __attribute__((always_inline)) void {fn}(const void* source, float* dest) {{')
        if p.route == "register_copy":
            out += ["  const float* frame = static_cast<const float*>(source);", "#pragma unroll",
                    f"  for (int k = 0; k < {bi * bj * 16}; ++k) dest[k] = frame[k];"]
        elif p.route == "accvgpr_receipt":
            out += ["  const float* frame = static_cast<const float*>(source);", "#pragma unroll",
                    f"  for (int k = 0; k < {bi * bj * 16}; ++k) {{",
                    "    float v;",
                    '    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(frame[k]));',
                    "    dest[k] = v;", "  }"]
        else:
            pitch = p.export["row_pitch_bytes"]
            out += ["  const unsigned char* tile = static_cast<const unsigned char*>(source);",
                    "  const int lane = threadIdx.x & 63;", "#pragma unroll",
                    f"  for (int i = 0; i < {bi}; ++i)", "#pragma unroll",
                    f"    for (int j = 0; j < {bj}; ++j)", "#pragma unroll",
                    "      for (int r = 0; r < 16; ++r) {",
                    "        const int row = 32 * i + 8 * (r / 4) + 4 * (lane >> 5) + r % 4, col = 32 * j + (lane & 31);",
                    f"        dest[(i * {bj} + j) * 16 + r] = *reinterpret_cast<const float*>(tile + row * {pitch} + col * 4);",
                    "      }"]
        out += ["}"]
        # the same, one 32 x 32 block (16 elements per lane, block = i * (cols / 32) + j) at a time: for a consumer whose
        # registers do not hold the whole tensor
        out.append(f'extern "C" __device__ __attribute__((always_inline)) void {fn}_block(const void* source, int block, float* dest) {{')
        if p.route == "register_copy":
            out += ["  const float* frame = static_cast<const float*>(source) + block * 16;", "#pragma unroll",
                    "  for (int k = 0; k < 16; ++k) dest[k] = frame[k];"]
        elif p.route == "accvgpr_receipt":
            out += ["  const float* frame = static_cast<const float*>(source) + block * 16;", "#pragma unroll",
                    "  for (int k = 0; k < 16; ++k) {", "    float v;",
                    '    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(frame[k]));', "    dest[k] = v;", "  }"]
        else:
            out += ["  const unsigned char* tile = static_cast<const unsigned char*>(source);",
                    f"  const int lane = threadIdx.x & 63, i = block / {bj}, j = block % {bj};", "#pragma unroll",
                    "  for (int r = 0; r < 16; ++r) {",
                    "    const int row = 32 * i + 8 * (r / 4) + 4 * (lane >> 5) + r % 4, col = 32 * j + (lane & 31);",
                    f"    dest[r] = *reinterpret_cast<const float*>(tile + row * {pitch} + col * 4);", "  }"]
        out += ["}", ""]
    return "\n".join(out)
