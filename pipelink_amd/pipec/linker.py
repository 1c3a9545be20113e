"""``pipec link``: packages + ``pipeline.json`` -> one gfx950 code object + ``link.json``.

Phase order as in the reference (pipec/src/pipec2/link.py:1614-1861): load the assembly
(read every ``.plink``, validate manifests, ``validate_assembly``) -> symbol uniqueness
(``L-SYM``) -> pair channels (``L-PAIR``/``L8``) -> expand protocols (``L-PROTO``) -> solve
(``L-OVERLAP``/``L-HANDLE``/``L-TOPO``/``L-REGS``/``L-ALIGN``/``L-PHASE``) -> params layout
(``L-PARAMS``) -> generate stub + dispatch -> device link -> resource audit -> ``link.json``.

Device link on gfx950: the generated translation units are compiled to AMDGPU bitcode with
the flags recorded in the packages' target stamp, ``llvm-link`` joins them with the stage
payloads, everything but the kernel is internalised and the merged module goes once through
``clang -O3 -mcpu=gfx950`` to a code object -- the place where binding stubs, trampolines and
stage exports are inlined into the dispatch kernel (nvJitLink ``-lto`` in the reference,
link.py:593-715).  The one-unit control (``build_one_unit``) ``#include``s the same generated
units and the stage sources in one translation unit and takes the same route
(evaluator/harness/parity/example.py:36-92).  The audit reads VGPR/AGPR/SGPR counts, LDS and
scratch bytes from the code object's metadata notes (``cuobjdump --dump-resource-usage`` in the
reference, link.py:910-919); scratch use is refused because it means a seam was not inlined."""
from __future__ import annotations

import json
import re
import subprocess
from pathlib import Path
from typing import Any

from . import plink
from .channels import expand_all, pair_channels
from .clauses import ClauseFailure, LinkError, PipeLinkError
from .glue import waves_per_simd, KERNEL_SYMBOL, collect_preludes, generate_dispatch, generate_stub, params_layout
from .manifest import Pipeline, Stage, load_pipeline, load_stage_manifest, validate_assembly
from .pack import DEVICE_FLAGS, HIPCC, INCLUDE_DIR, LLVM_BIN
from .tensors import generate_adapters, plan_connections
from .solver import solve


def _fail(clause: str, path: str, message: str, **detail: Any):
    raise LinkError([ClauseFailure(clause, path, message, detail)])


def _run(cmd: list[str], what: str) -> str:
    proc = subprocess.run([str(c) for c in cmd], capture_output=True, text=True)
    if proc.returncode != 0:
        _fail("L-LINK", what, f"{Path(str(cmd[0])).name} failed: {proc.stderr.strip()[-3000:]}")
    return proc.stdout


def load_assembly(pipeline_path: str | Path) -> tuple[Pipeline, list[Stage], dict[str, bytes], dict[str, str]]:
    """Read pipeline.json and every artifact it lists (paths relative to the pipeline file)."""
    pipeline_path = Path(pipeline_path)
    pipeline = load_pipeline(json.loads(pipeline_path.read_text()))
    stages, payloads, hashes = [], {}, {}
    for entry in pipeline.body["stages"]:
        art = (pipeline_path.parent / entry["artifact_path"]).resolve()
        manifest, payload = plink.read(art)
        stage = load_stage_manifest(manifest)
        if stage.id != entry["stage_id"]:
            _fail("L-PAIR", f"pipeline.stages.{entry['stage_id']}", "artifact holds a different stage",
                  actual=stage.id)
        stages.append(stage)
        payloads[stage.id] = payload
        hashes[stage.id] = plink.sha256_hex(art.read_bytes())
    failures = validate_assembly(pipeline, stages)
    if failures:
        raise LinkError(failures)
    return pipeline, stages, payloads, hashes


def check_symbols(stages: list[Stage]) -> None:
    owner: dict[str, str] = {}
    failures = []
    prefixes: dict[str, str] = {}
    for s in stages:
        if s.prefix in prefixes:
            failures.append(ClauseFailure("L-SYM", f"stages.{s.id}.stage.symbol_prefix",
                                          "normalised prefix is shared with another artifact", {"other": prefixes[s.prefix]}))
        prefixes[s.prefix] = s.id
        for sym in (s.manifest.get("symbols") or {}).get("defined_strong", []):
            if sym in owner and not sym.startswith("_Z"):
                failures.append(ClauseFailure("L-SYM", "$.symbols.defined_strong", "is defined by multiple artifacts",
                                              {"symbol": sym, "artifacts": [owner[sym], s.id]}))
            owner.setdefault(sym, s.id)
    if failures:
        raise LinkError(failures)


def plan(pipeline: Pipeline, stages: list[Stage]):
    """Everything up to (not including) code generation; pure Python, no toolchain."""
    check_symbols(stages)
    channels = pair_channels(stages)
    expansions = expand_all(channels, pipeline, stages)
    solution = solve(pipeline, stages, expansions)
    layout = params_layout(pipeline, stages)
    return channels, expansions, solution, layout


def _math_flags(stages: list[Stage]) -> list[str]:
    stamps = {json.dumps((s.manifest["pipelink_abi"]["target"].get("math") or {}).get("flags", DEVICE_FLAGS)) for s in stages}
    if len(stamps) > 1:
        _fail("L-LINK", "pipelink_abi.target.math", "packages were compiled under different math modes")
    return json.loads(next(iter(stamps)))


def host_section(stages: list[Any], layout: dict[str, Any], arch: str) -> dict[str, Any] | None:
    """link.json["host"]: the owner inventory a broker works from (the reference's host section,
    link.py:1301 and host/broker.py:818-830) -- one group per stage that declared a params group:
    its provider's entry points, the record types the provider must report, its caller-owned
    channels and the scalars it reads; plus the stages whose params are plain blobs."""
    groups, scalars, names = [], {}, set()
    entries = {e["stage_id"]: e for e in layout["entries"]}
    for stage in stages:
        host = stage.manifest.get("host")
        if not host:
            continue
        if host["params_group"] in names:
            _fail("L-HOSTCHAN", f"stages.{stage.id}.host.params_group", "two stages declare the same params group",
                  params_group=host["params_group"])
        names.add(host["params_group"])
        for sc in host["scalars"]:
            known = scalars.setdefault(sc["id"], sc)
            if known != sc:
                _fail("L-HOSTCHAN", f"stages.{stage.id}.host.scalars.{sc['name']}", "owners disagree on a shared scalar",
                      expected=known, actual=sc)
        suffix = host["provider"]
        groups.append({"params_group": host["params_group"], "owner": stage.id, "stage_ids": [stage.id],
                       "params": {"bytes": entries[stage.id]["bytes"], "offset": entries[stage.id]["offset"]},
                       "provider": {"symbols": {k: f"pipelink_params_{k}_{suffix}" for k in ("abi", "query", "build", "release")},
                                    "abi_types": host["abi_types"]},
                       "scalars": [sc["id"] for sc in host["scalars"]], "channels": host["channels"]})
    if not groups:
        return None
    owned = {g["owner"] for g in groups}
    return {"protocol": 2, "target": {"profile": arch}, "groups": groups,
            "scalars": [scalars[k] for k in sorted(scalars)],
            "params": {"blobs": [{"stage_id": e["stage_id"], "bytes": e["bytes"]} for e in layout["entries"]
                                 if e["stage_id"] not in owned]}}


def _to_bitcode(source: Path, out: Path, arch: str, flags: list[str], include_dirs: list[Path]) -> None:
    _run([HIPCC, f"--offload-arch={arch}", "-x", "hip", "-fgpu-rdc", "--cuda-device-only", "-emit-llvm", "-c", *flags,
          *[f"-I{d}" for d in [INCLUDE_DIR, *include_dirs]], source, "-o", out], f"compile.{source.name}")


def _finalise(bitcode: Path, hsaco: Path, arch: str) -> None:
    """Internalise everything but the kernel, run the -O3 pipeline once over the merged module
    (clang does not re-optimise IR input on its own), then emit the code object.  Where the
    pipeline's own inliner leaves a call behind (a very large role or export), the module is
    finalised again with every function marked always-inline: a linked kernel has no calls."""
    optimised = bitcode.with_suffix(".opt.bc")
    for forced in ([], ["-force-attribute=alwaysinline"]):
        _run([LLVM_BIN / "opt", "-passes=internalize,globaldce,default<O3>", f"-internalize-public-api-list={KERNEL_SYMBOL}",
              *forced, bitcode, "-o", optimised], "link.optimise")
        _run([LLVM_BIN / "clang", "-x", "ir", "-target", "amdgcn-amd-amdhsa", f"-mcpu={arch}", "-O3", "-nogpulib",
              optimised, "-o", hsaco], "link.codegen")
        text = _run([LLVM_BIN / "llvm-objdump", "-d", "--no-show-raw-insn", hsaco], "audit.disassemble")
        if not seam_calls(text):
            break


_LONG_BRANCH = re.compile(r"s_getpc_b64 (s\[\d+:\d+\])\s*\n\s*s_add_u32 s\d+, s\d+, (?:0x[0-9a-f]+|\d+)\s*\n\s*s_addc_u32 s\d+, s\d+, (?:0x[0-9a-f]+|-?\d+)\s*\n"
                          r"\s*s_setpc_b64 \1")


def seam_calls(disassembly: str) -> int:
    """Calls and returns left in a disassembled image (``llvm-objdump -d --no-show-raw-insn``): ``s_swappc_b64``, and
    ``s_setpc_b64`` unless it is the tail of a long branch -- past +-128 KB the compiler writes a branch as
    ``s_getpc_b64; s_add_u32 <constant>; s_addc_u32; s_setpc_b64``, which leaves the function no more than a
    ``s_branch`` does."""
    text = re.sub(r"[ \t]*//[^\n]*", "", disassembly)
    calls = len(re.findall(r"\bs_swappc_b64\b", text))
    return calls + len(re.findall(r"\bs_setpc_b64\b", text)) - len(_LONG_BRANCH.findall(text))


def audit(hsaco: Path) -> dict[str, int]:
    notes = _run([LLVM_BIN / "llvm-readelf", "--notes", hsaco], "audit.notes")
    out = {}
    for key in ("vgpr_count", "agpr_count", "sgpr_count", "group_segment_fixed_size", "private_segment_fixed_size",
                "vgpr_spill_count", "sgpr_spill_count", "max_flat_workgroup_size"):
        m = re.search(rf"\.{key}:\s+(\d+)", notes)
        out[key] = int(m.group(1)) if m else 0
    text = _run([LLVM_BIN / "llvm-objdump", "-d", "--no-show-raw-insn", hsaco], "audit.disassemble")
    out["calls"] = seam_calls(text)
    out["mfma"] = len(re.findall(r"\bv_mfma_", text))
    out["instructions"] = sum(1 for line in text.splitlines() if re.match(r"\s+[sv]_|\s+ds_|\s+global_|\s+flat_|\s+buffer_|\s+scratch_", line))
    return out


def link(pipeline_path: str | Path, out_dir: str | Path, *, include_dirs: list[str | Path] | None = None,
         codegen: bool = True) -> dict[str, Any]:
    """Link a pipeline.  Returns the ``link.json`` object (also written to ``out_dir``)."""
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    pipeline, stages, payloads, hashes = load_assembly(pipeline_path)
    channels, expansions, solution, layout = plan(pipeline, stages)
    tensor_plans = plan_connections(pipeline, stages)
    arch = pipeline.profile.name
    stub = generate_stub(pipeline, stages, channels, expansions, solution, layout)
    if tensor_plans:
        stub += "\n#include <hip/hip_runtime.h>\n" + generate_adapters(tensor_plans)
    dispatch = generate_dispatch(pipeline, stages, expansions, solution, layout)
    (out_dir / "prelude").mkdir(exist_ok=True)
    for name, text in collect_preludes(stages).items():
        (out_dir / "prelude" / name).write_text(text)
    (out_dir / "stub.hip").write_text(stub)
    (out_dir / "dispatch.hip").write_text(dispatch)
    observed = None
    if codegen:
        flags = _math_flags(stages)
        dirs = [Path(d) for d in (include_dirs or [])]
        parts = []
        for name in ("stub", "dispatch"):
            _to_bitcode(out_dir / f"{name}.hip", out_dir / f"{name}.bc", arch, flags, dirs)
            parts.append(out_dir / f"{name}.bc")
        for sid in pipeline.stage_ids:
            path = out_dir / (sid.replace(".", "_") + ".bc")
            path.write_bytes(payloads[sid])
            parts.append(path)
        _run([LLVM_BIN / "llvm-link", *parts, "-o", out_dir / "linked.bc"], "link.llvm-link")
        _finalise(out_dir / "linked.bc", out_dir / "pipeline.hsaco", arch)
        observed = audit(out_dir / "pipeline.hsaco")
        if observed["calls"]:
            _fail("L-LINK", "observed.calls", "linked kernel still calls across a package seam: an export was not inlined",
                  **observed)
        regs_cap = min(solution.regs_cap, pipeline.profile.regs_per_lane // waves_per_simd(stages))
        if observed["vgpr_count"] > regs_cap:
            _fail("L-REGS", "observed.vgpr_count", "linked kernel needs more registers than the launch leaves per lane",
                  **observed)
    host = host_section(stages, layout, arch)
    result = {
        **({"host": host} if host else {}),
        "kernel_symbol": KERNEL_SYMBOL,
        "threads": solution.threads,
        "regs_cap": solution.regs_cap,
        "dyn_smem_bytes": solution.dyn_smem_bytes,
        "workgroups_per_cu": max(1, min(pipeline.profile.lds_bytes // max(solution.dyn_smem_bytes, 1),
                                        pipeline.profile.max_waves_per_workgroup * 2 // max(solution.launch_warps, 1),
                                        pipeline.profile.regs_per_lane * pipeline.profile.simds_per_cu //
                                        max((observed or {}).get("vgpr_count") or solution.regs_cap, 1) // max(solution.launch_warps, 1)))
        if solution.dyn_smem_bytes else 1,
        "cluster": [1, 1, 1],
        "params": layout,
        "bindings": {k: [v, src] for k, (v, src) in sorted(solution.bindings.items())},
        "variants": {s: v["key"] for s, v in sorted(solution.variants.items())},
        "intervals": {d: [i.to_json_obj() for i in iv] for d, iv in sorted(solution.intervals.items())},
        "roles": {r: {"stage": s, "first_warp": lo, "warps": n} for r, (s, lo, n) in sorted(solution.role_warps.items())},
        "protocol_expansions": [e.to_json_obj() for e in expansions],
        "tensor_plans": [t.to_json_obj() for t in tensor_plans],
        "facts": {k: v for s in stages for k, v in sorted((s.manifest.get("facts") or {}).items())},
        "observed": observed,
        "input_hashes": hashes,
        "generated_hashes": {"stub.hip": plink.sha256_hex(stub.encode()), "dispatch.hip": plink.sha256_hex(dispatch.encode())},
        "solver": {"backend": "pipelink_amd.pipec.solver (deterministic enumeration)", "objective": [t["name"] for t in solution.tiers],
                   "tiers": solution.tiers, "core_clause_precedence": ["L-OVERLAP", "L-HANDLE", "L-TOPO", "L-REGS", "L-ALIGN", "L-PHASE", "L-OWNER", "L-PROTO"]},
        "target": {"profile": arch, "image": "pipeline.hsaco" if codegen else None},
    }
    (out_dir / "link.json").write_text(plink.canonical_dumps(result))
    return result


def build_one_unit(pipeline_path: str | Path, link_dir: str | Path, out: str | Path, *,
                   include_dirs: list[str | Path] | None = None) -> dict[str, int]:
    """The control build: generated glue + every stage source in ONE translation unit, same flags,
    same finalisation.  Needs the stage sources recorded in the packages' provenance."""
    link_dir, out = Path(link_dir), Path(out)
    pipeline, stages, _, _ = load_assembly(pipeline_path)
    flags = _math_flags(stages)
    lines = ["// generated by pipec: one-unit control build", f'#include "{(link_dir / "stub.hip").resolve()}"',
             f'#include "{(link_dir / "dispatch.hip").resolve()}"']
    by_id = {s.id: s for s in stages}
    for sid in pipeline.stage_ids:
        src = Path(by_id[sid].manifest["provenance"]["source"])
        if not src.exists():
            _fail("L-LINK", f"stages.{sid}.provenance.source", "stage source is not available for the one-unit control")
        lines.append(f'#include "{src}"')
    tu = out.with_suffix(".hip")
    tu.write_text("\n".join(lines) + "\n")
    bc = out.with_suffix(".bc")
    _to_bitcode(tu, bc, pipeline.profile.name, flags, [Path(d) for d in (include_dirs or [])])
    _finalise(bc, out, pipeline.profile.name)
    return audit(out)


def explain(err: PipeLinkError) -> str:
    return "pipec: " + str(err)
