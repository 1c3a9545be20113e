"""Builds the decode megakernel example: packs the interpreter and the op packages, links them into one
persistent gfx950 kernel, builds the one-unit control, then swaps ONLY the attention package
(mk.attn -> mk.attn.wide) and relinks.

Counterpart of campaigns/megakernel/port/build.sh in the reference (interpreter + op packages, relink
with another attention).  Output under ``build/``: the ``.plink`` packages, ``pipeline.json``,
``link/...``, ``one_unit.hsaco``, ``swap/{pipeline.json, link/...}`` and ``rebind/{pipeline.json, link/...}`` (the
same packages linked with other opcode numbers, campaigns/megakernel/port/pipelines/rebind-opcode.json)."""
from __future__ import annotations

import json
import shutil
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
BUILD = HERE / "build"
OPS = ["rmsnorm", "qkv", "rope", "attn", "attn_wide", "oproj", "upgate", "down", "lmhead"]


def stage_id(op: str) -> str:
    return "mk." + op.replace("_", ".")


def build(out: Path = BUILD, one_unit: bool = True) -> dict:
    from ...pipec import linker, pack

    out.mkdir(parents=True, exist_ok=True)
    reports = {"mk.interp": pack.pack_stage(HERE / "interp.hip", out / "mk.interp.plink")}
    for op in OPS:
        reports[stage_id(op)] = pack.pack_stage(HERE / f"op_{op}.hip", out / f"{stage_id(op)}.plink")
    (out / "pipeline.json").write_text((HERE / "pipeline.json").read_text())
    link = linker.link(out / "pipeline.json", out / "link")
    control = linker.build_one_unit(out / "pipeline.json", out / "link", out / "one_unit.hsaco") if one_unit else None
    swap = out / "swap"
    swap.mkdir(exist_ok=True)
    for f in out.glob("*.plink"):
        shutil.copy(f, swap / f.name)
    (swap / "pipeline.json").write_text((HERE / "pipeline_attn_wide.json").read_text())
    swapped = linker.link(swap / "pipeline.json", swap / "link")
    rebind = out / "rebind"   # the same packages, other opcode numbers: only the pipeline's forced bindings differ
    rebind.mkdir(exist_ok=True)
    for f in out.glob("*.plink"):
        shutil.copy(f, rebind / f.name)
    (rebind / "pipeline.json").write_text((HERE / "pipeline_rebind_opcodes.json").read_text())
    rebound = linker.link(rebind / "pipeline.json", rebind / "link")
    for d in (out, out / "link", swap, swap / "link", rebind, rebind / "link"):
        for junk in d.glob("*.bc"):
            junk.unlink()
    return {"packages": reports, "link": link, "one_unit": control, "swap": swapped, "rebind": rebound}


def images(out: Path = BUILD) -> dict:
    paths = {"link_json": out / "link" / "link.json", "linked": out / "link" / "pipeline.hsaco", "one_unit": out / "one_unit.hsaco",
             "swap_link_json": out / "swap" / "link" / "link.json", "swap_linked": out / "swap" / "link" / "pipeline.hsaco",
             "rebind_link_json": out / "rebind" / "link" / "link.json", "rebind_linked": out / "rebind" / "link" / "pipeline.hsaco"}
    missing = [str(p) for p in paths.values() if not p.exists()]
    if missing:
        raise FileNotFoundError("megakernel example is not built (run __graft_entry__.build()): " + ", ".join(missing))
    return paths


if __name__ == "__main__":
    sys.path.insert(0, str(HERE.parents[2]))
    from pipelink_amd.stages.megakernel.build import build as _build

    res = _build()
    print(json.dumps({"observed": res["link"]["observed"], "swap_observed": res["swap"]["observed"],
                      "dyn_smem_bytes": res["link"]["dyn_smem_bytes"], "params": res["link"]["params"]}, indent=1))
