"""Builds the routed-expert FFN forward cell: packs the three owner packages
(mok.framework, mok.gemm, mok.act), links them into one gfx950 code object and builds the
one-unit control next to it.

Counterpart of campaigns/mok/port/build.py in the reference (pack every owner, link the cell,
build ``one_tu.cu`` as the control).  Output layout under ``build/``:
``<stage>.plink``, ``pipeline.json``, ``link/{link.json, pipeline.hsaco, stub.hip, dispatch.hip}``,
``one_unit.hsaco``."""
from __future__ import annotations

import json
import shutil
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
BUILD = HERE / "build"
STAGES = [("mok.framework", "framework/framework.hip"), ("mok.gemm", "gemm/gemm.hip"), ("mok.act", "act_gptoss/act.hip")]


def build(clamp: int = 1, out: Path = BUILD, one_unit: bool = True) -> dict:
    from ...pipec import linker, pack

    out.mkdir(parents=True, exist_ok=True)
    reports = {}
    for stage_id, rel in STAGES:
        reports[stage_id] = pack.pack_stage(HERE / rel, out / f"{stage_id}.plink")
    pipeline = json.loads((HERE / "pipelines_fwd.json").read_text())
    pipeline["pipeline"]["forced_bindings"]["pipelink_mok_clamp"] = clamp
    (out / "pipeline.json").write_text(json.dumps(pipeline, indent=1))
    link = linker.link(out / "pipeline.json", out / "link")
    control = linker.build_one_unit(out / "pipeline.json", out / "link", out / "one_unit.hsaco") if one_unit else None
    for junk in list(out.glob("*.bc")) + list((out / "link").glob("*.bc")):
        junk.unlink()
    return {"packages": reports, "link": link, "one_unit": control}


def images(out: Path = BUILD) -> dict:
    """Paths of the built cell; raises if it has not been built."""
    paths = {"link_json": out / "link" / "link.json", "linked": out / "link" / "pipeline.hsaco",
             "one_unit": out / "one_unit.hsaco"}
    missing = [str(p) for p in paths.values() if not p.exists()]
    if missing:
        raise FileNotFoundError("MoK cell is not built (run __graft_entry__.build()): " + ", ".join(missing))
    return paths


if __name__ == "__main__":
    sys.path.insert(0, str(HERE.parents[2]))
    from pipelink_amd.stages.mok.build import build as _build

    res = _build()
    print(json.dumps({"observed": res["link"]["observed"], "one_unit": res["one_unit"],
                      "dyn_smem_bytes": res["link"]["dyn_smem_bytes"], "threads": res["link"]["threads"]}, indent=1))
