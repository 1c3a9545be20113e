"""Builds the three-package GEMM example C = GELU(A . B + bias): packs gs.loader, gs.mma and
gs.epilogue, links them into one gfx950 code object (ring depth chosen by the link) and builds
the one-unit control next to it.

Counterpart of examples/hopper-gemm-split/build.py and examples/ring-pipeline/build.py:20-40 in
the reference (pack the stages, write the pipeline with its depth handle, link).  Output under
``build/``: ``<stage>.plink``, ``pipeline.json``, ``link/{link.json, pipeline.hsaco, ...}``,
``one_unit.hsaco``."""
from __future__ import annotations

import json
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
BUILD = HERE / "build"
STAGES = [("gs.loader", "loader.hip"), ("gs.mma", "mma.hip"), ("gs.epilogue", "epilogue.hip")]


def build(out: Path = BUILD, depth: int | None = None, one_unit: bool = True) -> dict:
    """`depth` forces the ring depth (2 or 4); None lets the solver take the deepest that fits."""
    from ...pipec import linker, pack

    out.mkdir(parents=True, exist_ok=True)
    reports = {}
    for stage_id, rel in STAGES:
        reports[stage_id] = pack.pack_stage(HERE / rel, out / f"{stage_id}.plink")
    pipeline = json.loads((HERE / "pipeline.json").read_text())
    if depth is not None:
        pipeline["pipeline"]["forced_bindings"]["pipelink_gs_depth"] = depth
    (out / "pipeline.json").write_text(json.dumps(pipeline, indent=1))
    link = linker.link(out / "pipeline.json", out / "link")
    control = linker.build_one_unit(out / "pipeline.json", out / "link", out / "one_unit.hsaco") if one_unit else None
    for junk in list(out.glob("*.bc")) + list((out / "link").glob("*.bc")):
        junk.unlink()
    return {"packages": reports, "link": link, "one_unit": control}


def images(out: Path = BUILD) -> dict:
    """Paths of the built example; raises if it has not been built."""
    paths = {"link_json": out / "link" / "link.json", "linked": out / "link" / "pipeline.hsaco",
             "one_unit": out / "one_unit.hsaco"}
    missing = [str(p) for p in paths.values() if not p.exists()]
    if missing:
        raise FileNotFoundError("gemm_split example is not built (run __graft_entry__.build()): " + ", ".join(missing))
    return paths


if __name__ == "__main__":
    sys.path.insert(0, str(HERE.parents[2]))
    from pipelink_amd.stages.gemm_split.build import build as _build

    res = _build()
    print(json.dumps({"observed": res["link"]["observed"], "one_unit": res["one_unit"],
                      "dyn_smem_bytes": res["link"]["dyn_smem_bytes"], "threads": res["link"]["threads"],
                      "bindings": res["link"].get("bindings")}, indent=1))
