"""Builds the one-epilogue-many-producers example: packs the loader (the gs.loader package of the
three-package GEMM example, unchanged), three matrix packages that keep their accumulator in AGPRs, in
VGPRs and in an LDS tile, and ONE epilogue package; links the epilogue against each producer in turn
(the linker generates the accumulator import for each home) and builds each pipeline's one-unit control.
A fourth pipeline, ``wide``, is the same composition at the tile size the accumulation registers allow
(256 x 128 per workgroup, 128 x 64 per wave) that loader waves leave room for: its own loader, matrix and epilogue
packages.  A fifth, ``full``, is the 256 x 256 tile that takes all of a SIMD's registers: a matrix package whose waves
load their own operands, and its epilogue.

Counterpart of examples/one-epilogue-many-producers/build.py in the reference.  Output under
``build/``: the ``.plink`` packages and, per home (and ``wide``), ``<home>/{pipeline.json, link/..., one_unit.hsaco}``."""
from __future__ import annotations

import json
import shutil
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
BUILD = HERE / "build"
HOMES = ("agpr", "vgpr", "lds")
WIDE = "wide"   # the 256 x 128 tile: its own loader, matrix and epilogue packages (accumulator in 128 AGPRs)
FULL = "full"   # the 256 x 256 tile: a matrix package that loads its own operands, and its epilogue (256 AGPRs)
CELLS = HOMES + (WIDE, FULL)
PACKAGES = [("gs.loader", HERE.parent / "gemm_split" / "loader.hip"), ("oe.mma.agpr", HERE / "mma_agpr.hip"),
            ("oe.mma.vgpr", HERE / "mma_vgpr.hip"), ("oe.mma.lds", HERE / "mma_lds.hip"), ("oe.epilogue", HERE / "epilogue.hip"),
            ("oe.loader.wide", HERE / "loader_wide.hip"), ("oe.mma.wide", HERE / "mma_wide.hip"),
            ("oe.epilogue.wide", HERE / "epilogue_wide.hip"),
            ("oe.mma.full", HERE / "mma_full.hip"), ("oe.epilogue.full", HERE / "epilogue_full.hip")]


def _stages_of(cell_name: str) -> tuple[str, ...]:
    if cell_name == WIDE:
        return ("oe.loader.wide", "oe.mma.wide", "oe.epilogue.wide")
    if cell_name == FULL:
        return ("oe.mma.full", "oe.epilogue.full")
    return ("gs.loader", f"oe.mma.{cell_name}", "oe.epilogue")


def build(out: Path = BUILD, one_unit: bool = True) -> dict:
    from ...pipec import linker, pack

    out.mkdir(parents=True, exist_ok=True)
    reports = {sid: pack.pack_stage(src, out / f"{sid}.plink") for sid, src in PACKAGES}
    links, controls = {}, {}
    for home in CELLS:
        cell = out / home
        cell.mkdir(exist_ok=True)
        for sid in _stages_of(home):
            shutil.copy(out / f"{sid}.plink", cell / f"{sid}.plink")
        shutil.copy(HERE / f"pipeline_{home}.json", cell / "pipeline.json")
        links[home] = linker.link(cell / "pipeline.json", cell / "link")
        if one_unit:
            controls[home] = linker.build_one_unit(cell / "pipeline.json", cell / "link", cell / "one_unit.hsaco")
        for junk in list(cell.glob("*.bc")) + list((cell / "link").glob("*.bc")):
            junk.unlink()
    return {"packages": reports, "links": links, "one_unit": controls}


def images(home: str, out: Path = BUILD) -> dict:
    """Paths of one built pipeline; raises if it has not been built."""
    cell = out / home
    paths = {"link_json": cell / "link" / "link.json", "linked": cell / "link" / "pipeline.hsaco", "one_unit": cell / "one_unit.hsaco"}
    missing = [str(p) for p in paths.values() if not p.exists()]
    if missing:
        raise FileNotFoundError("one_epilogue example is not built (run __graft_entry__.build()): " + ", ".join(missing))
    return paths


if __name__ == "__main__":
    sys.path.insert(0, str(HERE.parents[2]))
    from pipelink_amd.stages.one_epilogue.build import build as _build

    res = _build()
    print(json.dumps({h: {"depth": l["bindings"].get("pipelink_gs_depth"), "dyn_smem_bytes": l["dyn_smem_bytes"],
                          "tensor_plans": l["tensor_plans"], "observed": l["observed"]} for h, l in res["links"].items()}, indent=1))
