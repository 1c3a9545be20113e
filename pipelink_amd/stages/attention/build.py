"""Builds the flash-attention prefill example: packs fa.core and fa.mask.causal, links them into one
gfx950 code object and builds the one-unit control.  The output projection that follows it is the bf16
GEMM of the one-epilogue example (``stages/one_epilogue``), a second linked pipeline.

Counterpart of campaigns/attention/build.py in the reference (core + mask + ... stages, one cell per
mask).  Output under ``build/``: the two ``.plink`` packages, ``pipeline.json``, ``link/...``,
``one_unit.hsaco``."""
from __future__ import annotations

import json
import shutil
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
BUILD = HERE / "build"
STAGES = [("fa.core", "core.hip"), ("fa.mask.causal", "mask_causal.hip"), ("fa.mask.window", "mask_window.hip")]


def build(out: Path = BUILD, one_unit: bool = True) -> dict:
    from ...pipec import linker, pack

    out.mkdir(parents=True, exist_ok=True)
    reports = {sid: pack.pack_stage(HERE / rel, out / f"{sid}.plink") for sid, rel in STAGES}
    (out / "pipeline.json").write_text((HERE / "pipeline.json").read_text())
    link = linker.link(out / "pipeline.json", out / "link")
    control = linker.build_one_unit(out / "pipeline.json", out / "link", out / "one_unit.hsaco") if one_unit else None
    window = out / "window"   # the same core package with the other mask package: only the link is redone
    window.mkdir(exist_ok=True)
    for f in out.glob("*.plink"):
        shutil.copy(f, window / f.name)
    (window / "pipeline.json").write_text((HERE / "pipeline_window.json").read_text())
    windowed = linker.link(window / "pipeline.json", window / "link")
    for junk in list(out.glob("*.bc")) + list((out / "link").glob("*.bc")) + list(window.glob("*.bc")) + list((window / "link").glob("*.bc")):
        junk.unlink()
    return {"packages": reports, "link": link, "one_unit": control, "window": windowed}


def images(out: Path = BUILD) -> dict:
    paths = {"link_json": out / "link" / "link.json", "linked": out / "link" / "pipeline.hsaco", "one_unit": out / "one_unit.hsaco",
             "window_link_json": out / "window" / "link" / "link.json", "window_linked": out / "window" / "link" / "pipeline.hsaco"}
    missing = [str(p) for p in paths.values() if not p.exists()]
    if missing:
        raise FileNotFoundError("attention example is not built (run __graft_entry__.build()): " + ", ".join(missing))
    return paths


if __name__ == "__main__":
    sys.path.insert(0, str(HERE.parents[2]))
    from pipelink_amd.stages.attention.build import build as _build

    res = _build()
    print(json.dumps({"observed": res["link"]["observed"], "dyn_smem_bytes": res["link"]["dyn_smem_bytes"],
                      "threads": res["link"]["threads"]}, indent=1))
