"""``pipec`` command line: pack | inspect | link | launch | clauses.

Same verbs and failure format as the reference's ``pipec2`` (pipec/src/pipec2/cli.py:193-276):
a rejected command exits 1 and prints ``pipec: [ID] path: message; [ID] ...`` on stderr."""
from __future__ import annotations

import argparse
import json
import sys

from . import plink
from .clauses import CLAUSE_PHASES, CLAUSES, PipeLinkError


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(prog="pipec")
    sub = ap.add_subparsers(dest="cmd", required=True)
    p = sub.add_parser("pack", help="compile one annotated HIP stage source into a .plink")
    p.add_argument("source")
    p.add_argument("-o", "--out", required=True)
    p.add_argument("-I", dest="include", action="append", default=[])
    p.add_argument("--profile", default="gfx950")
    p = sub.add_parser("inspect", help="print the manifest of a .plink")
    p.add_argument("artifact")
    p = sub.add_parser("link", help="link a pipeline.json into one code object + link.json")
    p.add_argument("pipeline")
    p.add_argument("--out-dir", required=True)
    p.add_argument("--plan-only", action="store_true", help="check contracts and solve, generate glue, skip code generation")
    p.add_argument("--one-unit", help="also build the one-unit control image at this path")
    p = sub.add_parser("launch", help="launch a linked image once (host-less route)")
    p.add_argument("link_json")
    p.add_argument("--grid", metavar="X[,Y,Z]", help="workgroups; the block size comes from the link")
    p.add_argument("--buffer", action="append", default=[], metavar="NAME=SPEC", help="FILE.npy or SHAPE:DTYPE, e.g. out=64x64:float32")
    p.add_argument("--params", metavar="PY_FILE:FUNCTION", help="Python builder: device addresses -> stage params bytes")
    p.add_argument("--blob", action="append", default=[], metavar="STAGE_ID=PATH", help="already-built stage params blob")
    p.add_argument("--output", action="append", default=[], metavar="NAME=FILE.npy", help="save a buffer after the launch")
    p.add_argument("--provider", action="append", default=[], metavar="GROUP=SO", help="owner provider shared object keyed by params group")
    p.add_argument("--host-inputs", help="caller scalar and buffer JSON for a link with a host section")
    p.add_argument("--device", type=int, default=0)
    p = sub.add_parser("clauses", help="list the named diagnostics")
    p.add_argument("--json", action="store_true")
    args = ap.parse_args(argv)
    try:
        if args.cmd == "pack":
            from .pack import pack_stage
            print(json.dumps(pack_stage(args.source, args.out, include_dirs=args.include, profile=args.profile), indent=1))
        elif args.cmd == "inspect":
            manifest, payload = plink.read(args.artifact)
            manifest.setdefault("payload", {})["size"] = len(payload)
            for pre in (manifest.get("hints") or {}).get("preludes", []):
                pre["text"] = f"<{len(pre['text'])} bytes>"
            print(json.dumps(manifest, indent=1, sort_keys=True))
        elif args.cmd == "link":
            from . import linker
            res = linker.link(args.pipeline, args.out_dir, codegen=not args.plan_only)
            if args.one_unit:
                res["one_unit"] = linker.build_one_unit(args.pipeline, args.out_dir, args.one_unit)
            print(json.dumps({k: res[k] for k in ("threads", "dyn_smem_bytes", "bindings", "params", "observed") if k in res}, indent=1))
        elif args.cmd == "launch":
            from . import launcher

            def pairs(items):
                return dict(item.split("=", 1) for item in items)
            grid = tuple(int(v) for v in args.grid.split(",")) if args.grid else None
            print(json.dumps(launcher.launch(args.link_json, grid=grid, buffers=pairs(args.buffer), params=args.params,
                                             blobs=pairs(args.blob), outputs=pairs(args.output), providers=pairs(args.provider),
                                             host_inputs=args.host_inputs, device=args.device), indent=1))
        elif args.cmd == "clauses":
            rows = [{"id": c, "phase": CLAUSE_PHASES[c], "description": CLAUSES[c]} for c in sorted(CLAUSES)]
            print(json.dumps(rows, indent=1) if args.json else "\n".join(f"{r['id']:12s} {r['phase']:9s} {r['description']}" for r in rows))
    except PipeLinkError as err:
        print(f"pipec: {err}", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
