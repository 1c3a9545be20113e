"""ISA gate: is the linked kernel the same machine code as the one-unit control?

The reference answers this on SASS (``evaluator/gates/normalization.py:10-51`` extracts the
instruction text per function and renames registers to first-use ordinals;
``evaluator/gates/comparison.py:43-115`` walks the two streams in order, tolerates only
individually listed integer operands and counts the local-memory / shared-memory / call
classes).  Here the same questions are asked of two gfx950 code objects, on the text of
``llvm-objdump -d --no-show-raw-insn``:

* registers are renamed per class (``v``, ``a``, ``s``; a range ``v[4:7]`` is named by its
  first register and keeps its width), ``vcc``/``exec``/``m0``/``scc``/``null``/``off`` and
  hardware-register names stay literal; branch targets lose their address;
* the ordered comparison reports the same six checks as the reference, and lists every operand
  that differs (integer operands are "enumerated deltas", anything else fails the check);
* the class counts are ``scratch_`` (AMD's local memory: must be zero), ``ds_`` (LDS),
  ``buffer_``/``global_`` (memory), ``v_mfma`` and calls (``s_swappc_b64``/``s_setpc_b64``:
  must be zero, everything is inlined), ``s_barrier`` and ``s_waitcnt``.

Two compilations of different IR modules are in general not instruction-identical on AMDGPU
(the one -O3 pipeline sees the packages' code in a different order), so the ordered checks
are reported, not enforced; what the link gate enforces is in ``GATE_CHECKS``: same functions,
nothing left as a call, the same number of instructions in every class that moves data or feeds
the matrix pipe, the same register and LDS footprint, and at most ``SPILL_LIMIT_BYTES`` of
scratch on either side (which values the register allocator parks there is its own choice per
module: one side may hold a dword more than the other).
"""
from __future__ import annotations

import re
import subprocess
from collections import Counter
from pathlib import Path
from typing import Any

LLVM_BIN = Path("/opt/rocm/lib/llvm/bin")

FUNCTION = re.compile(r"^[0-9a-f]+ <(.+)>:\s*$")
LABEL = re.compile(r"<[^>]*>")
REGISTER = re.compile(r"(?<![A-Za-z0-9_.])(v|a|s)(?:(\d+)|\[(\d+):(\d+)\])(?![A-Za-z0-9_])")
RENAMED = re.compile(r"(?<![A-Za-z0-9_])[vas]<\d+(?:x\d+)?>")
IMMEDIATE = re.compile(r"-?(?:0x[0-9a-fA-F]+|[0-9]+)\Z")
CLASSES = ("scratch_", "ds_", "buffer_", "global_", "v_mfma", "s_barrier", "s_waitcnt", "call")
GATE_CHECKS = ("function_identity_order_equal", "no_calls", "data_path_class_counts_equal", "register_footprint_equal",
               "spills_small")
DATA_PATH = ("ds_", "buffer_", "global_", "v_mfma", "s_barrier", "call")
SPILL_LIMIT_BYTES = 64  # a handful of dwords the register allocator parks in scratch; it may park one more on one side


def disassemble(hsaco: str | Path) -> str:
    return subprocess.run([str(LLVM_BIN / "llvm-objdump"), "-d", "--no-show-raw-insn", str(hsaco)], check=True,
                          capture_output=True, text=True).stdout


def resources(hsaco: str | Path) -> dict[str, int]:
    notes = subprocess.run([str(LLVM_BIN / "llvm-readelf"), "--notes", str(hsaco)], check=True, capture_output=True,
                           text=True).stdout
    out = {}
    for key in ("vgpr_count", "agpr_count", "sgpr_count", "group_segment_fixed_size", "private_segment_fixed_size"):
        m = re.search(rf"\.{key}:\s+(\d+)", notes)
        out[key] = int(m.group(1)) if m else 0
    return out


def sections(text: str) -> list[tuple[str, list[str]]]:
    """[(function, [instruction text ...])] in file order; comments and addresses dropped."""
    result: list[tuple[str, list[str]]] = []
    name, body = None, []
    for line in text.splitlines():
        head = FUNCTION.match(line)
        if head:
            if name is not None:
                result.append((name, body))
            name, body = head.group(1), []
            continue
        if name is None or not line.startswith(("\t", " ")):
            continue
        instruction = line.split("//")[0].strip()
        if instruction:
            body.append(LABEL.sub("<label>", instruction))
    if name is not None:
        result.append((name, body))
    return result


def canonicalize(body: list[str]) -> list[str]:
    """Rename registers to first-use ordinals, one numbering per class."""
    names: dict[tuple[str, int], int] = {}
    next_id = Counter()

    def rename(m: re.Match[str]) -> str:
        kind = m.group(1)
        first = int(m.group(2) if m.group(2) is not None else m.group(3))
        width = 1 if m.group(2) is not None else int(m.group(4)) - first + 1
        ordinals = []
        for reg in range(first, first + width):
            if (kind, reg) not in names:
                names[(kind, reg)] = next_id[kind]
                next_id[kind] += 1
            ordinals.append(names[(kind, reg)])
        return f"{kind}<{ordinals[0]}>" if width == 1 else f"{kind}<{ordinals[0]}x{width}>"

    return [REGISTER.sub(rename, line) for line in body]


def instruction_parts(line: str) -> tuple[str, list[str]]:
    """(opcode with its suffixes, operands); modifiers after the last operand stay with it."""
    opcode, _, rest = line.partition(" ")
    operands, depth, start = [], 0, 0
    for i, ch in enumerate(rest):
        if ch in "[(":
            depth += 1
        elif ch in "])":
            depth -= 1
        elif ch == "," and depth == 0:
            operands.append(rest[start:i].strip())
            start = i + 1
    if rest[start:].strip():
        operands.append(rest[start:].strip())
    return opcode, operands


def _class_counts(body: list[str]) -> dict[str, int]:
    ops = Counter(line.split(" ", 1)[0] for line in body)
    out = {}
    for cls in CLASSES:
        if cls == "call":
            out[cls] = ops["s_swappc_b64"] + ops["s_setpc_b64"]
        else:
            out[cls] = sum(n for op, n in ops.items() if op.startswith(cls))
    return out


def compare_streams(control: list[tuple[str, list[str]]], linked: list[tuple[str, list[str]]]) -> dict[str, Any]:
    """Ordered comparison of two canonicalised streams plus the class counts of each."""
    checks = {
        "function_identity_order_equal": [n for n, _ in control] == [n for n, _ in linked],
        "instruction_counts_equal": [len(b) for _, b in control] == [len(b) for _, b in linked],
        "opcode_sequence_including_modifiers_equal": True,
        "register_relationships_equal_under_frozen_renaming": True,
        "all_non_enumerated_instruction_text_equal": True,
    }
    memory = {label: [{"function": name, "counts": _class_counts(body)} for name, body in stream]
              for label, stream in (("control", control), ("linked", linked))}
    checks["memory_op_class_counts_equal"] = memory["control"] == memory["linked"]
    checks["no_calls"] = all(row["counts"]["call"] == 0 for rows in memory.values() for row in rows)
    checks["no_local_traffic"] = all(row["counts"]["scratch_"] == 0 for rows in memory.values() for row in rows)
    checks["data_path_class_counts_equal"] = ([[r["counts"][c] for c in DATA_PATH] for r in memory["control"]]
                                              == [[r["counts"][c] for c in DATA_PATH] for r in memory["linked"]])
    deltas = []
    for (function, left), (_, right) in zip(control, linked):
        if len(left) != len(right):
            # without equal lengths a positional walk says nothing about the rest
            checks["opcode_sequence_including_modifiers_equal"] = False
            checks["register_relationships_equal_under_frozen_renaming"] = False
            checks["all_non_enumerated_instruction_text_equal"] = False
            continue
        for index, (old, new) in enumerate(zip(left, right)):
            old_op, old_operands = instruction_parts(old)
            new_op, new_operands = instruction_parts(new)
            checks["opcode_sequence_including_modifiers_equal"] &= old_op == new_op
            checks["register_relationships_equal_under_frozen_renaming"] &= RENAMED.findall(old) == RENAMED.findall(new)
            same_text = old_op == new_op and len(old_operands) == len(new_operands)
            for k, (a, b) in enumerate(zip(old_operands, new_operands)):
                if a == b:
                    continue
                integer = bool(IMMEDIATE.fullmatch(a) and IMMEDIATE.fullmatch(b))
                deltas.append({"function": function, "instruction_index_zero_based": index, "operand_index_zero_based": k,
                               "control_instruction": old, "linked_instruction": new, "old_value": a, "new_value": b,
                               "integer_operand_encoding": integer})
                same_text &= integer
            checks["all_non_enumerated_instruction_text_equal"] &= same_text
    return {
        "checks": checks,
        "seam_structure_clean": all(checks.values()),
        "instruction_counts": {label: sum(len(b) for _, b in stream) for label, stream in (("control", control), ("linked", linked))},
        "memory_op_class_counts": memory,
        "deltas": deltas,
    }


def opcode_histogram_delta(control: list[tuple[str, list[str]]], linked: list[tuple[str, list[str]]]) -> dict[str, list[int]]:
    """{opcode: [count in control, count in linked]} for every opcode whose counts differ."""
    def hist(stream):
        return Counter(line.split(" ", 1)[0] for _, body in stream for line in body)
    a, b = hist(control), hist(linked)
    return {op: [a[op], b[op]] for op in sorted(set(a) | set(b)) if a[op] != b[op]}


def waves_per_simd(res: dict[str, int]) -> int:
    """Waves of this kernel that fit one SIMD's 512 unified vector registers per lane (allocated in blocks of 8;
    at most 8 waves; a SIMD's 800 scalar registers allow 8 waves of up to 100 each, more than 102 leave 7 or fewer)."""
    by_vgpr = 512 // max(8, -(-res["vgpr_count"] // 8) * 8)
    by_sgpr = 800 // max(16, -(-res["sgpr_count"] // 16) * 16)
    return max(1, min(8, by_vgpr, by_sgpr))


def gate(control_hsaco: str | Path, linked_hsaco: str | Path) -> dict[str, Any]:
    """Run the comparison on two code objects.  ``passed`` covers ``GATE_CHECKS``; the ordered
    checks are in ``checks`` for the reader."""
    control = [(n, canonicalize(b)) for n, b in sections(disassemble(control_hsaco))]
    linked = [(n, canonicalize(b)) for n, b in sections(disassemble(linked_hsaco))]
    report = compare_streams(control, linked)
    res = {"control": resources(control_hsaco), "linked": resources(linked_hsaco)}
    report["resources"] = res
    report["checks"]["resources_equal"] = res["control"] == res["linked"]
    # What the footprint decides is how many waves share a SIMD and how many workgroups an LDS: the accumulator block
    # and the LDS must match exactly, the vector registers in the number of waves they leave room for (the allocator
    # of one module may end a few registers below the other's where neither spills).
    report["checks"]["register_footprint_equal"] = (
        all(res["control"][k] == res["linked"][k] for k in ("agpr_count", "group_segment_fixed_size"))
        and waves_per_simd(res["control"]) == waves_per_simd(res["linked"]))
    report["checks"]["spills_small"] = all(r["private_segment_fixed_size"] <= SPILL_LIMIT_BYTES for r in res.values())
    report["opcode_histogram_delta"] = opcode_histogram_delta(control, linked)
    report["bytes_identical"] = Path(control_hsaco).read_bytes() == Path(linked_hsaco).read_bytes()
    report["passed"] = all(report["checks"][c] for c in GATE_CHECKS)
    return report


def summary(report: dict[str, Any]) -> str:
    """The report as the few lines of text a reader wants."""
    lines = [f"gate passed: {report['passed']}   (enforced: {', '.join(GATE_CHECKS)})",
             f"code objects byte-identical: {report['bytes_identical']}", "", "checks:"]
    lines += [f"  {name:55s} {value}" for name, value in report["checks"].items()]
    lines += ["", f"instructions: control {report['instruction_counts']['control']}, linked {report['instruction_counts']['linked']}",
              f"resources control: {report['resources']['control']}", f"resources linked:  {report['resources']['linked']}", "",
              "class counts (control | linked):"]
    for a, b in zip(report["memory_op_class_counts"]["control"], report["memory_op_class_counts"]["linked"]):
        lines.append(f"  {a['function']}")
        lines += [f"    {cls:12s} {a['counts'][cls]:6d} | {b['counts'][cls]:6d}" for cls in CLASSES]
    lines += ["", "opcodes whose counts differ (control, linked):"]
    lines += [f"  {op:28s} {a:6d} {b:6d}" for op, (a, b) in report["opcode_histogram_delta"].items()] or ["  none"]
    return "\n".join(lines) + "\n"


def main(argv: list[str] | None = None) -> int:
    import argparse
    ap = argparse.ArgumentParser(description="compare a linked code object with its one-unit control")
    ap.add_argument("control")
    ap.add_argument("linked")
    args = ap.parse_args(argv)
    report = gate(args.control, args.linked)
    print(summary(report), end="")
    return 0 if report["passed"] else 1


if __name__ == "__main__":
    raise SystemExit(main())
