"""The ISA gate: normalisation and ordered comparison on text, then on the real pair of code
objects (linked image vs one-unit control) of the MoK forward pipeline."""
from pathlib import Path

import pytest

from pipelink_amd.pipec import isagate
from pipelink_amd.stages.mok import build as mok_build

DUMP = """
x.hsaco:	file format elf64-amdgpu

Disassembly of section .text:

0000000000001900 <pipelink_kernel>:
	s_load_dwordx2 s[28:29], s[0:1], 0x0                       // 000000001900: C0060700
	v_mov_b32_e32 v252, v0                                     // 000000001908: 7FF80300
	v_add_u32_e32 v3, 16, v252
	s_cbranch_scc1 6820 <pipelink_kernel+0x1aa4>
	v_mfma_scale_f32_32x32x64_f8f6f4 a[0:15], v[4:11], v[12:19], a[0:15], v3, v252 op_sel_hi:[0,0,0]
	ds_read_b128 v[4:7], v3 offset:32
	s_endpgm
"""


def _renumbered(text: str) -> str:
    # another register allocation of the same program: v252 -> v100, v3 -> v200, s[28:29] -> s[40:41]
    return text.replace("v252", "v100").replace("v3,", "v200,").replace(", v3", ", v200").replace("s[28:29]", "s[40:41]")


def test_sections_drop_addresses_comments_and_branch_targets():
    (name, body), = isagate.sections(DUMP)
    assert name == "pipelink_kernel"
    assert body[0] == "s_load_dwordx2 s[28:29], s[0:1], 0x0"
    assert body[3] == "s_cbranch_scc1 6820 <label>"
    assert len(body) == 7


def test_renaming_is_by_first_use_per_class_and_keeps_range_width():
    (_, body), = isagate.sections(DUMP)
    canon = isagate.canonicalize(body)
    assert canon[0] == "s_load_dwordx2 s<0x2>, s<2x2>, 0x0"
    assert canon[1] == "v_mov_b32_e32 v<0>, v<1>"
    assert canon[2] == "v_add_u32_e32 v<2>, 16, v<0>"
    assert canon[4].startswith("v_mfma_scale_f32_32x32x64_f8f6f4 a<0x16>, v<3x8>, v<11x8>, a<0x16>, v<2>, v<0>")
    assert canon[5] == "ds_read_b128 v<3x4>, v<2> offset:32"


def _stream(text):
    return [(n, isagate.canonicalize(b)) for n, b in isagate.sections(text)]


def test_another_register_allocation_of_the_same_program_passes_every_check():
    report = isagate.compare_streams(_stream(DUMP), _stream(_renumbered(DUMP)))
    assert all(report["checks"].values()), report["checks"]
    assert report["seam_structure_clean"] and report["deltas"] == []


def test_integer_operand_delta_is_enumerated_not_fatal():
    other = DUMP.replace("v_add_u32_e32 v3, 16, v252", "v_add_u32_e32 v3, 48, v252")
    report = isagate.compare_streams(_stream(DUMP), _stream(other))
    assert report["checks"]["all_non_enumerated_instruction_text_equal"]
    (delta,) = report["deltas"]
    assert (delta["old_value"], delta["new_value"], delta["integer_operand_encoding"]) == ("16", "48", True)
    assert delta["instruction_index_zero_based"] == 2 and delta["operand_index_zero_based"] == 1


def test_changed_register_relationship_fails():
    other = DUMP.replace("v_add_u32_e32 v3, 16, v252", "v_add_u32_e32 v3, 16, v0")
    report = isagate.compare_streams(_stream(DUMP), _stream(other))
    assert not report["checks"]["register_relationships_equal_under_frozen_renaming"]
    assert not report["checks"]["all_non_enumerated_instruction_text_equal"]
    assert report["checks"]["opcode_sequence_including_modifiers_equal"]


def test_changed_modifier_fails_the_text_check():
    other = DUMP.replace("offset:32", "offset:48")
    report = isagate.compare_streams(_stream(DUMP), _stream(other))
    assert not report["checks"]["all_non_enumerated_instruction_text_equal"]


def test_calls_and_scratch_are_counted():
    other = DUMP.replace("\ts_endpgm", "\tscratch_store_dword off, v3, off offset:4\n\ts_swappc_b64 s[30:31], s[4:5]\n\ts_endpgm")
    report = isagate.compare_streams(_stream(other), _stream(other))
    counts = report["memory_op_class_counts"]["linked"][0]["counts"]
    assert counts["scratch_"] == 1 and counts["call"] == 1 and counts["v_mfma"] == 1 and counts["ds_"] == 1
    assert not report["checks"]["no_calls"] and not report["checks"]["no_local_traffic"]


@pytest.fixture(scope="module")
def pair(tmp_path_factory):
    out = tmp_path_factory.mktemp("mok_gate")
    mok_build.build(out=out, one_unit=True)
    return out / "one_unit.hsaco", out / "link" / "pipeline.hsaco"


def test_linked_image_passes_the_gate_against_the_one_unit_control(pair):
    control, linked = pair
    report = isagate.gate(control, linked)
    assert report["passed"], isagate.summary(report)
    assert report["checks"]["no_calls"]
    counts = report["memory_op_class_counts"]
    assert counts["control"][0]["counts"]["v_mfma"] == counts["linked"][0]["counts"]["v_mfma"] > 0
    assert report["checks"]["register_footprint_equal"] and report["checks"]["data_path_class_counts_equal"]
    # a handful of spilled dwords at most on either side
    assert max(r["private_segment_fixed_size"] for r in report["resources"].values()) <= isagate.SPILL_LIMIT_BYTES
    text = isagate.summary(report)
    assert "gate passed: True" in text and "v_mfma" in text


def test_link_audit_tells_a_long_branch_from_a_call():
    """An image larger than a branch's reach (+-128 KB) jumps with s_getpc / s_add / s_addc / s_setpc: not a seam call."""
    from pipelink_amd.pipec.linker import seam_calls

    long_branch = ("\ts_cbranch_scc0 6   // 00194C: BF840006 <pipelink_kernel+0x68>\n"
                   "\ts_getpc_b64 s[98:99]                                       // 000000001950: BEE21C00\n"
                   "\ts_add_u32 s98, s98, 0x1ff0c                                // 000000001954: 8062FF62 0001FF0C\n"
                   "\ts_addc_u32 s99, s99, 0                                     // 00000000195C: 8263FF63 00000000\n"
                   "\ts_setpc_b64 s[98:99]                                       // 000000001964: BE801D62\n")
    assert seam_calls(long_branch) == 0
    call = ("\ts_getpc_b64 s[4:5]\n\ts_add_u32 s4, s4, 0x10\n\ts_addc_u32 s5, s5, 0\n\ts_swappc_b64 s[30:31], s[4:5]\n")
    assert seam_calls(call) == 1
    assert seam_calls("\tv_add_f32 v0, v0, v1\n\ts_setpc_b64 s[30:31]\n") == 1                      # a return: somebody was called
    assert seam_calls(long_branch.replace("s_setpc_b64 s[98:99]", "s_setpc_b64 s[30:31]")) == 1  # not the pc it just computed
